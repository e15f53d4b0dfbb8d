// Attention through a shared latent: what lies between the packed projection and the attention kernel, and the
// small products per head on either side of it.
//
// Every token has one latent row c (C entries, normed) and one rotated key part kr (R entries) for all heads; a
// head's plain key is Wuk_h c and its value Wuv_h c.  Since q_h . (Wuk_h c) = (Wuk_h^T q_h) . c, the keys and
// values never have to be formed: the cache holds [c | kr] as the one key row of a token (and c as its value
// row), the query of head h becomes [Wuk_h^T q_plain_h | q_turned_h], the attention runs with one key/value
// head of C + R and C entries, and a head's output is Wuv_h applied to what the attention gives.
//
//   latent_prepare   row = [q (H heads of [D plain | R turned]) | c_raw (C) | kr_raw (R)] of a token:
//                    c = c_raw / sqrt(mean(c_raw^2) + eps) * w;  kr and every head's turned part rotated in pairs of
//                    neighbours (2i, 2i + 1) by the token's row of the step's table (R/2 cosines, then R/2 sines);
//                    cache K <- [c | kr], cache V <- c at the token's slot; q2[t, h, C : C + R] <- the head's turned part.
//                    Sums, scale and rotation float; each output rounded once to the element type.
//   heads_linear     y[t, h, n] = sum_k W[h, n, k] x[t, h, k] for every head by itself, with strides for all three:
//                    the plain parts of q into the latent's space (W read as [h, k, n]) and the attention's output
//                    out of it.  A float sum over k in ascending order per output, rounded once.
#include "common.h"

template <typename T>
__global__ void __launch_bounds__(256)
latent_prepare_kernel(const T* __restrict__ proj, int64_t stride, int heads, int dim, int rot, int rank,
                      const void* __restrict__ weight, int w_is_f32, float eps, const float* __restrict__ rot_table,
                      T* __restrict__ q2, int64_t q2_stride, const int32_t* __restrict__ slots,
                      T* __restrict__ k_cache, T* __restrict__ v_cache, int page_size) {
    __shared__ float scratch[16];
    const int64_t t = blockIdx.x;
    const int tid = threadIdx.x;
    const T* row = proj + t * stride;
    const int qd = heads * (dim + rot);
    const int slot = slots ? slots[t] : -1;
    const float* rot_row = rot_table + t * (int64_t)rot;
    const int half = rot / 2;
    // a turned entry d of a part that starts at `at` in the row
    auto turned = [&](int at, int d) -> float {
        const float x = to_float(row[at + d]), y = to_float(row[at + (d ^ 1)]);
        const float c = rot_row[d >> 1], sn = rot_row[half + (d >> 1)];
        return (d & 1) ? x * c + y * sn : x * c - y * sn;
    };
    for (int i = tid; i < heads * rot; i += blockDim.x) {
        const int h = i / rot, d = i % rot;
        q2[t * q2_stride + (int64_t)h * (rank + rot) + rank + d] = from_float<T>(turned(h * (dim + rot) + dim, d));
    }
    float ss = 0.f;
    for (int i = tid; i < rank; i += blockDim.x) {
        const float x = to_float(row[qd + i]);
        ss += x * x;
    }
    ss = block_sum(ss, scratch);
    if (slot < 0 || !k_cache) return;
    const float scale = rsqrtf(ss / (float)rank + eps);
    const int page = slot / page_size, off = slot % page_size;
    const int vt = nva_v_tile(page_size);
    T* krow = k_cache + ((int64_t)page * page_size + off) * (rank + rot);
    T* vpage = v_cache + (int64_t)page * rank * page_size;
    for (int i = tid; i < rank; i += blockDim.x) {
        const float w = w_is_f32 ? static_cast<const float*>(weight)[i] : to_float(static_cast<const T*>(weight)[i]);
        const T c = from_float<T>(to_float(row[qd + i]) * scale * w);
        krow[i] = c;
        vpage[nva_v_offset(off, i, rank, vt)] = c;
    }
    for (int d = tid; d < rot; d += blockDim.x) krow[rank + d] = from_float<T>(turned(qd + rank, d));
}

// proj [tokens, H * (D + R) + C + R] elements, rows `stride` apart; weight [C] (float or elements); rot_table float
// [tokens, R]; q2 [tokens, H * (C + R)] rows q2_stride apart; K cache [pages, 1, page, C + R], V cache
// [pages, 1, page / vt, C, vt]; slots may be null with the caches (nothing is stored then).
NVA_EXPORT int NVA_NAME(nva_latent_prepare)(const void* proj, int64_t stride, int64_t tokens, int heads, int dim, int rot,
                                            int rank, const void* weight, int w_is_f32, float eps, const float* rot_table,
                                            void* q2, int64_t q2_stride, const int32_t* slots, void* k_cache,
                                            void* v_cache, int page_size, hipStream_t stream) {
    if (tokens == 0) return 0;
    if (tokens < 0 || tokens > 0x7fffffff) return nva_fail("latent_prepare: bad token count %lld", (long long)tokens);
    if (heads <= 0 || dim <= 0 || rot <= 0 || rot % 2 || rank <= 0)
        return nva_fail("latent_prepare: bad sizes heads=%d dim=%d rot=%d rank=%d", heads, dim, rot, rank);
    if (!proj || !weight || !rot_table || !q2 || stride < (int64_t)heads * (dim + rot) + rank + rot ||
        q2_stride < (int64_t)heads * (rank + rot))
        return nva_fail("latent_prepare: a tensor is missing or too narrow");
    if ((k_cache || v_cache) && (!k_cache || !v_cache || !slots || page_size <= 0))
        return nva_fail("latent_prepare: storing needs both caches, the slots and the page size");
    hipLaunchKernelGGL(latent_prepare_kernel<elem_t>, dim3((unsigned)tokens), dim3(256), 0, stream, (const elem_t*)proj,
                       stride, heads, dim, rot, rank, weight, w_is_f32, eps, rot_table, (elem_t*)q2, q2_stride, slots,
                       (elem_t*)k_cache, (elem_t*)v_cache, page_size);
    return nva_check_launch("latent_prepare");
}

#define HL_TOKENS 16        // tokens of a workgroup
#define HL_MAX_K 1024

// A workgroup of four waves: 16 tokens of one head and 64 outputs; a lane an output, a wave four of the tokens.
template <typename T>
__global__ void __launch_bounds__(256)
heads_linear_kernel(const T* __restrict__ x, int64_t x_stride, int64_t x_head, const T* __restrict__ w, int64_t w_head,
                    int64_t w_n, int64_t w_k, T* __restrict__ y, int64_t y_stride, int64_t y_head, int64_t tokens,
                    int n_out, int k_in) {
    extern __shared__ __attribute__((aligned(16))) float x_s[];       // [HL_TOKENS][k_in]
    const int64_t t0 = (int64_t)blockIdx.x * HL_TOKENS;
    const int h = blockIdx.y;
    const int tid = threadIdx.x, lane = tid % NVA_WAVE, wave = tid / NVA_WAVE;
    for (int i = tid; i < HL_TOKENS * k_in; i += blockDim.x) {
        const int r = i / k_in, k = i % k_in;
        x_s[i] = t0 + r < tokens ? to_float(x[(t0 + r) * x_stride + h * x_head + k]) : 0.f;
    }
    __syncthreads();
    const int n = blockIdx.z * NVA_WAVE + lane;
    if (n >= n_out) return;
    const T* wn = w + h * w_head + n * w_n;
    const float* xr = x_s + (wave * 4) * k_in;
    float acc[4] = {0.f, 0.f, 0.f, 0.f};
    int k = 0;
    for (; k + 4 <= k_in; k += 4) {
        float ww[4];
#pragma unroll
        for (int u = 0; u < 4; ++u) ww[u] = to_float(wn[(k + u) * w_k]);
#pragma unroll
        for (int u = 0; u < 4; ++u)
#pragma unroll
            for (int r = 0; r < 4; ++r) acc[r] += ww[u] * xr[r * k_in + k + u];
    }
    for (; k < k_in; ++k) {
        const float ww = to_float(wn[k * w_k]);
#pragma unroll
        for (int r = 0; r < 4; ++r) acc[r] += ww * xr[r * k_in + k];
    }
#pragma unroll
    for (int r = 0; r < 4; ++r) {
        const int64_t t = t0 + wave * 4 + r;
        if (t < tokens) y[t * y_stride + h * y_head + n] = from_float<T>(acc[r]);
    }
}

// x: head h of token t starts at x + t * x_stride + h * x_head (k_in entries side by side); w: W[h, n, k] at
// w + h * w_head + n * w_n + k * w_k; y: head h of token t at y + t * y_stride + h * y_head (n_out entries).
NVA_EXPORT int NVA_NAME(nva_heads_linear)(const void* x, int64_t x_stride, int64_t x_head, const void* w, int64_t w_head,
                                          int64_t w_n, int64_t w_k, void* y, int64_t y_stride, int64_t y_head,
                                          int64_t tokens, int heads, int n_out, int k_in, hipStream_t stream) {
    if (tokens == 0) return 0;
    if (tokens < 0 || tokens > 0x7fffffff || heads <= 0 || heads > 65535 || n_out <= 0 || k_in <= 0 || k_in > HL_MAX_K)
        return nva_fail("heads_linear: bad sizes tokens=%lld heads=%d outputs=%d inputs=%d (up to %d)", (long long)tokens,
                        heads, n_out, k_in, HL_MAX_K);
    if (!x || !w || !y) return nva_fail("heads_linear: a tensor is missing");
    auto kernel = heads_linear_kernel<elem_t>;
    const size_t lds = (size_t)HL_TOKENS * k_in * sizeof(float);
    static bool raised = false;
    if (!raised && lds > 48 * 1024) {
        if (hipFuncSetAttribute((const void*)kernel, hipFuncAttributeMaxDynamicSharedMemorySize, HL_TOKENS * HL_MAX_K * 4) != hipSuccess)
            return nva_fail("heads_linear: cannot have %zu bytes of LDS", lds);
        raised = true;
    }
    const int64_t groups = (tokens + HL_TOKENS - 1) / HL_TOKENS;
    dim3 grid((unsigned)groups, (unsigned)heads, (unsigned)((n_out + NVA_WAVE - 1) / NVA_WAVE));
    hipLaunchKernelGGL(kernel, grid, dim3(256), lds, stream, (const elem_t*)x, x_stride, x_head, (const elem_t*)w, w_head,
                       w_n, w_k, (elem_t*)y, y_stride, y_head, tokens, n_out, k_in);
    return nva_check_launch("heads_linear");
}

NVA_DEFINE_LAST_ERROR(nva_latent)
