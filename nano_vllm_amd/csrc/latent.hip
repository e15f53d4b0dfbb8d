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

#if defined(NVA_BF16)
// ---------------------------------------------------------------------------- the product per head on the matrix cores
// W [heads, n_out, k_in] with k side by side.  A wave takes 16 tokens of one head and 64 outputs: the rows of W are the
// A operand and the tokens' rows the B operand of v_mfma_f32_16x16x32_bf16, both straight from global memory (a lane 16
// bytes a load); a fragment of x serves four products.  The sum over k runs in the order of the steps of 32, whatever
// the other tokens of the tile.
typedef __attribute__((ext_vector_type(8))) __bf16 hl_bf16x8;
typedef __attribute__((ext_vector_type(4))) float hl_f32x4;

__global__ void __launch_bounds__(NVA_WAVE)
heads_linear_mfma_kernel(const __bf16* __restrict__ x, int64_t x_stride, int64_t x_head, const __bf16* __restrict__ w,
                         __bf16* __restrict__ y, int64_t y_stride, int64_t y_head, int64_t tokens, int n_out, int k_in) {
    const int64_t t0 = (int64_t)blockIdx.x * 16;
    const int h = blockIdx.y, n0 = blockIdx.z * 64;
    const int lane = threadIdx.x, col = lane & 15, g = lane >> 4;
    const int64_t t = t0 + col;
    const __bf16* xr = x + (t < tokens ? t : tokens - 1) * x_stride + h * x_head + 8 * g;
    const __bf16* wr[4];
#pragma unroll
    for (int b = 0; b < 4; ++b) wr[b] = w + ((int64_t)h * n_out + min(n0 + 16 * b + col, n_out - 1)) * k_in + 8 * g;
    hl_f32x4 acc[4];
#pragma unroll
    for (int b = 0; b < 4; ++b) acc[b] = hl_f32x4{0.f, 0.f, 0.f, 0.f};
    const int k_last = k_in - 8;                    // k_in is a multiple of 8: a piece lies inside the row or outside
#pragma unroll 4
    for (int k0 = 0; k0 < k_in; k0 += 32) {
        const bool inside = k0 + 8 * g <= k_last;
        const int at = inside ? k0 : -8 * g;        // (every load unconditional: a piece outside the row reads the row's first, and counts as zero)
        hl_bf16x8 xf = *reinterpret_cast<const hl_bf16x8*>(xr + at);
        hl_bf16x8 wf[4];
#pragma unroll
        for (int b = 0; b < 4; ++b) wf[b] = *reinterpret_cast<const hl_bf16x8*>(wr[b] + at);
        if (!inside) {
#pragma unroll
            for (int e = 0; e < 8; ++e) xf[e] = (__bf16)0.f;
        }
#pragma unroll
        for (int b = 0; b < 4; ++b) acc[b] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wf[b], xf, acc[b], 0, 0, 0);
    }
    // acc[b][i] = y[token col][n0 + 16 b + 4 g + i]
    if (t >= tokens) return;
    __bf16* yr = y + t * y_stride + h * y_head;
#pragma unroll
    for (int b = 0; b < 4; ++b)
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int n = n0 + 16 * b + 4 * g + i;
            if (n < n_out) yr[n] = (__bf16)acc[b][i];
        }
}

// As nva_heads_linear with w_n = k_in, w_k = 1 (W [heads * n_out, k_in], contiguous).  Returns 1 (and a message) for
// shapes it does not take: k_in a multiple of 8, x rows and heads at multiples of 8 elements, 16-byte aligned pointers.
NVA_EXPORT int nva_heads_linear_mfma_bf16(const void* x, int64_t x_stride, int64_t x_head, const void* w, void* y,
                                          int64_t y_stride, int64_t y_head, int64_t tokens, int heads, int n_out, int k_in,
                                          hipStream_t stream) {
    if (tokens == 0) return 0;
    if (k_in % 8 || k_in <= 0 || x_stride % 8 || x_head % 8 || !nva_aligned(x, 16) || !nva_aligned(w, 16)) {
        nva_fail("heads_linear_mfma: rows that are not aligned for 16-byte loads (k_in %d)", k_in);
        return 1;
    }
    if (tokens < 0 || tokens > 0x7fffffffLL * 16 || heads <= 0 || heads > 65535 || n_out <= 0 || (n_out + 63) / 64 > 65535 ||
        !x || !w || !y)
        return nva_fail("heads_linear_mfma: bad sizes tokens=%lld heads=%d outputs=%d", (long long)tokens, heads, n_out);
    dim3 grid((unsigned)((tokens + 15) / 16), (unsigned)heads, (unsigned)((n_out + 63) / 64));
    hipLaunchKernelGGL(heads_linear_mfma_kernel, grid, dim3(NVA_WAVE), 0, stream, (const __bf16*)x, x_stride, x_head,
                       (const __bf16*)w, (__bf16*)y, y_stride, y_head, tokens, n_out, k_in);
    return nva_check_launch("heads_linear_mfma");
}

// ---------------------------------------------------------------------------- the attention itself, on the matrix cores
// One key/value head for all query heads: the query heads of a token are the 16 columns of the products, so a key row
// that is fetched serves all of them.  A wave takes one token, 16 of its heads and a share of its keys, in tiles of 32:
//     S^T = K Q^T      K rows straight from the cache as the A operand (a lane 16 bytes of a key row), Q^T in registers
//     O^T += V^T P^T   V^T from the value cache, which holds the latent transposed in tiles of 32 keys (a lane 2 x 8
//                      bytes of a channel's row), P^T as the lanes hold it after the first product: the second
//                      product's index over the keys is 8 g + j <-> key 4 g + j (j < 4) and 16 + 4 g + j - 4 (j >= 4)
//                      of the tile, for both operands, so that nothing is exchanged between lanes
// with an online softmax in float (exp2 with log2 e folded in), the sink as the first share's starting maximum with a
// sum of one.  All tokens are treated alike, a prompt's and single ones (every row of a tile has the same position, so
// only a token's last tile is masked).  With more than one share the shares leave (maximum, sum, unnormalised output)
// and latent_attn_merge_kernel joins them in the order of the shares.
typedef __attribute__((ext_vector_type(8))) __bf16 lat_bf16x8;
typedef __attribute__((ext_vector_type(4))) __bf16 lat_bf16x4;
typedef __attribute__((ext_vector_type(4))) float lat_f32x4;
#define LAT_TILE 32
#define LAT_MAX_ROT 128

template <int MAXC>
__global__ void __launch_bounds__(NVA_WAVE)
latent_attn_kernel(const __bf16* __restrict__ q2, int64_t q_stride, __bf16* __restrict__ out, int64_t out_stride,
                   float* __restrict__ part, const __bf16* __restrict__ k_cache, const __bf16* __restrict__ v_cache,
                   const int32_t* __restrict__ block_tables, int table_stride, const int32_t* __restrict__ token_seq,
                   const int32_t* __restrict__ positions, int heads, int rank, int rot, int page_size, float scale,
                   const float* __restrict__ sinks, int32_t* error_flag) {
    constexpr int KS = (MAXC + LAT_MAX_ROT) / 32;      // steps of 32 channels of the first product, at most
    constexpr int CB = MAXC / 16;                      // blocks of 16 latent channels of the output, at most
    // (the step's last tokens first: in a prompt's portion they have the most keys, and the workgroups that start first
    // should be the long ones)
    const int64_t t = (int64_t)gridDim.x - 1 - blockIdx.x;
    const int share = blockIdx.y, shares = gridDim.y;
    const int lane = threadIdx.x, col = lane & 15, g = lane >> 4;
    const int head = blockIdx.z * 16 + col;
    const bool head_ok = head < heads;
    const int width = rank + rot;                      // a key row
    const int steps = (width + 31) / 32, blocks = rank / 16;
    const int pos = positions[t];
    const int32_t* table = block_tables + (int64_t)token_seq[t] * table_stride;
    const int tiles = pos / LAT_TILE + 1;
    const int per = (tiles + shares - 1) / shares;
    const int tile_lo = share * per, tile_hi = min(tiles, tile_lo + per);

    lat_bf16x8 qf[KS];
    const __bf16* qrow = q2 + t * q_stride + (int64_t)(head_ok ? head : 0) * width;
#pragma unroll
    for (int c = 0; c < KS; ++c) {
#pragma unroll
        for (int e = 0; e < 8; ++e) qf[c][e] = (__bf16)0.f;
        if (c < steps && head_ok && 32 * c + 8 * g < width) qf[c] = *reinterpret_cast<const lat_bf16x8*>(qrow + 32 * c + 8 * g);
    }
    lat_f32x4 acc[CB];
#pragma unroll
    for (int b = 0; b < CB; ++b) acc[b] = lat_f32x4{0.f, 0.f, 0.f, 0.f};
    const bool with_sink = sinks && share == 0 && head_ok;
    float m_run = with_sink ? sinks[head] : -INFINITY, l_run = with_sink ? 1.f : 0.f;      // of the scaled scores
    const float log2e = 1.4426950408889634f;
    const int tiles_per_page = page_size / LAT_TILE;

    for (int tile = tile_lo; tile < tile_hi; ++tile) {
        const int kb = tile * LAT_TILE;
        int page = table[kb / page_size];
        const bool no_page = page < 0;
        if (no_page) {
            if (error_flag && lane == 0) atomicOr(error_flag, 2);        // a visible key has no page
            page = 0;
        }
        const int in_page = kb % page_size;
        // ---- scores: rows of K as they lie, keys kb + col and kb + 16 + col
        const __bf16* k0 = k_cache + ((int64_t)page * page_size + in_page + col) * width + 8 * g;
        const __bf16* k1 = k0 + (int64_t)16 * width;
        // (all of the tile's loads are asked for before anything is used: a wave is alone on its SIMD, and what it has
        // on its way is all that hides the memory's latency)
        const __bf16* v0 = v_cache + (((int64_t)page * tiles_per_page + in_page / LAT_TILE) * rank + col) * LAT_TILE + 4 * g;
        lat_bf16x8 ka[KS], kc[KS];
        lat_bf16x4 vlo[CB], vhi[CB];
#pragma unroll
        for (int c = 0; c < KS; ++c) {
#pragma unroll
            for (int e = 0; e < 8; ++e) ka[c][e] = kc[c][e] = (__bf16)0.f;
            if (c < steps && 32 * c + 8 * g < width) {
                ka[c] = *reinterpret_cast<const lat_bf16x8*>(k0 + 32 * c);
                kc[c] = *reinterpret_cast<const lat_bf16x8*>(k1 + 32 * c);
            }
        }
#pragma unroll
        for (int b = 0; b < CB; ++b)
            if (b < blocks) {
                vlo[b] = *reinterpret_cast<const lat_bf16x4*>(v0 + (int64_t)b * 16 * LAT_TILE);
                vhi[b] = *reinterpret_cast<const lat_bf16x4*>(v0 + (int64_t)b * 16 * LAT_TILE + 16);
            }
        lat_f32x4 sa = {0.f, 0.f, 0.f, 0.f}, sb = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int c = 0; c < KS; ++c) {
            if (c < steps) {
                sa = __builtin_amdgcn_mfma_f32_16x16x32_bf16(ka[c], qf[c], sa, 0, 0, 0);
                sb = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kc[c], qf[c], sb, 0, 0, 0);
            }
        }
        // this lane: head `col`, keys kb + 4 g + i (sa) and kb + 16 + 4 g + i (sb)
        float s[8];
        float m_new = m_run;
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            const int key = kb + (i < 4 ? 4 * g + i : 16 + 4 * g + i - 4);
            const float raw = (i < 4 ? sa[i] : sb[i - 4]) * scale;
            s[i] = key <= pos && !no_page ? raw : -INFINITY;
            m_new = fmaxf(m_new, s[i]);
        }
        m_new = nva_max_over_rows(m_new);
        const float m_use = fmaxf(m_new, -1e30f);
        lat_bf16x8 pf;
        float psum = 0.f;
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            const __bf16 p = (__bf16)__builtin_amdgcn_exp2f((s[i] - m_use) * log2e);
            pf[i] = p;
            psum += (float)p;              // the sum of what the product below really uses
        }
        psum = nva_sum_over_rows(psum);
        const float alpha = __builtin_amdgcn_exp2f((fmaxf(m_run, -1e30f) - m_use) * log2e);
        l_run = l_run * alpha + psum;
        m_run = m_new;
        // ---- O^T += V^T P^T: channel 16 b + col, keys kb + 4 g .. + 3 and kb + 16 + 4 g .. + 3
        const bool whole = kb + LAT_TILE - 1 <= pos && !no_page;
#pragma unroll
        for (int b = 0; b < CB; ++b) {
            if (b < blocks) {
                lat_bf16x8 vf;
#pragma unroll
                for (int e = 0; e < 4; ++e) vf[e] = vlo[b][e], vf[4 + e] = vhi[b][e];
                if (!whole) {              // what the cache holds beyond the token's own key may be anything
#pragma unroll
                    for (int e = 0; e < 8; ++e)
                        if (no_page || kb + (e < 4 ? 4 * g + e : 16 + 4 * g + e - 4) > pos) vf[e] = (__bf16)0.f;
                }
                lat_f32x4 a = acc[b];
                a[0] *= alpha; a[1] *= alpha; a[2] *= alpha; a[3] *= alpha;
                acc[b] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vf, pf, a, 0, 0, 0);
            }
        }
    }
    // acc[b][i] = O[head col][channel 16 b + 4 g + i]
    if (!head_ok) return;
    if (shares == 1) {
        const float inv = l_run > 0.f ? 1.f / l_run : 0.f;
        __bf16* orow = out + t * out_stride + (int64_t)head * rank;
#pragma unroll
        for (int b = 0; b < CB; ++b)
            if (b < blocks) {
                lat_bf16x4 v;
#pragma unroll
                for (int i = 0; i < 4; ++i) v[i] = (__bf16)(acc[b][i] * inv);
                *reinterpret_cast<lat_bf16x4*>(orow + 16 * b + 4 * g) = v;
            }
        return;
    }
    float* mine = part + ((t * heads + head) * shares + share) * (int64_t)(2 + rank);
    if (g == 0) mine[0] = m_run, mine[1] = l_run;
#pragma unroll
    for (int b = 0; b < CB; ++b)
        if (b < blocks) {
#pragma unroll
            for (int i = 0; i < 4; ++i) mine[2 + 16 * b + 4 * g + i] = acc[b][i];
        }
}

// The same attention for portions of prompts: a workgroup of WAVES waves (eight, or four where a latent of more than
// 384 channels leaves a SIMD's registers to one wave) takes as many tokens in a row of one request (a part of a row tile
// of 32 queries; tiles as for the other prefill kernels, most keys first), a wave one token.  The tiles of keys and of
// transposed values, which the tokens share, go through LDS once for all of them:
// the next tile is asked for (into registers) before the products of the tile at hand and stored after them.  The
// arithmetic of a token is that of latent_attn_kernel with one share, operation for operation.
template <int MAXC, int WAVES>
__global__ void __launch_bounds__(WAVES * NVA_WAVE)
latent_attn_quad_kernel(const __bf16* __restrict__ q2, int64_t q_stride, __bf16* __restrict__ out, int64_t out_stride,
                        const __bf16* __restrict__ k_cache, const __bf16* __restrict__ v_cache,
                        const int32_t* __restrict__ block_tables, int table_stride, const int32_t* __restrict__ cu_seqlens_q,
                        const int32_t* __restrict__ kv_lens, const int32_t* __restrict__ row_tiles, int heads, int rank, int rot,
                        int page_size, float scale, const float* __restrict__ sinks, int32_t* error_flag) {
    constexpr int KS = (MAXC + LAT_MAX_ROT) / 32, CB = MAXC / 16;
    constexpr int THREADS = WAVES * NVA_WAVE, PER_TILE = 32 / WAVES;   // tokens of a workgroup: WAVES; workgroups of a row tile
    constexpr int KP = (4 * (MAXC + LAT_MAX_ROT) + THREADS - 1) / THREADS, VP = (4 * MAXC + THREADS - 1) / THREADS;   // 16-byte pieces of a tile a thread moves, at most
    extern __shared__ __attribute__((aligned(16))) __bf16 lat_s[];
    const int width = rank + rot, KSTR = width + 8, VSTR = LAT_TILE + 4;
    __bf16* const k_s = lat_s;                          // [32 keys][KSTR]
    __bf16* const v_s = lat_s + LAT_TILE * KSTR;        // [rank channels][VSTR]
    const int ti = blockIdx.x / PER_TILE, quad = blockIdx.x % PER_TILE;
    const int seq = row_tiles[2 * ti], row_tile = row_tiles[2 * ti + 1];
    const int q_begin = cu_seqlens_q[seq];
    const int q_len = cu_seqlens_q[seq + 1] - q_begin;
    const int start = kv_lens[seq] - q_len;             // position of the request's first query of this step
    const int row0 = row_tile * 32 + quad * WAVES;
    if (row0 >= q_len) return;                          // (the whole workgroup)
    const int tid = threadIdx.x, wave = tid / NVA_WAVE, lane = tid % NVA_WAVE, col = lane & 15, g = lane >> 4;
    const int row = row0 + wave;
    const bool token_ok = row < q_len;
    const int pos = token_ok ? start + row : -1;
    const int64_t t = q_begin + (token_ok ? row : row0);
    const int tiles = (start + min(row0 + WAVES - 1, q_len - 1)) / LAT_TILE + 1;
    const int head = blockIdx.z * 16 + col;
    const bool head_ok = head < heads;
    const int steps = (width + 31) / 32, blocks = rank / 16;
    const int32_t* table = block_tables + (int64_t)seq * table_stride;
    const int tiles_per_page = page_size / LAT_TILE;
    const int k_pieces = 4 * width, v_pieces = 4 * rank;

    lat_bf16x8 qf[KS];
    const __bf16* qrow = q2 + t * q_stride + (int64_t)(head_ok ? head : 0) * width;
#pragma unroll
    for (int c = 0; c < KS; ++c) {
#pragma unroll
        for (int e = 0; e < 8; ++e) qf[c][e] = (__bf16)0.f;
        if (c < steps && head_ok && token_ok && 32 * c + 8 * g < width) qf[c] = *reinterpret_cast<const lat_bf16x8*>(qrow + 32 * c + 8 * g);
    }
    lat_f32x4 acc[CB];
#pragma unroll
    for (int b = 0; b < CB; ++b) acc[b] = lat_f32x4{0.f, 0.f, 0.f, 0.f};
    const bool with_sink = sinks && head_ok;
    float m_run = with_sink ? sinks[head] : -INFINITY, l_run = with_sink ? 1.f : 0.f;
    const float log2e = 1.4426950408889634f;

    lat_bf16x8 kreg[KP], vreg[VP];
    bool no_page = false, no_page_next = false;
    auto ask = [&](int tile) __attribute__((always_inline)) {       // a tile's keys and values, as they lie in the cache, into registers
        const int kb = tile * LAT_TILE;
        int page = table[kb / page_size];
        no_page_next = page < 0;
        if (no_page_next) {
            if (error_flag && tid == 0) atomicOr(error_flag, 2);    // a visible key has no page
            page = 0;
        }
        const int in_page = kb % page_size;
        const __bf16* kbase = k_cache + ((int64_t)page * page_size + in_page) * width;
        const __bf16* vbase = v_cache + ((int64_t)page * tiles_per_page + in_page / LAT_TILE) * rank * LAT_TILE;
#pragma unroll
        for (int i = 0; i < KP; ++i) {
            const int p = tid + THREADS * i;
            if (p < k_pieces) kreg[i] = *reinterpret_cast<const lat_bf16x8*>(kbase + (int64_t)p * 8);
        }
#pragma unroll
        for (int i = 0; i < VP; ++i) {
            const int p = tid + THREADS * i;
            if (p < v_pieces) vreg[i] = *reinterpret_cast<const lat_bf16x8*>(vbase + (int64_t)p * 8);
        }
    };
    auto put = [&]() __attribute__((always_inline)) {
        const int per_key = width / 8;
#pragma unroll
        for (int i = 0; i < KP; ++i) {
            const int p = tid + THREADS * i;
            if (p < k_pieces) *reinterpret_cast<lat_bf16x8*>(&k_s[(p / per_key) * KSTR + (p % per_key) * 8]) = kreg[i];
        }
#pragma unroll
        for (int i = 0; i < VP; ++i) {
            const int p = tid + THREADS * i;
            if (p < v_pieces) {
                // (rows of 36 elements: two 8-byte stores)
                lat_bf16x4 lo, hi;
#pragma unroll
                for (int e = 0; e < 4; ++e) lo[e] = vreg[i][e], hi[e] = vreg[i][4 + e];
                __bf16* dst = &v_s[(p / 4) * VSTR + (p % 4) * 8];
                *reinterpret_cast<lat_bf16x4*>(dst) = lo;
                *reinterpret_cast<lat_bf16x4*>(dst + 4) = hi;
            }
        }
    };
    ask(0);
    for (int tile = 0; tile < tiles; ++tile) {
        const int kb = tile * LAT_TILE;
        put();
        no_page = no_page_next;
        __syncthreads();
        if (tile + 1 < tiles) ask(tile + 1);
        if (kb <= pos) {                                    // (the same for the whole wave)
            lat_f32x4 sa = {0.f, 0.f, 0.f, 0.f}, sb = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int c = 0; c < KS; ++c) {
                if (c < steps) {
                    lat_bf16x8 ka, kc;
#pragma unroll
                    for (int e = 0; e < 8; ++e) ka[e] = kc[e] = (__bf16)0.f;
                    if (32 * c + 8 * g < width) {
                        ka = *reinterpret_cast<const lat_bf16x8*>(&k_s[col * KSTR + 32 * c + 8 * g]);
                        kc = *reinterpret_cast<const lat_bf16x8*>(&k_s[(16 + col) * KSTR + 32 * c + 8 * g]);
                    }
                    sa = __builtin_amdgcn_mfma_f32_16x16x32_bf16(ka, qf[c], sa, 0, 0, 0);
                    sb = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kc, qf[c], sb, 0, 0, 0);
                }
            }
            float s[8];
            float m_new = m_run;
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                const int key = kb + (i < 4 ? 4 * g + i : 16 + 4 * g + i - 4);
                const float raw = (i < 4 ? sa[i] : sb[i - 4]) * scale;
                s[i] = key <= pos && !no_page ? raw : -INFINITY;
                m_new = fmaxf(m_new, s[i]);
            }
            m_new = nva_max_over_rows(m_new);
            const float m_use = fmaxf(m_new, -1e30f);
            lat_bf16x8 pf;
            float psum = 0.f;
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                const __bf16 p = (__bf16)__builtin_amdgcn_exp2f((s[i] - m_use) * log2e);
                pf[i] = p;
                psum += (float)p;
            }
            psum = nva_sum_over_rows(psum);
            const float alpha = __builtin_amdgcn_exp2f((fmaxf(m_run, -1e30f) - m_use) * log2e);
            l_run = l_run * alpha + psum;
            m_run = m_new;
            const bool whole = kb + LAT_TILE - 1 <= pos && !no_page;
#pragma unroll
            for (int b = 0; b < CB; ++b) {
                if (b < blocks) {
                    const lat_bf16x4 lo = *reinterpret_cast<const lat_bf16x4*>(&v_s[(16 * b + col) * VSTR + 4 * g]);
                    const lat_bf16x4 hi = *reinterpret_cast<const lat_bf16x4*>(&v_s[(16 * b + col) * VSTR + 16 + 4 * g]);
                    lat_bf16x8 vf;
#pragma unroll
                    for (int e = 0; e < 4; ++e) vf[e] = lo[e], vf[4 + e] = hi[e];
                    if (!whole) {
#pragma unroll
                        for (int e = 0; e < 8; ++e)
                            if (no_page || kb + (e < 4 ? 4 * g + e : 16 + 4 * g + e - 4) > pos) vf[e] = (__bf16)0.f;
                    }
                    lat_f32x4 a = acc[b];
                    a[0] *= alpha; a[1] *= alpha; a[2] *= alpha; a[3] *= alpha;
                    acc[b] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vf, pf, a, 0, 0, 0);
                }
            }
        }
        __syncthreads();                                    // all have read the tile: the next may be stored
    }
    if (!head_ok || !token_ok) return;
    const float inv = l_run > 0.f ? 1.f / l_run : 0.f;
    __bf16* orow = out + t * out_stride + (int64_t)head * rank;
#pragma unroll
    for (int b = 0; b < CB; ++b)
        if (b < blocks) {
            lat_bf16x4 v;
#pragma unroll
            for (int i = 0; i < 4; ++i) v[i] = (__bf16)(acc[b][i] * inv);
            *reinterpret_cast<lat_bf16x4*>(orow + 16 * b + 4 * g) = v;
        }
}

// One wave per (token, head, 128 channels): the shares' results joined, in the order of the shares.
__global__ void __launch_bounds__(NVA_WAVE)
latent_attn_merge_kernel(const float* __restrict__ part, int shares, __bf16* __restrict__ out, int64_t out_stride,
                         int heads, int rank) {
    const int64_t t = blockIdx.x;
    const int h = blockIdx.y, lane = threadIdx.x;
    const float* mine = part + (t * heads + h) * shares * (int64_t)(2 + rank);
    float m = -INFINITY;
    for (int s = 0; s < shares; ++s) m = fmaxf(m, mine[s * (int64_t)(2 + rank)]);
    float l = 0.f;
    float acc[2] = {0.f, 0.f};
    const int d0 = blockIdx.z * 2 * NVA_WAVE + lane;                 // this lane's channels: d0 and d0 + 64
    // (four shares at a time, their loads unconditional: a share without keys has weight zero)
    for (int s0 = 0; s0 < shares; s0 += 4) {
        float f[4], ls[4], v[4][2];
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const float* p = mine + min(s0 + j, shares - 1) * (int64_t)(2 + rank);
            const float ms = p[0];
            ls[j] = p[1];
            f[j] = (s0 + j >= shares || ms == -INFINITY) ? 0.f : __expf(ms - m);
#pragma unroll
            for (int i = 0; i < 2; ++i) v[j][i] = d0 + i * NVA_WAVE < rank ? p[2 + d0 + i * NVA_WAVE] : 0.f;
        }
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            l += ls[j] * f[j];
            acc[0] += v[j][0] * f[j];
            acc[1] += v[j][1] * f[j];
        }
    }
    const float inv = l > 0.f ? 1.f / l : 0.f;
    __bf16* orow = out + t * out_stride + (int64_t)h * rank;
#pragma unroll
    for (int i = 0; i < 2; ++i) {
        const int d = d0 + i * NVA_WAVE;
        if (d < rank) orow[d] = (__bf16)(acc[i] * inv);
    }
}

// q2 [tokens, heads * (rank + rot)], out [tokens, heads * rank]; K cache [pages, 1, page, rank + rot], V cache
// [pages, 1, page / 32, rank, 32]; part: float [tokens * heads * shares * (2 + rank)] where shares > 1.
// Returns 1 (and a message) for sizes it does not take: the caller runs the general kernel then.
NVA_EXPORT int nva_latent_attention_bf16(const void* q2, int64_t q_stride, void* out, int64_t out_stride, float* part,
                                         int shares, const void* k_cache, const void* v_cache,
                                         const int32_t* block_tables, int table_stride, const int32_t* token_seq,
                                         const int32_t* positions, int64_t tokens, int heads, int rank, int rot,
                                         int page_size, float scale, const float* sinks, int32_t* error_flag,
                                         hipStream_t stream) {
    if (tokens == 0) return 0;
    if (rank % 16 || rank <= 0 || rank > 512 || rot % 8 || rot <= 0 || rot > LAT_MAX_ROT || page_size % LAT_TILE || page_size <= 0) {
        nva_fail("latent_attention: needs a latent of a multiple of 16 up to 512, a rotated part of a multiple of 8 up to %d and "
                 "pages of a multiple of %d keys (got %d, %d, %d)", LAT_MAX_ROT, LAT_TILE, rank, rot, page_size);
        return 1;
    }
    if (tokens < 0 || tokens > 0x7fffffff || heads <= 0 || shares < 1 || shares > 65535 || (shares > 1 && !part) ||
        table_stride <= 0 || !(scale > 0.f))
        return nva_fail("latent_attention: bad sizes tokens=%lld heads=%d shares=%d", (long long)tokens, heads, shares);
    if (q_stride % 8 || out_stride % 4 || !nva_aligned(q2, 16) || !nva_aligned(out, 8) || !nva_aligned(k_cache, 16) ||
        !nva_aligned(v_cache, 8)) {
        nva_fail("latent_attention: rows that are not aligned for vector access");
        return 1;
    }
    dim3 grid((unsigned)tokens, (unsigned)shares, (unsigned)((heads + 15) / 16));
#define LAT_LAUNCH(MC)                                                                                               \
    hipLaunchKernelGGL(latent_attn_kernel<MC>, grid, dim3(NVA_WAVE), 0, stream, (const __bf16*)q2, q_stride,            \
                       (__bf16*)out, out_stride, part, (const __bf16*)k_cache, (const __bf16*)v_cache, block_tables,     \
                       table_stride, token_seq, positions, heads, rank, rot, page_size, scale, sinks, error_flag)
    if (rank <= 128) LAT_LAUNCH(128);
    else if (rank <= 256) LAT_LAUNCH(256);
    else if (rank <= 384) LAT_LAUNCH(384);
    else LAT_LAUNCH(512);
#undef LAT_LAUNCH
    if (shares > 1)
        hipLaunchKernelGGL(latent_attn_merge_kernel, dim3((unsigned)tokens, (unsigned)heads, (unsigned)((rank + 127) / 128)),
                           dim3(NVA_WAVE), 0, stream, part,
                           shares, (__bf16*)out, out_stride, heads, rank);
    return nva_check_launch("latent_attention");
}

// The portions of prompts of a step: row_tiles is int32 [num_tiles][2] = (request, row tile of 32 queries), requests described
// by cu_seqlens_q and kv_lens as for the other prefill kernels; q2 and out hold all the step's tokens.  Takes what
// nva_latent_attention takes, and returns 1 for what it does not.
NVA_EXPORT int nva_latent_attention_prefill_bf16(const void* q2, int64_t q_stride, void* out, int64_t out_stride,
                                                 const void* k_cache, const void* v_cache, const int32_t* block_tables,
                                                 int table_stride, const int32_t* cu_seqlens_q, const int32_t* kv_lens,
                                                 const int32_t* row_tiles, int64_t num_tiles, int heads, int rank, int rot,
                                                 int page_size, float scale, const float* sinks, int32_t* error_flag,
                                                 hipStream_t stream) {
    if (num_tiles == 0) return 0;
    if (rank % 16 || rank <= 0 || rank > 512 || rot % 8 || rot <= 0 || rot > LAT_MAX_ROT || page_size % LAT_TILE || page_size <= 0) {
        nva_fail("latent_attention_prefill: sizes it does not take (%d, %d, %d)", rank, rot, page_size);
        return 1;
    }
    if (!row_tiles || num_tiles < 0 || num_tiles * 8 > 0x7fffffff || heads <= 0 || table_stride <= 0 || !(scale > 0.f))
        return nva_fail("latent_attention_prefill: bad sizes tiles=%lld heads=%d", (long long)num_tiles, heads);
    if (q_stride % 8 || out_stride % 4 || !nva_aligned(q2, 16) || !nva_aligned(out, 8) || !nva_aligned(k_cache, 16) ||
        !nva_aligned(v_cache, 16)) {
        nva_fail("latent_attention_prefill: rows that are not aligned for vector access");
        return 1;
    }
    const size_t lds = ((size_t)LAT_TILE * (rank + rot + 8) + (size_t)rank * (LAT_TILE + 4)) * sizeof(__bf16);
    const int waves = rank <= 384 ? 8 : 4;       // tokens of a workgroup (what the registers of a SIMD hold two waves of)
    dim3 grid((unsigned)(num_tiles * (32 / waves)), 1, (unsigned)((heads + 15) / 16));
#define LAT_LAUNCH(MC, WV)                                                                                           \
    do {                                                                                                             \
        auto kernel = latent_attn_quad_kernel<MC, WV>;                                                                 \
        static bool raised = false;                                                                                  \
        if (!raised && lds > 48 * 1024) {                                                                            \
            if (hipFuncSetAttribute((const void*)kernel, hipFuncAttributeMaxDynamicSharedMemorySize, 96 * 1024) != hipSuccess) \
                return nva_fail("latent_attention_prefill: cannot have %zu bytes of LDS", lds);                      \
            raised = true;                                                                                           \
        }                                                                                                            \
        hipLaunchKernelGGL(kernel, grid, dim3(WV * NVA_WAVE), lds, stream, (const __bf16*)q2, q_stride, (__bf16*)out,    \
                           out_stride, (const __bf16*)k_cache, (const __bf16*)v_cache, block_tables, table_stride,      \
                           cu_seqlens_q, kv_lens, row_tiles, heads, rank, rot, page_size, scale, sinks, error_flag);    \
    } while (0)
    if (rank <= 128) LAT_LAUNCH(128, 8);
    else if (rank <= 256) LAT_LAUNCH(256, 8);
    else if (rank <= 384) LAT_LAUNCH(384, 8);
    else LAT_LAUNCH(512, 4);
#undef LAT_LAUNCH
    return nva_check_launch("latent_attention_prefill");
}
#endif

NVA_DEFINE_LAST_ERROR(nva_latent)
