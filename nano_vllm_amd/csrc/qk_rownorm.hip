// Preparation of q, k and v of an attention whose query and key norms run over the whole
// projection, before it is split into heads, and whose positions enter through the length of the
// query only (no rotation):
//
//     q <- q / sqrt(mean(q^2) + eps) * wq * temp(p)        mean over all Hq * D entries of the token's q
//     k <- k / sqrt(mean(k^2) + eps) * wk                  mean over all Hkv * D entries
//     temp(p) = 1 + coef * ln(floor((p + 1) / every) + 1)  (coef 0: no temperature)
//     q, k <- rotation of the first R channels of every head, pairs (i, i + R/2), by the token's row of
//             rot_table (R/2 cosines, then R/2 sines; null: no rotation), after norm and temperature
//     cache <- k, v                                        at the token's slot (slot < 0: nothing is written)
//
// The row is the packed projection [q | k | v] of Hq * D, Hkv * D and Hkv * DV entries, biases added
// by the product (or still to be added: the row may come as the float partial sums of a product whose
// k range was split, which are added up here).  Sums of squares, scales, the logarithm and the products
// are float; q is written out and k, v into the cache, each rounded once to the element type.  The weights are
// plain (not one-plus), stored as elements or float.
// Cache layout: K [pages, Hkv, page, D], V [pages, Hkv, page / vt, DV, vt] (common.h).
// With per_head the two norms run over every head by itself, mean over its D entries, with weights of D
// entries that the heads share.
// rot_interleaved: the rotation pairs the neighbours (2i, 2i + 1) of the first R channels instead of (i, i + R/2);
// the table's row is the same (R/2 cosines, then R/2 sines, of the angles p * f_i).
// v_norm: every value head is divided by its root mean square over DV (eps inside the root, no weight).
// v_first_out, float [tokens, Hkv * DV]: the values as they are after the norm are also written there, unrounded (the
// first of the layers that mix values hands them to the later ones of the same step).  v_first_in with v_mix (one
// float read on the device): v <- (1 - v_mix) v + v_mix v_first_in, after the norm, before the store.
// One workgroup per token.
#include "common.h"

template <typename T>
__global__ void __launch_bounds__(1024)
qk_rownorm_store_kernel(const T* __restrict__ qkv, int64_t stride, PartialInput part, T* __restrict__ q_out,
                        int64_t q_stride, int num_heads, int num_kv_heads, int head_dim, int v_dim,
                        const void* __restrict__ q_weight, const void* __restrict__ k_weight, int w_is_f32, float eps,
                        const int32_t* __restrict__ positions, float temp_coef, int temp_every,
                        const float* __restrict__ rot_table, int rot,
                        const int32_t* __restrict__ slots, T* __restrict__ k_cache, T* __restrict__ v_cache,
                        int page_size, int per_head, int rot_interleaved, int v_norm,
                        const float* __restrict__ v_first_in, const float* __restrict__ v_mix,
                        float* __restrict__ v_first_out) {
    extern __shared__ __attribute__((aligned(16))) float row_s[];      // the token's row, as float; then a scale per head
    __shared__ float scratch[16];
    const int64_t t = blockIdx.x;
    const int qd = num_heads * head_dim, kd = num_kv_heads * head_dim, vd = num_kv_heads * v_dim;
    const int width = qd + kd + vd;
    const int tid = threadIdx.x;
    // what the slot and the position say is asked for before the row arrives
    const int slot = slots ? slots[t] : -1;
    const int steps = temp_coef != 0.f ? (positions[t] + 1) / temp_every : 0;

    float sq = 0.f, sk = 0.f;
    for (int i = tid; i < width; i += blockDim.x) {
        const float x = part.sums ? partial_value<T>(part, t, width, i) : to_float(qkv[t * stride + i]);
        row_s[i] = x;
        if (i < qd) sq += x * x; else if (i < qd + kd) sk += x * x;
    }
    float* const head_scale = row_s + width;                           // [num_heads + num_kv_heads], with per_head
    float* const v_scale = head_scale + (per_head ? num_heads + num_kv_heads : 0);      // [num_kv_heads], with v_norm
    if (v_norm) {
        __syncthreads();
        const int wave = tid / NVA_WAVE, lane = tid % NVA_WAVE, nwaves = blockDim.x / NVA_WAVE;
        for (int g = wave; g < num_kv_heads; g += nwaves) {
            float ss = 0.f;
            for (int d = lane; d < v_dim; d += NVA_WAVE) ss += row_s[qd + kd + g * v_dim + d] * row_s[qd + kd + g * v_dim + d];
            ss = wave_sum(ss);
            if (lane == 0) v_scale[g] = rsqrtf(ss / (float)v_dim + eps);
        }
    }
    if (per_head) {
        __syncthreads();
        const int wave = tid / NVA_WAVE, lane = tid % NVA_WAVE, nwaves = blockDim.x / NVA_WAVE;
        for (int hh = wave; hh < num_heads + num_kv_heads; hh += nwaves) {
            float ss = 0.f;
            for (int d = lane; d < head_dim; d += NVA_WAVE) ss += row_s[hh * head_dim + d] * row_s[hh * head_dim + d];
            ss = wave_sum(ss);
            if (lane == 0) head_scale[hh] = rsqrtf(ss / (float)head_dim + eps);
        }
        __syncthreads();
    } else {
        sq = block_sum(sq, scratch);
        sk = kd ? block_sum(sk, scratch) : 0.f;
    }

    float q_scale = q_weight && !per_head ? rsqrtf(sq / (float)qd + eps) : 1.f;
    if (temp_coef != 0.f) q_scale *= 1.f + temp_coef * logf((float)steps + 1.f);
    T* qrow = q_out + t * q_stride;
    const float* rot_row = rot_table ? rot_table + t * (int64_t)rot : nullptr;
    const int half = rot / 2;
    auto weight_of = [&](const void* w, int i) -> float {
        return !w ? 1.f : w_is_f32 ? static_cast<const float*>(w)[i] : to_float(static_cast<const T*>(w)[i]);
    };
    // entry i of a projection that starts at `at` in the row, scaled and weighted, then turned with its partner
    auto prepared = [&](int at, int i, float scale, const void* w) -> float {
        const int d = i % head_dim;
        if (per_head && w) scale *= head_scale[(at + i) / head_dim];   // (at is a multiple of the head size)
        const float x = row_s[at + i] * scale * weight_of(w, per_head ? d : i);
        if (!rot_row || d >= rot) return x;
        if (rot_interleaved) {
            const int j = (d & 1) ? i - 1 : i + 1;
            const float y = row_s[at + j] * scale * weight_of(w, per_head ? j % head_dim : j);
            const float c = rot_row[d >> 1], sn = rot_row[half + (d >> 1)];
            return (d & 1) ? x * c + y * sn : x * c - y * sn;
        }
        const int f = d < half ? d : d - half;
        const int j = d < half ? i + half : i - half;
        const float y = row_s[at + j] * scale * weight_of(w, per_head ? j % head_dim : j);
        const float c = rot_row[f], sn = rot_row[half + f];
        return d < half ? x * c - y * sn : x * c + y * sn;
    };
    for (int i = tid; i < qd; i += blockDim.x) qrow[i] = from_float<T>(prepared(0, i, q_scale, q_weight));
    if (v_norm) __syncthreads();                                      // (the values' scales; without per_head no barrier came since)
    const float lam = v_first_in ? v_mix[0] : 0.f;
    auto value_of = [&](int i) -> float {
        float v = row_s[qd + kd + i];
        if (v_norm) v *= v_scale[i / v_dim];
        if (v_first_in) v = (1.f - lam) * v + lam * v_first_in[t * vd + i];
        return v;
    };
    if (v_first_out)                                                  // also for a token that stores nothing
        for (int i = tid; i < vd; i += blockDim.x) v_first_out[t * vd + i] = row_s[qd + kd + i] * (v_norm ? v_scale[i / v_dim] : 1.f);
    if (!kd || slot < 0 || !k_cache) return;
    const float k_scale = k_weight && !per_head ? rsqrtf(sk / (float)kd + eps) : 1.f;
    const int page = slot / page_size, off = slot % page_size;
    const int vt = nva_v_tile(page_size);
    for (int i = tid; i < kd; i += blockDim.x) {
        const int g = i / head_dim, d = i % head_dim;
        k_cache[(((int64_t)page * num_kv_heads + g) * page_size + off) * head_dim + d] =
            from_float<T>(prepared(qd, i, k_scale, k_weight));
    }
    for (int i = tid; i < vd; i += blockDim.x) {
        const int g = i / v_dim, d = i % v_dim;
        v_cache[((int64_t)page * num_kv_heads + g) * v_dim * (int64_t)page_size + nva_v_offset(off, d, v_dim, vt)] =
            from_float<T>(value_of(i));
    }
}

// qkv: [tokens, Hq * D + Hkv * D + Hkv * DV] with rows `stride` elements apart, or (sums != null) the float
// partial sums [splits][tokens][width] of the projection with its bias, which are added up here.
// q_out: [tokens, Hq * D] with rows q_stride apart (it may be qkv itself: q is then rewritten in place).
// q_weight [Hq * D], k_weight [Hkv * D] (per_head: both [D]): both or none.  positions are needed with a temperature.
// rot_table: float [tokens, rot], a row per token of this call, or null.
// slots (with the caches) may be null: nothing is stored then.  num_kv_heads 0: the row holds q only.
NVA_EXPORT int NVA_NAME(nva_qk_rownorm_store)(const void* qkv, int64_t stride, const float* sums, int splits,
                                              int64_t split_stride, const void* bias, void* q_out, int64_t q_stride,
                                              int64_t tokens, int num_heads, int num_kv_heads,
                                              int head_dim, int v_dim, const void* q_weight, const void* k_weight,
                                              int w_is_f32, float eps, const int32_t* positions, float temp_coef,
                                              int temp_every, const float* rot_table, int rot, const int32_t* slots,
                                              void* k_cache, void* v_cache, int page_size, int per_head,
                                              int rot_interleaved, int v_norm, const float* v_first_in,
                                              const float* v_mix, float* v_first_out, hipStream_t stream) {
    if (tokens == 0) return 0;
    if (tokens < 0 || tokens > 0x7fffffff) return nva_fail("qk_rownorm_store: bad token count %lld", (long long)tokens);
    if (num_heads <= 0 || num_kv_heads < 0 || head_dim <= 0 || v_dim <= 0)
        return nva_fail("qk_rownorm_store: bad sizes heads=%d kv_heads=%d head_dim=%d v_dim=%d", num_heads, num_kv_heads,
                        head_dim, v_dim);
    const int64_t width = (int64_t)(num_heads + num_kv_heads) * head_dim + (int64_t)num_kv_heads * v_dim;
    if (width > 36 * 1024) return nva_fail("qk_rownorm_store: a row of %lld entries does not fit the LDS", (long long)width);
    if (!sums && (!qkv || stride < width))
        return nva_fail("qk_rownorm_store: rows of %lld elements are %lld apart", (long long)width, (long long)stride);
    if (sums && (splits <= 0 || split_stride < tokens * width)) return nva_fail("qk_rownorm_store: bad partial sums");
    if (!q_out || q_stride < (int64_t)num_heads * head_dim) return nva_fail("qk_rownorm_store: no room for q");
    if (num_kv_heads && (q_weight == nullptr) != (k_weight == nullptr))
        return nva_fail("qk_rownorm_store: give both norm weights or none");
    if (temp_coef != 0.f && (!positions || temp_every <= 0))
        return nva_fail("qk_rownorm_store: a query temperature needs positions and a positive step");
    if (rot_table && (rot <= 0 || rot % 2 || rot > head_dim))
        return nva_fail("qk_rownorm_store: %d rotated channels of a head of %d", rot, head_dim);
    if (v_first_in && (!v_mix || v_first_out)) return nva_fail("qk_rownorm_store: mixing values needs the factor, and reads or writes the first values, not both");
    if ((k_cache || v_cache) && (!k_cache || !v_cache || !slots || page_size <= 0 || !num_kv_heads))
        return nva_fail("qk_rownorm_store: storing needs both caches, the slots and the page size");
    auto kernel = qk_rownorm_store_kernel<elem_t>;
    const size_t lds = (size_t)(width + (per_head ? num_heads + num_kv_heads : 0) + (v_norm ? num_kv_heads : 0)) * sizeof(float);
    static bool raised = false;
    if (!raised && lds > 48 * 1024) {
        if (hipFuncSetAttribute((const void*)kernel, hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024) != hipSuccess)
            return nva_fail("qk_rownorm_store: cannot have %zu bytes of LDS", lds);
        raised = true;
    }
    const PartialInput part{sums, splits, split_stride, bias};
    // few tokens (a decode step): more threads a token, so that a row of partial sums is asked for at once
    const int threads = tokens <= 64 && width >= 2048 ? 1024 : 256;
    hipLaunchKernelGGL(kernel, dim3((unsigned)tokens), dim3(threads), lds, stream, (const elem_t*)qkv, stride, part,
                       (elem_t*)q_out, q_stride, num_heads, num_kv_heads, head_dim, v_dim, q_weight, k_weight, w_is_f32, eps,
                       positions, temp_coef, temp_every, rot_table, rot_table ? rot : 0, slots, (elem_t*)k_cache, (elem_t*)v_cache, page_size,
                       per_head ? 1 : 0, rot_interleaved ? 1 : 0, v_norm ? 1 : 0, v_first_in, v_mix, v_first_out);
    return nva_check_launch("qk_rownorm_store");
}

NVA_DEFINE_LAST_ERROR(nva_qk_rownorm)
