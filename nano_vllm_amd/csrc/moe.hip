// A routed feed-forward (mixture of experts): the choice of experts, and the experts' products over
// the tokens sorted by expert.  Nothing here asks the host how the tokens were shared out: every
// kernel's launch depends on the number of tokens alone.
//
//   route     s = sigmoid(z) of the router's float logits z [tokens, E]; the experts form `group_count` equal
//             groups of neighbours; a group's score is the sum of its two largest scores (of its one score
//             where a group holds one expert); the `group_keep` groups with the largest scores stay; of
//             their experts the `top` with the largest scores are chosen (equal scores: the lower number);
//             ids [tokens, top], weights [tokens, top] = scale * s.
//             With softmax_top the logits (plus an optional float bias per expert) are compared as they are: the
//             `top` largest are chosen (no groups) and weighted by the softmax over the chosen logits alone.
//             With softmax_choice (mode 2) s = softmax(z) over all experts; an expert is chosen by s + bias (a float per
//             expert), a group counts by the largest such choice score in it, only the kept groups' experts can be
//             chosen (the others do not take part, whatever the sign of the scores); the weights are the chosen
//             experts' s (without the bias) divided by their sum + 1e-20.
//             Experts numbered from `experts` on (the kernels of the products are told how many real ones there are)
//             are identities: their output is the token's input itself.
//   plan      the pairs (token, choice) counted and sorted by expert: place[pair] = the pair's row among the
//             sorted ones, rows[place] = pair; the sorted rows cut into tiles of 32 or 128 rows of one expert:
//             tile_expert[i], tile_row0[i], tile_rows[i], and their number.
//   up        h[row] = act(x[token of row] Wu_e^T)         rows sorted by expert, a tile of rows and 64 or 128
//             gated: h[row] = act(x Wg_e^T) * (x Wu_e^T), an expert's matrix holding its gate rows, then its up rows
//   down      o[row] = h[row] Wd_e^T                       outputs to a workgroup
//   combine   y[token] = sum over its choices of weight * o[place] (x[token] for an identity) (+ add[token], times
//             sigmoid(add_gate[token]) where a float gate logit per token is given)
//
// The products are float sums of a row by itself (on the vector units over k in ascending order, one chain per
// output; on the matrix cores in the order of the instruction's steps), so a token's result does not depend on
// what else is in the batch or on where its row fell among the sorted ones; operands and results are elements
// (rounded once), the combination is float.
#include "common.h"

#define MOE_BM 32
#define MOE_BN 64
#define MOE_BK 32
#define MOE_MAX_EXPERTS 1024

// The largest value among the lanes' candidates and its index (of equal values the lower index), in all lanes.
__device__ __forceinline__ void moe_wave_best(float& v, int& idx) {
#pragma unroll
    for (int off = NVA_WAVE / 2; off > 0; off >>= 1) {
        const float ov = __shfl_xor(v, off, NVA_WAVE);
        const int oi = __shfl_xor(idx, off, NVA_WAVE);
        if (ov > v || (ov == v && oi < idx)) { v = ov; idx = oi; }
    }
}

// One wave per token: a lane looks after the experts (and groups) lane, lane + 64, ...; every choice is a
// maximum over the wave.
__global__ void __launch_bounds__(NVA_WAVE)
moe_route_kernel(const float* __restrict__ logits, int64_t stride, int experts, int top, int group_count, int group_keep,
                 float scale, int softmax_top, const float* __restrict__ bias, int32_t* __restrict__ ids,
                 float* __restrict__ weights) {
    __shared__ float s_s[MOE_MAX_EXPERTS];           // what the experts are compared by
    __shared__ float w_s[MOE_MAX_EXPERTS];           // softmax_choice: the scores without the bias
    __shared__ float g_s[MOE_MAX_EXPERTS];           // group scores; -inf once taken
    __shared__ unsigned char open_s[MOE_MAX_EXPERTS];
    const int64_t t = blockIdx.x;
    const int lane = threadIdx.x;
    const bool all_groups = group_keep == group_count;
    const bool choice = softmax_top == 2;
    if (choice) {
        float m = -INFINITY;
        for (int e = lane; e < experts; e += NVA_WAVE) m = fmaxf(m, logits[t * stride + e]);
        m = wave_max(m);
        float sum = 0.f;
        for (int e = lane; e < experts; e += NVA_WAVE) {
            const float x = expf(logits[t * stride + e] - m);
            w_s[e] = x;
            sum += x;
        }
        sum = wave_sum(sum);
        for (int e = lane; e < experts; e += NVA_WAVE) {
            w_s[e] /= sum;
            s_s[e] = w_s[e] + (bias ? bias[e] : 0.f);
            open_s[e] = all_groups ? 1 : 0;
        }
    } else
    for (int e = lane; e < experts; e += NVA_WAVE) {
        const float z = logits[t * stride + e] + (bias ? bias[e] : 0.f);
        s_s[e] = softmax_top ? z : 1.f / (1.f + expf(-z));
        open_s[e] = all_groups ? 1 : 0;
    }
    __syncthreads();
    const int per = experts / group_count;
    if (!all_groups) {
        for (int g = lane; g < group_count; g += NVA_WAVE) {
            float a = -INFINITY, b = -INFINITY;      // the two largest of the group
            for (int i = 0; i < per; ++i) {
                const float v = s_s[g * per + i];
                if (v > a) { b = a; a = v; } else if (v > b) b = v;
            }
            g_s[g] = per > 1 && !choice ? a + b : a;
        }
        __syncthreads();
        for (int k = 0; k < group_keep; ++k) {
            float v = -INFINITY;
            int best = 0x7fffffff;
            for (int g = lane; g < group_count; g += NVA_WAVE)
                if (g_s[g] > v) { v = g_s[g]; best = g; }
            moe_wave_best(v, best);
            __syncthreads();
            if (lane == 0) g_s[best] = -INFINITY;
            for (int i = lane; i < per; i += NVA_WAVE) open_s[best * per + i] = 1;
            __syncthreads();
        }
    }
    for (int k = 0; k < top; ++k) {
        float v = -INFINITY;
        int best = 0x7fffffff;
        for (int e = lane; e < experts; e += NVA_WAVE)
            if (open_s[e] && s_s[e] > v) { v = s_s[e]; best = e; }
        moe_wave_best(v, best);
        __syncthreads();
        if (lane == 0) {
            open_s[best] = 0;
            ids[t * top + k] = best;
            weights[t * top + k] = choice ? w_s[best] : softmax_top ? v : scale * v;
        }
        __syncthreads();
    }
    if (choice) {
        if (lane == 0) {
            float sum = 0.f;
            for (int k = 0; k < top; ++k) sum += weights[t * top + k];
            sum += 1e-20f;
            for (int k = 0; k < top; ++k) weights[t * top + k] /= sum;
        }
    } else if (softmax_top && lane == 0) {
        // the chosen logits, largest first: their softmax among themselves, summed in the order of the choice
        const float m = weights[t * top];
        float sum = 0.f;
        for (int k = 0; k < top; ++k) sum += expf(weights[t * top + k] - m);
        for (int k = 0; k < top; ++k) weights[t * top + k] = expf(weights[t * top + k] - m) / sum;
    }
}

// One workgroup.  Counts and offsets live in LDS; pairs is tokens * top.  Where a pair falls among the rows
// of its expert depends on the order in which the threads arrive; no result does, since every row of the
// products is computed by itself.
__global__ void __launch_bounds__(1024)
moe_plan_kernel(const int32_t* __restrict__ ids, int64_t pairs, int experts, int bm, int32_t* __restrict__ place,
                int32_t* __restrict__ rows, int32_t* __restrict__ tile_expert, int32_t* __restrict__ tile_row0,
                int32_t* __restrict__ tile_rows, int32_t* __restrict__ num_tiles) {
    __shared__ int count_s[MOE_MAX_EXPERTS], cursor_s[MOE_MAX_EXPERTS], begin_s[MOE_MAX_EXPERTS], tile0_s[MOE_MAX_EXPERTS];
    for (int e = threadIdx.x; e < experts; e += blockDim.x) count_s[e] = cursor_s[e] = 0;
    __syncthreads();
    for (int64_t i = threadIdx.x; i < pairs; i += blockDim.x)
        if (ids[i] < experts) atomicAdd(&count_s[ids[i]], 1);      // (an identity takes no row of the products)
    __syncthreads();
    if (threadIdx.x == 0) {
        int at = 0, tiles = 0;
        for (int e = 0; e < experts; ++e) {
            begin_s[e] = at;
            tile0_s[e] = tiles;
            at += count_s[e];
            tiles += (count_s[e] + bm - 1) / bm;
        }
        num_tiles[0] = tiles;
    }
    __syncthreads();
    for (int e = threadIdx.x; e < experts; e += blockDim.x) {
        const int n = count_s[e];
        for (int i = 0; i * bm < n; ++i) {
            tile_expert[tile0_s[e] + i] = e;
            tile_row0[tile0_s[e] + i] = begin_s[e] + i * bm;
            tile_rows[tile0_s[e] + i] = min(bm, n - i * bm);
        }
    }
    for (int64_t i = threadIdx.x; i < pairs; i += blockDim.x) {
        const int e = ids[i];
        if (e >= experts) { place[i] = -1; continue; }
        const int r = begin_s[e] + atomicAdd(&cursor_s[e], 1);
        place[i] = r;
        rows[r] = (int32_t)i;
    }
}

// Tile product: out[row0 + r, n0 + c] = f(sum_k a[src(row0 + r), k] * w[e * n + n0 + c, k]).
// UP: src = token of the pair (rows[row] / top), f = act; else src = the row itself, f = identity.
// GATED (with UP): the expert's matrix has 2 n rows, gate rows then up rows, and out = act(gate sum) * up sum.
template <typename T, bool UP, bool GATED = false>
__global__ void __launch_bounds__(256)
moe_tile_kernel(const T* __restrict__ a, int64_t a_stride, const T* __restrict__ w, int n, int k,
                const int32_t* __restrict__ rows, int top, const int32_t* __restrict__ tile_expert,
                const int32_t* __restrict__ tile_row0, const int32_t* __restrict__ tile_rows,
                const int32_t* __restrict__ num_tiles, int act, T* __restrict__ out, int64_t out_stride) {
    __shared__ float a_s[MOE_BM][MOE_BK + 1];
    __shared__ float w_s[MOE_BN][MOE_BK + 1];
    __shared__ float u_s[GATED ? MOE_BN : 1][MOE_BK + 1];          // the up rows of the same outputs
    __shared__ int src_s[MOE_BM];
    const int tile = blockIdx.x;
    if (tile >= num_tiles[0]) return;
    const int e = tile_expert[tile], row0 = tile_row0[tile], nrows = tile_rows[tile];
    const int n0 = blockIdx.y * MOE_BN;
    const int tid = threadIdx.x;
    if (tid < MOE_BM) src_s[tid] = tid < nrows ? (UP ? rows[row0 + tid] / top : row0 + tid) : -1;
    __syncthreads();
    const T* we = w + (int64_t)e * (GATED ? 2 : 1) * n * k;
    const int ty = tid / 16, tx = tid % 16;          // rows ty, ty + 16; columns tx + 16 j
    float acc[2][4] = {{0.f, 0.f, 0.f, 0.f}, {0.f, 0.f, 0.f, 0.f}};
    float up[2][4] = {{0.f, 0.f, 0.f, 0.f}, {0.f, 0.f, 0.f, 0.f}};
    for (int k0 = 0; k0 < k; k0 += MOE_BK) {
        for (int i = tid; i < MOE_BM * MOE_BK; i += 256) {
            const int r = i / MOE_BK, c = i % MOE_BK;
            a_s[r][c] = src_s[r] >= 0 && k0 + c < k ? to_float(a[(int64_t)src_s[r] * a_stride + k0 + c]) : 0.f;
        }
        for (int i = tid; i < MOE_BN * MOE_BK; i += 256) {
            const int r = i / MOE_BK, c = i % MOE_BK;
            w_s[r][c] = n0 + r < n && k0 + c < k ? to_float(we[(int64_t)(n0 + r) * k + k0 + c]) : 0.f;
            if (GATED) u_s[r][c] = n0 + r < n && k0 + c < k ? to_float(we[(int64_t)(n + n0 + r) * k + k0 + c]) : 0.f;
        }
        __syncthreads();
#pragma unroll
        for (int c = 0; c < MOE_BK; ++c) {
            const float a0 = a_s[ty][c], a1 = a_s[ty + 16][c];
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const float b = w_s[tx + 16 * j][c];
                acc[0][j] += a0 * b;
                acc[1][j] += a1 * b;
                if (GATED) {
                    const float u = u_s[tx + 16 * j][c];
                    up[0][j] += a0 * u;
                    up[1][j] += a1 * u;
                }
            }
        }
        __syncthreads();
    }
#pragma unroll
    for (int i = 0; i < 2; ++i) {
        const int r = ty + 16 * i;
        if (r >= nrows) continue;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int c = n0 + tx + 16 * j;
            if (c < n) out[(int64_t)(row0 + r) * out_stride + c] = from_float<T>(
                GATED ? nva_gate_act(act, acc[i][j]) * up[i][j]
                      : UP ? nva_gate_act(act, acc[i][j]) : acc[i][j]);
        }
    }
}

#if defined(NVA_BF16)
// ---------------------------------------------------------------------------- the tile product on the matrix cores
// A workgroup of four waves takes a tile of BM rows (of one expert) and 4 * WR outputs: a wave 16 or 32 rows of the
// expert's matrix as the A operand of v_mfma_f32_16x16x32_bf16, straight from global memory into registers (a lane 16
// bytes of a row a load; every byte of the matrix is read once per tile of rows), and all BM rows of x as B operands
// from LDS, where the tile's rows are gathered a chunk of MOE_KC columns at a time.  A row's sum over k runs in the
// order of the chunks whatever the tile it fell into.  GATED (with UP; WR a multiple of 32): the expert's matrix has
// 2 n rows, gate rows then up rows; a wave takes WR / 2 outputs, the first half of its fragments their gate rows and
// the second half their up rows, and gates in its epilogue.
typedef __attribute__((ext_vector_type(8))) __bf16 moe_bf16x8;
typedef __attribute__((ext_vector_type(4))) float moe_f32x4;
#define MOE_KC 128

template <int BM, int WR, bool UP, bool GATED = false>
__global__ void __launch_bounds__(256)
moe_mfma_kernel(const __bf16* __restrict__ a, int64_t a_stride, const __bf16* __restrict__ w, int n, int k,
                const int32_t* __restrict__ rows, int top, const int32_t* __restrict__ tile_expert,
                const int32_t* __restrict__ tile_row0, const int32_t* __restrict__ tile_rows,
                const int32_t* __restrict__ num_tiles, int act, __bf16* __restrict__ out, int64_t out_stride) {
    constexpr int MB = BM / 16, FR = WR / 16, XS = MOE_KC + 8;
    constexpr int KS = MOE_KC / 32;                         // products' steps of 32 columns in a chunk
    constexpr int XP = BM * (MOE_KC / 8) / 256;             // 16-byte pieces of a chunk of x a thread gathers
    static_assert(BM * (MOE_KC / 8) % 256 == 0, "the pieces of a chunk of x divide among the threads");
    __shared__ __attribute__((aligned(16))) __bf16 x_s[2][BM * XS];      // two chunks: one multiplied, one arriving
    __shared__ int src_s[BM];
    const int tile = blockIdx.x;
    if (tile >= num_tiles[0]) return;
    const int e = tile_expert[tile], row0 = tile_row0[tile], nrows = tile_rows[tile];
    const int tid = threadIdx.x, wave = tid / NVA_WAVE, lane = tid % NVA_WAVE, col = lane & 15, g = lane >> 4;
    static_assert(!GATED || (UP && FR % 2 == 0), "gating needs an even number of fragments");
    constexpr int WO = GATED ? WR / 2 : WR;                 // outputs of a wave
    constexpr int FO = GATED ? FR / 2 : FR;                 // fragments of 16 outputs
    const int n0 = blockIdx.y * 4 * WO + wave * WO;
    if (tid < BM) src_s[tid] = tid < nrows ? (UP ? rows[row0 + tid] / top : row0 + tid) : -1;
    __syncthreads();
    const __bf16* we = w + (int64_t)e * (GATED ? 2 : 1) * n * k;
    const __bf16* wrow[FR];
#pragma unroll
    for (int f = 0; f < FR; ++f)
        wrow[f] = we + ((int64_t)min(n0 + 16 * (f % FO) + col, n - 1) + (f >= FO ? n : 0)) * k + 8 * g;
    // the rows of x this thread gathers: piece i is row (tid + 256 i) / (MOE_KC / 8), columns 8 ((tid + 256 i) % (MOE_KC / 8))
    const __bf16* xsrc[XP];
    int xcol[XP];
#pragma unroll
    for (int i = 0; i < XP; ++i) {
        const int idx = tid + 256 * i, r = idx / (MOE_KC / 8);
        xcol[i] = (idx % (MOE_KC / 8)) * 8;
        xsrc[i] = src_s[r] >= 0 ? a + (int64_t)src_s[r] * a_stride + xcol[i] : nullptr;
    }
    moe_f32x4 acc[FR][MB];
#pragma unroll
    for (int f = 0; f < FR; ++f)
#pragma unroll
        for (int b = 0; b < MB; ++b) acc[f][b] = moe_f32x4{0.f, 0.f, 0.f, 0.f};
    const int k_last = k - 8;                      // k is a multiple of 8 (checked by the launcher)
    // (two sets of registers for the matrix's part, named apart so that neither is ever indexed at run time)
    moe_bf16x8 fa0[KS][FR], fa1[KS][FR], xr[XP];
    auto ask = [&](int k0, moe_bf16x8 (&fa)[KS][FR]) __attribute__((always_inline)) {   // a chunk's part of the matrix and of x
#pragma unroll
        for (int c = 0; c < KS; ++c)
#pragma unroll
            for (int f = 0; f < FR; ++f)
                fa[c][f] = *reinterpret_cast<const moe_bf16x8*>(wrow[f] + min(k0 + 32 * c, k_last - 8 * g));
#pragma unroll
        for (int i = 0; i < XP; ++i) {
#pragma unroll
            for (int q = 0; q < 8; ++q) xr[i][q] = (__bf16)0.f;
            if (xsrc[i] && k0 + xcol[i] < k) xr[i] = *reinterpret_cast<const moe_bf16x8*>(xsrc[i] + k0);
        }
    };
    auto put = [&](__bf16* xs) __attribute__((always_inline)) {           // the gathered chunk of x into LDS
#pragma unroll
        for (int i = 0; i < XP; ++i) {
            const int idx = tid + 256 * i;
            *reinterpret_cast<moe_bf16x8*>(&xs[(idx / (MOE_KC / 8)) * XS + xcol[i]]) = xr[i];
        }
    };
    // one chunk: the next one is asked for first and is on its way during this chunk's products
    auto chunk = [&](int k0, moe_bf16x8 (&fa)[KS][FR], moe_bf16x8 (&fa_next)[KS][FR], const __bf16* xs, __bf16* xs_next)
                     __attribute__((always_inline)) {
        const bool more = k0 + MOE_KC < k;
        if (more) ask(k0 + MOE_KC, fa_next);
#pragma unroll
        for (int c = 0; c < KS; ++c) {
            if (k0 + 32 * c >= k) break;           // (columns of x beyond k are zero, the matrix's clamped)
#pragma unroll
            for (int b = 0; b < MB; ++b) {
                const moe_bf16x8 fb = *reinterpret_cast<const moe_bf16x8*>(&xs[(16 * b + col) * XS + 32 * c + 8 * g]);
#pragma unroll
                for (int f = 0; f < FR; ++f) acc[f][b] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(fa[c][f], fb, acc[f][b], 0, 0, 0);
            }
        }
        if (more) put(xs_next);                    // (what lay there was read before the last barrier)
        __syncthreads();
    };
    ask(0, fa0);
    put(x_s[0]);
    __syncthreads();
    for (int k0 = 0; k0 < k; k0 += 2 * MOE_KC) {
        chunk(k0, fa0, fa1, x_s[0], x_s[1]);
        if (k0 + MOE_KC < k) chunk(k0 + MOE_KC, fa1, fa0, x_s[1], x_s[0]);
    }
    // acc[f][b][i] = out[row 16 b + col][n0 + 16 f + 4 g + i]  (gated: fragment f + FO holds the up sums of the same outputs)
#pragma unroll
    for (int f = 0; f < FO; ++f)
#pragma unroll
        for (int b = 0; b < MB; ++b) {
            const int r = 16 * b + col;
            if (r >= nrows) continue;
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const int c = n0 + 16 * f + 4 * g + i;
                float v = acc[f][b][i];
                if (GATED) v = nva_gate_act(act, v) * acc[GATED ? f + FO : f][b][i];
                else if (UP) v = nva_gate_act(act, v);
                if (c < n) out[(int64_t)(row0 + r) * out_stride + c] = (__bf16)v;
            }
        }
}
#endif

template <typename T>
__global__ void __launch_bounds__(256)
moe_combine_kernel(const T* __restrict__ o, int64_t o_stride, const int32_t* __restrict__ place,
                   const float* __restrict__ weights, int top, const T* __restrict__ add, int64_t add_stride,
                   const float* __restrict__ add_gate, int64_t gate_stride, const T* __restrict__ x, int64_t x_stride,
                   T* __restrict__ y, int64_t y_stride, int width) {
    const int64_t t = blockIdx.y;
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= width) return;
    float sum = 0.f;
    for (int c = 0; c < top; ++c) {
        const int at = place[t * top + c];
        sum += weights[t * top + c] * to_float(at < 0 ? x[t * x_stride + i] : o[(int64_t)at * o_stride + i]);
    }
    if (add) {
        const float a = to_float(add[t * add_stride + i]);
        sum += add_gate ? a / (1.f + expf(-add_gate[t * gate_stride])) : a;
    }
    y[t * y_stride + i] = from_float<T>(sum);
}

NVA_EXPORT int NVA_NAME(nva_moe_route)(const float* logits, int64_t stride, int64_t tokens, int experts, int top,
                                       int group_count, int group_keep, float scale, int softmax_top, const float* bias,
                                       int32_t* ids, float* weights, hipStream_t stream) {
    if (tokens == 0) return 0;
    if (tokens < 0 || tokens > 0x7fffffff || experts <= 0 || experts > MOE_MAX_EXPERTS)
        return nva_fail("moe_route: bad counts tokens=%lld experts=%d (up to %d)", (long long)tokens, experts, MOE_MAX_EXPERTS);
    if (group_count <= 0 || experts % group_count || group_keep <= 0 || group_keep > group_count || top <= 0 ||
        top > group_keep * (experts / group_count) || softmax_top < 0 || softmax_top > 2)
        return nva_fail("moe_route: %d of %d experts in %d groups of which %d stay", top, experts, group_count, group_keep);
    if (!logits || !ids || !weights || stride < experts) return nva_fail("moe_route: a tensor is missing");
    hipLaunchKernelGGL(moe_route_kernel, dim3((unsigned)tokens), dim3(NVA_WAVE), 0, stream, logits, stride, experts, top,
                       group_count, group_keep, scale, softmax_top, bias, ids, weights);
    return nva_check_launch("moe_route");
}

// Rows of a tile of the experts' products for this many pairs (token, choice) and experts: the plan's arrays are
// sized with it.  Many rows an expert: tall tiles, so that an expert's matrix is read few times.
static int moe_tile_rows(int64_t pairs, int experts, int k, int ff) {
#if defined(NVA_BF16)
    if (k % 8 == 0 && ff % 8 == 0) return pairs >= 64 * (int64_t)experts ? 128 : 32;
#endif
    return MOE_BM;
}
NVA_EXPORT int NVA_NAME(nva_moe_tile_rows)(int64_t pairs, int experts, int k, int ff) { return moe_tile_rows(pairs, experts, k, ff); }

// ids from `experts` on are identities (x itself).  add_gate: float, one logit a token gate_stride apart, or null.
// x [tokens, k] elements; ids, weights [tokens, top]; up [E * ff, k] (gated: [E * 2 ff, k], an expert's gate rows, then
// its up rows), down [E * k, ff] elements; add [tokens, k] or null.
// Scratch: place, rows int32 [tokens * top]; tiles int32 [3 * max_tiles + 1] with max_tiles = tokens * top / MOE_BM + E
// (expert, first row, rows of every tile, then their number); hidden [tokens * top, ff], outs [tokens * top, k] elements.
NVA_EXPORT int NVA_NAME(nva_moe_experts)(const void* x, int64_t x_stride, const int32_t* ids, const float* weights,
                                         int64_t tokens, int top, int experts, int k, int ff, const void* up,
                                         const void* down, int act, int gated, const void* add, int64_t add_stride,
                                         const float* add_gate, int64_t gate_stride, int32_t* place,
                                         int32_t* rows, int32_t* tiles, int64_t max_tiles, void* hidden, void* outs, void* y,
                                         int64_t y_stride, hipStream_t stream) {
    if (tokens == 0) return 0;
    const int64_t pairs = tokens * top;
    if (tokens < 0 || top <= 0 || experts <= 0 || experts > MOE_MAX_EXPERTS || k <= 0 || ff <= 0 || pairs > 0x7fffffff)
        return nva_fail("moe_experts: bad sizes tokens=%lld top=%d experts=%d k=%d ff=%d", (long long)tokens, top, experts, k, ff);
    const int bm = moe_tile_rows(pairs, experts, k, ff);
    if (max_tiles < pairs / bm + experts || max_tiles > 0x7fffffff)
        return nva_fail("moe_experts: room for %lld tiles, %lld may be needed", (long long)max_tiles, (long long)(pairs / bm + experts));
    if (act < 0 || act > 3) return nva_fail("moe_experts: unknown activation %d", act);
    if (!x || !ids || !weights || !up || !down || !place || !rows || !tiles || !hidden || !outs || !y)
        return nva_fail("moe_experts: a tensor is missing");
    int32_t* tile_expert = tiles;
    int32_t* tile_row0 = tiles + max_tiles;
    int32_t* tile_rows = tiles + 2 * max_tiles;
    int32_t* num_tiles = tiles + 3 * max_tiles;
    hipLaunchKernelGGL(moe_plan_kernel, dim3(1), dim3(1024), 0, stream, ids, pairs, experts, bm, place, rows, tile_expert,
                       tile_row0, tile_rows, num_tiles);
    if ((ff + MOE_BN - 1) / MOE_BN > 65535 || (k + MOE_BN - 1) / MOE_BN > 65535) return nva_fail("moe_experts: too wide");
#if defined(NVA_BF16)
    if (k % 8 == 0 && ff % 8 == 0 && x_stride % 8 == 0 && nva_aligned(x, 16) && nva_aligned(up, 16) && nva_aligned(down, 16) &&
        nva_aligned(hidden, 16)) {
#define MOE_LAUNCH(BMV, WRV)                                                                                                  \
        hipLaunchKernelGGL((moe_mfma_kernel<BMV, WRV, true>), dim3((unsigned)max_tiles, (ff + 4 * WRV - 1) / (4 * WRV)),        \
                           dim3(256), 0, stream, (const __bf16*)x, x_stride, (const __bf16*)up, ff, k, rows, top, tile_expert, \
                           tile_row0, tile_rows, num_tiles, act, (__bf16*)hidden, (int64_t)ff);                                 \
        hipLaunchKernelGGL((moe_mfma_kernel<BMV, WRV, false>), dim3((unsigned)max_tiles, (k + 4 * WRV - 1) / (4 * WRV)),        \
                           dim3(256), 0, stream, (const __bf16*)hidden, (int64_t)ff, (const __bf16*)down, k, ff, rows, top,     \
                           tile_expert, tile_row0, tile_rows, num_tiles, act, (__bf16*)outs, (int64_t)k)
#define MOE_LAUNCH_GATED(BMV, WRV)                                                                                            \
        hipLaunchKernelGGL((moe_mfma_kernel<BMV, WRV, true, true>), dim3((unsigned)max_tiles, (ff + 2 * WRV - 1) / (2 * WRV)),  \
                           dim3(256), 0, stream, (const __bf16*)x, x_stride, (const __bf16*)up, ff, k, rows, top, tile_expert, \
                           tile_row0, tile_rows, num_tiles, act, (__bf16*)hidden, (int64_t)ff);                                 \
        hipLaunchKernelGGL((moe_mfma_kernel<BMV, WRV / 2, false>), dim3((unsigned)max_tiles, (k + 2 * WRV - 1) / (2 * WRV)),    \
                           dim3(256), 0, stream, (const __bf16*)hidden, (int64_t)ff, (const __bf16*)down, k, ff, rows, top,     \
                           tile_expert, tile_row0, tile_rows, num_tiles, act, (__bf16*)outs, (int64_t)k)
        if (gated) {
            if (bm == 128) { MOE_LAUNCH_GATED(128, 64); } else { MOE_LAUNCH_GATED(32, 32); }
        } else if (bm == 128) { MOE_LAUNCH(128, 32); } else { MOE_LAUNCH(32, 16); }
#undef MOE_LAUNCH_GATED
#undef MOE_LAUNCH
    } else
#endif
    {
    if (gated)
        hipLaunchKernelGGL((moe_tile_kernel<elem_t, true, true>), dim3((unsigned)max_tiles, (ff + MOE_BN - 1) / MOE_BN), dim3(256), 0,
                           stream, (const elem_t*)x, x_stride, (const elem_t*)up, ff, k, rows, top, tile_expert, tile_row0,
                           tile_rows, num_tiles, act, (elem_t*)hidden, (int64_t)ff);
    else
    hipLaunchKernelGGL((moe_tile_kernel<elem_t, true>), dim3((unsigned)max_tiles, (ff + MOE_BN - 1) / MOE_BN), dim3(256), 0,
                       stream, (const elem_t*)x, x_stride, (const elem_t*)up, ff, k, rows, top, tile_expert, tile_row0,
                       tile_rows, num_tiles, act, (elem_t*)hidden, (int64_t)ff);
    hipLaunchKernelGGL((moe_tile_kernel<elem_t, false>), dim3((unsigned)max_tiles, (k + MOE_BN - 1) / MOE_BN), dim3(256), 0,
                       stream, (const elem_t*)hidden, (int64_t)ff, (const elem_t*)down, k, ff, rows, top, tile_expert,
                       tile_row0, tile_rows, num_tiles, act, (elem_t*)outs, (int64_t)k);
    }
    for (int64_t t0 = 0; t0 < tokens; t0 += 65535) {
        const unsigned nt = (unsigned)((tokens - t0) < 65535 ? (tokens - t0) : 65535);
        hipLaunchKernelGGL((moe_combine_kernel<elem_t>), dim3((k + 255) / 256, nt), dim3(256), 0, stream, (const elem_t*)outs,
                           (int64_t)k, place + t0 * top, weights + t0 * top, top,
                           add ? (const elem_t*)add + t0 * add_stride : nullptr, add_stride,
                           add_gate ? add_gate + t0 * gate_stride : nullptr, gate_stride, (const elem_t*)x + t0 * x_stride,
                           x_stride, (elem_t*)y + t0 * y_stride, y_stride, k);
    }
    return nva_check_launch("moe_experts");
}

NVA_DEFINE_LAST_ERROR(nva_moe)
