// The gated delta rule with a decay per key channel, after its projections: a linear attention over a state
// of fixed size per request that forgets channel by channel and, at every token, is corrected towards the value
// its key should read out.
//
//   proj [T, 2 G D + H DV + H] = [q | k | v | b]        elements; G query/key heads of D, H value heads of DV
//   q, k, v <- silu(sum over the last `taps` tokens of w[c][j] * input[c])      per channel c, no bias; the inputs
//              before a portion come from the request's kept inputs (conv_state), zeros before its start
//   q <- q / sqrt(sum(q^2) + 1e-6) * D^-1/2,  k <- k / sqrt(sum(k^2) + 1e-6)    per head
//   beta = sigmoid(b)                                                            per value head
//   a = exp(-exp(a_log[h]) * softplus(decay_in[h][d] + dt_bias[h][d]))          per value head and key channel
//   per value head h, with its query/key head h / (H / G), S [D, DV]:
//       S <- diag(a) S;   u = beta (v - S^T k);   S <- S + k u^T;   o = S^T q
//   y = o / sqrt(mean(o^2) + eps) * norm_w * sigmoid(gate_in)                   per head, norm_w [DV]
//
// Everything after the projections is float whatever the element type (the convolutions' sums, the unit norms,
// softplus and the exponentials by the accurate routines, the state, the read-out, the norm and the gate); y is
// rounded once.  A token's sums run in an order that neither the portion's cut nor the batch changes: the
// recurrence goes token by token, 8 or 16 lanes holding one column of S in registers.
//
//   delta_prepare     one workgroup per (token, head of q, k or v): the convolutions, unit norms, beta and the decay,
//                     written as floats
//   delta_keep        the request's new kept inputs (its last taps - 1), after delta_prepare has read the old ones
//   delta_scan        four waves per (request, head, 16 or 32 columns of S), 16 or 8 lanes a column: the recurrence over the
//                     portion's tokens, the tokens' q, k, a and beta staged in LDS a batch at a time in two buffers,
//                     v asked for a batch ahead
//   delta_finish      one wave per (token, head): the norm and the gate
#include "common.h"

#define DELTA_MAX_TAPS 16
#define DELTA_BATCH 8            // tokens whose q, k and a lie in LDS at a time
#define DELTA_THREADS 256        // of the recurrence's workgroup: four waves
#define DELTA_MAX_DIM 256        // key channels of a head at most
#define DELTA_PREPARE_THREADS 128

// One workgroup per (token, unit); a unit is a query head, a key head, or a value head with its decays and beta.
// Rows of qn, kn and decay are DP = dim rounded up to 4 floats apart, the padding zero.
template <typename T>
__global__ void __launch_bounds__(DELTA_PREPARE_THREADS)
delta_prepare_kernel(const T* __restrict__ proj, int64_t stride, const float* __restrict__ decay_in,
                     const T* __restrict__ conv_w, const float* __restrict__ dt_bias, const float* __restrict__ a_log,
                     const float* __restrict__ conv_state, const int32_t* __restrict__ token_seq,
                     const int32_t* __restrict__ cu_seqlens_q, const int32_t* __restrict__ seq_starts,
                     const int32_t* __restrict__ state_slots, int heads, int kv_heads, int dim, int vdim, int taps,
                     float* __restrict__ qn, float* __restrict__ kn, float* __restrict__ vf, float* __restrict__ decay,
                     float* __restrict__ beta) {
    __shared__ float sum_s[16];
    const int64_t t = blockIdx.x;
    const int unit = blockIdx.y;
    const int seq = token_seq[t];
    const int begin = cu_seqlens_q[seq];
    const int local = (int)t - begin;                                   // the token's place in its portion
    const bool has_past = seq_starts[seq] > 0;
    const int slot = state_slots[seq];
    const int qk = kv_heads * dim, vv = heads * vdim, channels = 2 * qk + vv;
    const int dp = (dim + 3) & ~3;
    const int tid = threadIdx.x;
    auto conv_silu = [&](int c) __attribute__((always_inline)) {
        float sum = 0.f;
        for (int j = 0; j < taps; ++j) {
            const int src = local - (taps - 1) + j;                     // < 0: before the portion
            float x = 0.f;
            if (src >= 0) x = to_float(proj[(int64_t)(begin + src) * stride + c]);
            else if (has_past) x = conv_state[((int64_t)slot * channels + c) * (taps - 1) + (taps - 1 + src)];
            sum += to_float(conv_w[(int64_t)c * taps + j]) * x;
        }
        return sum / (1.f + expf(-sum));
    };
    if (unit < 2 * kv_heads) {
        // a query or key head: its channels are unit * dim .. + dim of the row; the unit norm over the head
        constexpr int PER = (DELTA_MAX_DIM + DELTA_PREPARE_THREADS - 1) / DELTA_PREPARE_THREADS;
        float y[PER];
        float ss = 0.f;
#pragma unroll
        for (int i = 0; i < PER; ++i) {
            const int d = i * DELTA_PREPARE_THREADS + tid;
            y[i] = d < dim ? conv_silu(unit * dim + d) : 0.f;
            ss += y[i] * y[i];
        }
        ss = block_sum(ss, sum_s);
        const bool is_q = unit < kv_heads;
        float scale = 1.f / sqrtf(ss + 1e-6f);
        if (is_q) scale *= 1.f / sqrtf((float)dim);
        float* dst = (is_q ? qn + (t * kv_heads + unit) * dp : kn + (t * kv_heads + (unit - kv_heads)) * dp);
#pragma unroll
        for (int i = 0; i < PER; ++i) {
            const int d = i * DELTA_PREPARE_THREADS + tid;
            if (d < dp) dst[d] = y[i] * scale;                          // (zeros in the padding)
        }
        return;
    }
    const int h = unit - 2 * kv_heads;
    for (int d = tid; d < vdim; d += DELTA_PREPARE_THREADS) vf[t * vv + h * vdim + d] = conv_silu(2 * qk + h * vdim + d);
    const float rate = expf(a_log[h]);
    for (int d = tid; d < dp; d += DELTA_PREPARE_THREADS) {
        float a = 0.f;
        if (d < dim) {
            const float z = decay_in[t * (int64_t)(heads * dim) + h * dim + d] + dt_bias[h * dim + d];
            const float step = z > 20.f ? z : log1pf(expf(z));
            a = expf(-rate * step);
        }
        decay[(t * heads + h) * dp + d] = a;
    }
    if (tid == 0) beta[t * heads + h] = 1.f / (1.f + expf(-to_float(proj[t * stride + channels + h])));
}

// One thread a (request, channel): the request's last taps - 1 inputs, from the portion where it is long enough,
// else from what was kept before (zeros at a request's start).
template <typename T>
__global__ void __launch_bounds__(256)
delta_keep_kernel(const T* __restrict__ proj, int64_t stride, float* __restrict__ conv_state,
                  const int32_t* __restrict__ cu_seqlens_q, const int32_t* __restrict__ seq_starts,
                  const int32_t* __restrict__ state_slots, int channels, int taps) {
    const int seq = blockIdx.y;
    const int c = blockIdx.x * blockDim.x + threadIdx.x;
    if (c >= channels) return;
    const int begin = cu_seqlens_q[seq], n = cu_seqlens_q[seq + 1] - begin;
    const bool has_past = seq_starts[seq] > 0;
    float* kept = conv_state + ((int64_t)state_slots[seq] * channels + c) * (taps - 1);
    float fresh[DELTA_MAX_TAPS];
    for (int i = 0; i < taps - 1; ++i) {
        const int src = n - (taps - 1) + i;
        fresh[i] = src >= 0 ? to_float(proj[(int64_t)(begin + src) * stride + c]) : has_past ? kept[taps - 1 + src] : 0.f;
    }
    for (int i = 0; i < taps - 1; ++i) kept[i] = fresh[i];
}

// The sum of x over the L = 8 or 16 neighbouring lanes that share a column of S: two exchanges inside the quads, then
// one between the two quads of every 8 lanes, which by then hold one value each, then one between the two eights.
template <int L>
__device__ __forceinline__ float delta_sum_lanes(float x) {
    x += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(x), 0xB1, 0xF, 0xF, true));     // lanes 1 0 3 2
    x += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(x), 0x4E, 0xF, 0xF, true));     // lanes 2 3 0 1
    x += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(x), 0x141, 0xF, 0xF, true));    // lanes 7 .. 0 of each 8
    if (L == 16) x += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(x), 0x140, 0xF, 0xF, true));   // 15 .. 0 of each 16
    return x;
}

// One workgroup of four waves per (request, head, 256 / L columns of S).  A column's DMAX rows (rows beyond D: zeros,
// with q, k and a staged as zeros) lie in L neighbouring lanes: lane r of them holds the rows 4 (r + L j) .. + 3 for
// j < DMAX / (4 L), so that the L lanes read consecutive floats of a staged row at a time.  Per token, in this order:
// S <- a S, u = beta (v - S^T k), S <- S + k u, o = S^T q; each of the two sums over the rows runs as four chains a
// lane and then over the L lanes, in an order that depends on D alone.  The tokens' q, k, a and beta go through LDS,
// a batch at a time in two buffers: the next batch is asked for before this one's sums and stored after them.
template <int DMAX, int L>
__global__ void __launch_bounds__(DELTA_THREADS)
delta_scan_kernel(const float* __restrict__ qn, const float* __restrict__ kn, const float* __restrict__ vf,
                  const float* __restrict__ decay, const float* __restrict__ beta, float* __restrict__ o_raw,
                  float* __restrict__ state, const int32_t* __restrict__ cu_seqlens_q,
                  const int32_t* __restrict__ seq_starts, const int32_t* __restrict__ state_slots, int heads,
                  int kv_heads, int dim, int vdim) {
    constexpr int R4 = DMAX / (4 * L);                                  // float4s of rows a lane holds
    constexpr int COLS = DELTA_THREADS / L;                             // columns of S a workgroup holds
    constexpr int ROW4 = DMAX / 4;                                      // float4s of a staged row
    constexpr int STAGED4 = 3 * DELTA_BATCH * ROW4;                     // q, k, a of a batch
    constexpr int NP = (STAGED4 + DELTA_THREADS - 1) / DELTA_THREADS;
    __shared__ float4 qka_s[2][3][DELTA_BATCH][ROW4];
    __shared__ float beta_s[2][DELTA_BATCH];
    const int seq = blockIdx.x, h = blockIdx.y, tid = threadIdx.x;
    const int r = tid % L;
    const int col = blockIdx.z * COLS + tid / L;
    const bool live = col < vdim;
    const int g = h / (heads / kv_heads);
    const int begin = cu_seqlens_q[seq], n = cu_seqlens_q[seq + 1] - begin;
    const int vv = heads * vdim;
    const int dp = (dim + 3) & ~3, dp4 = dp / 4;
    float* S_g = state + (((int64_t)state_slots[seq] * heads + h) * dim) * vdim + col;
    const bool has_past = seq_starts[seq] > 0;
    float S[4 * R4];
#pragma unroll
    for (int j = 0; j < R4; ++j)
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            const int row = 4 * (r + L * j) + e;
            S[4 * j + e] = has_past && live && row < dim ? S_g[(int64_t)row * vdim] : 0.f;
        }

    // a batch's q, k, a (and beta) from global memory into registers, and from there into one of the two buffers
    float4 pre[NP];
    float pre_beta = 0.f;
    auto ask = [&](int t0) __attribute__((always_inline)) {
        const int nb = min(DELTA_BATCH, n - t0);
#pragma unroll
        for (int i = 0; i < NP; ++i) {
            const int e = i * DELTA_THREADS + tid;
            const int which = e / (DELTA_BATCH * ROW4), b = (e / ROW4) % DELTA_BATCH, d4 = e % ROW4;
            float4 x = make_float4(0.f, 0.f, 0.f, 0.f);
            if (e < STAGED4 && b < nb && d4 < dp4) {
                const int64_t tok = begin + t0 + b;
                const float* row = which == 0 ? qn + (tok * kv_heads + g) * dp : which == 1 ? kn + (tok * kv_heads + g) * dp
                                                                                             : decay + (tok * heads + h) * dp;
                x = *reinterpret_cast<const float4*>(row + 4 * d4);
            }
            pre[i] = x;
        }
        pre_beta = tid < nb ? beta[(int64_t)(begin + t0 + tid) * heads + h] : 0.f;
    };
    auto put = [&](int buf) __attribute__((always_inline)) {
        float4* flat = &qka_s[buf][0][0][0];
#pragma unroll
        for (int i = 0; i < NP; ++i) {
            const int e = i * DELTA_THREADS + tid;
            if (e < STAGED4) flat[e] = pre[i];
        }
        if (tid < DELTA_BATCH) beta_s[buf][tid] = pre_beta;
    };
    float v_next[DELTA_BATCH];
#pragma unroll
    for (int b = 0; b < DELTA_BATCH; ++b) v_next[b] = live && b < n ? vf[(int64_t)(begin + b) * vv + h * vdim + col] : 0.f;
    ask(0);
    put(0);
    __syncthreads();
    int buf = 0;
    for (int t0 = 0; t0 < n; t0 += DELTA_BATCH, buf ^= 1) {
        const int nb = min(DELTA_BATCH, n - t0);
        const bool more = t0 + DELTA_BATCH < n;
        if (more) ask(t0 + DELTA_BATCH);
        float v_now[DELTA_BATCH];
#pragma unroll
        for (int b = 0; b < DELTA_BATCH; ++b) {
            v_now[b] = v_next[b];
            const int tn = t0 + DELTA_BATCH + b;                        // the batch after: asked for now
            v_next[b] = live && tn < n ? vf[(int64_t)(begin + tn) * vv + h * vdim + col] : 0.f;
        }
        // a token's q, k, a and beta are read from LDS while the token before it is summed
        float4 a_c[R4], k_c[R4], q_c[R4];
        float beta_c;
        auto fetch = [&](int b, float4* a, float4* k, float4* q, float& be) __attribute__((always_inline)) {
#pragma unroll
            for (int j = 0; j < R4; ++j) {
                a[j] = qka_s[buf][2][b][r + L * j];
                k[j] = qka_s[buf][1][b][r + L * j];
                q[j] = qka_s[buf][0][b][r + L * j];
            }
            be = beta_s[buf][b];
        };
        fetch(0, a_c, k_c, q_c, beta_c);
#pragma unroll
        for (int b = 0; b < DELTA_BATCH; ++b) {
            if (b >= nb) break;
            float4 a_n[R4], k_n[R4], q_n[R4];
            float beta_n = 0.f;
            if (b + 1 < DELTA_BATCH) fetch(b + 1, a_n, k_n, q_n, beta_n);      // (rows past the batch's last hold zeros)
            float d0 = 0.f, d1 = 0.f, d2 = 0.f, d3 = 0.f;
#pragma unroll
            for (int j = 0; j < R4; ++j) {
                const float4 a = a_c[j], k = k_c[j];
                S[4 * j] *= a.x; S[4 * j + 1] *= a.y; S[4 * j + 2] *= a.z; S[4 * j + 3] *= a.w;
                d0 += S[4 * j] * k.x; d1 += S[4 * j + 1] * k.y; d2 += S[4 * j + 2] * k.z; d3 += S[4 * j + 3] * k.w;
            }
            const float u = beta_c * (v_now[b] - delta_sum_lanes<L>((d0 + d1) + (d2 + d3)));
            float o0 = 0.f, o1 = 0.f, o2 = 0.f, o3 = 0.f;
#pragma unroll
            for (int j = 0; j < R4; ++j) {
                const float4 k = k_c[j], q = q_c[j];
                S[4 * j] += k.x * u; S[4 * j + 1] += k.y * u; S[4 * j + 2] += k.z * u; S[4 * j + 3] += k.w * u;
                o0 += S[4 * j] * q.x; o1 += S[4 * j + 1] * q.y; o2 += S[4 * j + 2] * q.z; o3 += S[4 * j + 3] * q.w;
            }
            const float o = delta_sum_lanes<L>((o0 + o1) + (o2 + o3));
            if (live && r == 0) o_raw[(int64_t)(begin + t0 + b) * vv + h * vdim + col] = o;
            if (b + 1 < DELTA_BATCH) {
#pragma unroll
                for (int j = 0; j < R4; ++j) a_c[j] = a_n[j], k_c[j] = k_n[j], q_c[j] = q_n[j];
                beta_c = beta_n;
            }
        }
        if (more) put(buf ^ 1);
        __syncthreads();                                                // the next batch is in; this one is done with
    }
    if (live) {
#pragma unroll
        for (int j = 0; j < R4; ++j)
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                const int row = 4 * (r + L * j) + e;
                if (row < dim) S_g[(int64_t)row * vdim] = S[4 * j + e];
            }
    }
}

template <typename T>
__global__ void __launch_bounds__(NVA_WAVE)
delta_finish_kernel(const float* __restrict__ o_raw, const T* __restrict__ gate, int64_t gate_stride,
                    const float* __restrict__ norm_w, float eps, T* __restrict__ out, int64_t out_stride, int heads,
                    int vdim) {
    const int64_t t = blockIdx.x;
    const int h = blockIdx.y, lane = threadIdx.x;
    const float* o = o_raw + (t * heads + h) * (int64_t)vdim;
    float ss = 0.f;
    for (int d = lane; d < vdim; d += NVA_WAVE) ss += o[d] * o[d];
    ss = wave_sum(ss);
    const float scale = 1.f / sqrtf(ss / (float)vdim + eps);
    for (int d = lane; d < vdim; d += NVA_WAVE) {
        const float gt = 1.f / (1.f + expf(-to_float(gate[t * gate_stride + h * vdim + d])));
        out[t * out_stride + h * vdim + d] = from_float<T>(o[d] * scale * norm_w[d] * gt);
    }
}

// proj: elements [tokens, 2 G D + H DV + H], rows `stride` apart.  decay_in: float [tokens, H D].  gate_in: elements
// [tokens, H DV], rows gate_stride apart.  conv_w: elements [2 G D + H DV, taps].  dt_bias float [H D], a_log float [H],
// norm_w float [DV].  conv_state float [slots, 2 G D + H DV, taps - 1], s_state float [slots, H, D, DV]: a request's
// rows by state_slots, taken as zero where seq_starts is 0.  scratch: float [tokens * ((2 G + H) DP + 2 H DV + H)], DP = D rounded up to 4, 16-byte aligned.
// The step's requests by cu_seqlens_q [seqs + 1]; token_seq [tokens].  out: elements [tokens, H DV].
NVA_EXPORT int NVA_NAME(nva_channel_delta)(const void* proj, int64_t stride, const float* decay_in, const void* gate_in,
                                           int64_t gate_stride, float* scratch, void* out, int64_t out_stride,
                                           float* s_state, float* conv_state, const int32_t* token_seq,
                                           const int32_t* cu_seqlens_q, const int32_t* seq_starts,
                                           const int32_t* state_slots, int64_t seqs, int64_t tokens, int heads,
                                           int kv_heads, int dim, int vdim, int taps, const void* conv_w,
                                           const float* dt_bias, const float* a_log, const float* norm_w, float eps,
                                           hipStream_t stream) {
    if (tokens == 0) return 0;
    if (tokens < 0 || tokens > 0x7fffffff || seqs <= 0 || seqs > 65535 * 32)
        return nva_fail("channel_delta: bad counts tokens=%lld requests=%lld", (long long)tokens, (long long)seqs);
    if (heads <= 0 || kv_heads <= 0 || heads % kv_heads || heads > 65535 || dim <= 0 || vdim <= 0)
        return nva_fail("channel_delta: bad sizes heads=%d kv_heads=%d dim=%d vdim=%d", heads, kv_heads, dim, vdim);
    if (dim > DELTA_MAX_DIM) return nva_fail("channel_delta: a head of %d key channels (up to %d)", dim, DELTA_MAX_DIM);
    if (taps < 1 || taps > DELTA_MAX_TAPS) return nva_fail("channel_delta: %d taps (1 to %d)", taps, DELTA_MAX_TAPS);
    const int qk = kv_heads * dim, vv = heads * vdim, channels = 2 * qk + vv;
    if (!proj || stride < channels + heads || !decay_in || !gate_in || gate_stride < vv || !scratch || !out || out_stride < vv ||
        !s_state || (taps > 1 && !conv_state) || !token_seq || !cu_seqlens_q || !seq_starts || !state_slots || !conv_w ||
        !dt_bias || !a_log || !norm_w)
        return nva_fail("channel_delta: a tensor is missing or too narrow");
    if (2 * (int64_t)kv_heads + heads > 65535) return nva_fail("channel_delta: %d heads", heads);
    // scratch: q, k and the decays in rows of dim rounded up to 4 floats, then v, the read-outs and beta
    const int dp = (dim + 3) & ~3;
    float* qn = scratch;
    float* kn = qn + tokens * kv_heads * dp;
    float* decay = kn + tokens * kv_heads * dp;
    float* vf = decay + tokens * (int64_t)heads * dp;
    float* o_raw = vf + tokens * vv;
    float* beta = o_raw + tokens * vv;
    if ((uintptr_t)scratch % 16) return nva_fail("channel_delta: the scratch memory must be 16-byte aligned");
    hipLaunchKernelGGL(delta_prepare_kernel<elem_t>, dim3((unsigned)tokens, (unsigned)(2 * kv_heads + heads)),
                       dim3(DELTA_PREPARE_THREADS), 0, stream, (const elem_t*)proj, stride, decay_in, (const elem_t*)conv_w, dt_bias,
                       a_log, conv_state, token_seq, cu_seqlens_q, seq_starts, state_slots, heads, kv_heads, dim, vdim, taps, qn, kn,
                       vf, decay, beta);
    if (taps > 1) {
        if (seqs > 65535) return nva_fail("channel_delta: %lld requests a step", (long long)seqs);
        hipLaunchKernelGGL(delta_keep_kernel<elem_t>, dim3((channels + 255) / 256, (unsigned)seqs), dim3(256), 0, stream,
                           (const elem_t*)proj, stride, conv_state, cu_seqlens_q, seq_starts, state_slots, channels, taps);
    }
    {
        // 16 lanes a column where a head has rows for them (twice the waves, half the sums a lane), else 8
#define DELTA_SCAN(DM, LL)                                                                                                \
        hipLaunchKernelGGL((delta_scan_kernel<DM, LL>), dim3((unsigned)seqs, (unsigned)heads, (vdim + DELTA_THREADS / LL - 1) / (DELTA_THREADS / LL)), \
                           dim3(DELTA_THREADS), 0, stream, qn, kn, vf, decay, beta, o_raw, s_state, cu_seqlens_q, seq_starts,   \
                           state_slots, heads, kv_heads, dim, vdim)
        if (dim <= 32) DELTA_SCAN(32, 8); else if (dim <= 64) DELTA_SCAN(64, 16); else if (dim <= 128) DELTA_SCAN(128, 16); else DELTA_SCAN(256, 16);
#undef DELTA_SCAN
    }
    hipLaunchKernelGGL(delta_finish_kernel<elem_t>, dim3((unsigned)tokens, (unsigned)heads), dim3(NVA_WAVE), 0, stream, o_raw,
                       (const elem_t*)gate_in, gate_stride, norm_w, eps, (elem_t*)out, out_stride, heads, vdim);
    return nva_check_launch("channel_delta");
}

NVA_DEFINE_LAST_ERROR(nva_delta)
