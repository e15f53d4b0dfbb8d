// Gating of a feed-forward: out[t, i] = act(x[t, i]) * x[t, inner + i].  SwiGLU is act = silu,
// silu(g) = g * sigmoid(g) (nanovllm/layers/activation.py:8-11); the other activations are relu and
// the tanh form of gelu, 0.5 g (1 + tanh(sqrt(2/pi) (g + 0.044715 g^3))).  Computed in float and
// rounded once.
#include "common.h"

#define NVA_ACT_SILU 0
#define NVA_ACT_RELU 1
#define NVA_ACT_GELU_TANH 2

template <int ACT> __device__ __forceinline__ float nva_act(float g) {
    if (ACT == NVA_ACT_RELU) return fmaxf(g, 0.f);
    if (ACT == NVA_ACT_GELU_TANH) return 0.5f * g * (1.f + tanhf(0.7978845608028654f * (g + 0.044715f * g * g * g)));
    return g / (1.f + nva_exp(-g));
}

template <typename T, bool VEC, int ACT>
__global__ void __launch_bounds__(256)
act_mul_kernel(const T* __restrict__ x, int64_t x_stride, T* __restrict__ out, int64_t out_stride, int inner) {
    const int64_t row = blockIdx.y;
    const T* gate = x + row * x_stride;
    const T* up = gate + inner;
    T* o = out + row * out_stride;
    if (VEC) {
        const int i = (blockIdx.x * blockDim.x + threadIdx.x) * 8;
        if (i >= inner) return;
        float g[8], u[8];
        load8(gate + i, g);
        load8(up + i, u);
#pragma unroll
        for (int j = 0; j < 8; ++j) g[j] = nva_act<ACT>(g[j]) * u[j];
        store8(o + i, g);
    } else {
        const int i = blockIdx.x * blockDim.x + threadIdx.x;
        if (i >= inner) return;
        const float g = to_float(gate[i]);
        o[i] = from_float<T>(nva_act<ACT>(g) * to_float(up[i]));
    }
}

template <int ACT>
static int launch_act_mul(const void* x, int64_t x_stride, void* out, int64_t out_stride, int64_t rows, int inner,
                          hipStream_t stream) {
    if (rows == 0) return 0;
    if (rows < 0 || rows > 65535LL * 65535LL || inner <= 0)
        return nva_fail("act_mul: bad shape rows=%lld inner=%d", (long long)rows, inner);
    const size_t vb = 8 * sizeof(elem_t);
    const bool vec = inner % 8 == 0 && x_stride % 8 == 0 && out_stride % 8 == 0 && nva_aligned(x, vb) &&
                     nva_aligned(out, vb);
    // grid.y is limited to 65535 rows per launch
    const elem_t* xp = (const elem_t*)x;
    elem_t* op = (elem_t*)out;
    for (int64_t r0 = 0; r0 < rows; r0 += 65535) {
        const unsigned nr = (unsigned)((rows - r0) < 65535 ? (rows - r0) : 65535);
        if (vec) {
            dim3 grid((inner / 8 + 255) / 256, nr);
            hipLaunchKernelGGL((act_mul_kernel<elem_t, true, ACT>), grid, dim3(256), 0, stream, xp + r0 * x_stride,
                               x_stride, op + r0 * out_stride, out_stride, inner);
        } else {
            dim3 grid((inner + 255) / 256, nr);
            hipLaunchKernelGGL((act_mul_kernel<elem_t, false, ACT>), grid, dim3(256), 0, stream, xp + r0 * x_stride,
                               x_stride, op + r0 * out_stride, out_stride, inner);
        }
    }
    return nva_check_launch("act_mul");
}

// act: 0 silu, 1 relu, 2 gelu (tanh form)
NVA_EXPORT int NVA_NAME(nva_act_mul)(const void* x, int64_t x_stride, void* out, int64_t out_stride,
                                     int64_t rows, int inner, int act, hipStream_t stream) {
    switch (act) {
        case NVA_ACT_SILU: return launch_act_mul<NVA_ACT_SILU>(x, x_stride, out, out_stride, rows, inner, stream);
        case NVA_ACT_RELU: return launch_act_mul<NVA_ACT_RELU>(x, x_stride, out, out_stride, rows, inner, stream);
        case NVA_ACT_GELU_TANH: return launch_act_mul<NVA_ACT_GELU_TANH>(x, x_stride, out, out_stride, rows, inner, stream);
    }
    return nva_fail("act_mul: unknown activation %d", act);
}

NVA_EXPORT int NVA_NAME(nva_silu_mul)(const void* x, int64_t x_stride, void* out, int64_t out_stride,
                                      int64_t rows, int inner, hipStream_t stream) {
    return launch_act_mul<NVA_ACT_SILU>(x, x_stride, out, out_stride, rows, inner, stream);
}

// An activation without a gate: out[t, i] = act(x[t, i]); act by the codes of nva_gate_act (3: relu squared).
template <typename T>
__global__ void __launch_bounds__(256)
act_kernel(const T* __restrict__ x, int64_t x_stride, T* __restrict__ out, int64_t out_stride, int64_t rows, int width, int act) {
    const int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (idx >= rows * width) return;
    const int64_t r = idx / width;
    const int i = (int)(idx % width);
    out[r * out_stride + i] = from_float<T>(nva_gate_act(act, to_float(x[r * x_stride + i])));
}

NVA_EXPORT int NVA_NAME(nva_act)(const void* x, int64_t x_stride, void* out, int64_t out_stride, int64_t rows, int width,
                                 int act, hipStream_t stream) {
    if (rows == 0) return 0;
    if (rows < 0 || width <= 0 || act < 0 || act > 3) return nva_fail("act: bad shape rows=%lld width=%d or activation %d", (long long)rows, width, act);
    const int64_t total = rows * width;
    if ((total + 255) / 256 > 0x7fffffff) return nva_fail("act: too many entries");
    hipLaunchKernelGGL((act_kernel<elem_t>), dim3((unsigned)((total + 255) / 256)), dim3(256), 0, stream, (const elem_t*)x,
                       x_stride, (elem_t*)out, out_stride, rows, width, act);
    return nva_check_launch("act");
}

// A gate on finished outputs: out[t, i] = x[t, i] * sigmoid(g[t, i]), in float, rounded once (out may be x).
template <typename T>
__global__ void __launch_bounds__(256)
sigmoid_mul_kernel(const T* __restrict__ x, int64_t x_stride, const T* __restrict__ g, int64_t g_stride, T* __restrict__ out,
                   int64_t out_stride, int64_t rows, int width) {
    const int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (idx >= rows * width) return;
    const int64_t r = idx / width;
    const int i = (int)(idx % width);
    const float gate = 1.f / (1.f + nva_exp(-to_float(g[r * g_stride + i])));
    out[r * out_stride + i] = from_float<T>(to_float(x[r * x_stride + i]) * gate);
}

NVA_EXPORT int NVA_NAME(nva_sigmoid_mul)(const void* x, int64_t x_stride, const void* g, int64_t g_stride, void* out,
                                         int64_t out_stride, int64_t rows, int width, hipStream_t stream) {
    if (rows == 0) return 0;
    if (rows < 0 || width <= 0 || !x || !g || !out) return nva_fail("sigmoid_mul: bad shape rows=%lld width=%d", (long long)rows, width);
    const int64_t total = rows * width;
    if ((total + 255) / 256 > 0x7fffffff) return nva_fail("sigmoid_mul: too many entries");
    hipLaunchKernelGGL((sigmoid_mul_kernel<elem_t>), dim3((unsigned)((total + 255) / 256)), dim3(256), 0, stream,
                       (const elem_t*)x, x_stride, (const elem_t*)g, g_stride, (elem_t*)out, out_stride, rows, width);
    return nva_check_launch("sigmoid_mul");
}

NVA_DEFINE_LAST_ERROR(nva_activation)
