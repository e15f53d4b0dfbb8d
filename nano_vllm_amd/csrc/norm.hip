// RMS normalisation over the last dimension, alone and fused with the residual sum.
//
//   rms_norm:      y = cast(x * rsqrt(mean(x^2) + eps)) * w
//   add_rms_norm:  s = x + r;  r <- cast(s);  y = cast(s * rsqrt(mean(s^2) + eps)) * w
//
// as nanovllm/layers/layernorm.py:16-40 computes them: square, mean, rsqrt and scaling in
// float, the cast to the element type before the product with the weight, and the variance
// of the unrounded sum.  One block per row.  The weight is stored as elements or as float.
//
// x may also be given as float partial sums [splits][rows][width] of a product whose k range
// was split over workgroups (gemm_skinny.hip): the kernel then adds the partials in the order of
// the splits, adds the optional bias and rounds to the element type, which is what the product's
// own finishing pass would have stored.
#include "common.h"

#define NORM_KEEP 2

template <typename T, bool ADD, bool VEC>
__global__ void __launch_bounds__(512)
rms_norm_kernel(const T* x, int64_t x_stride, PartialInput part, T* residual, int64_t r_stride,
                const void* __restrict__ weight, int w_is_f32, T* y, int64_t y_stride,
                int width, float eps) {
    __shared__ float scratch[16];
    const int64_t row = blockIdx.x;
    const T* xr = part.sums ? nullptr : x + row * x_stride;
    T* rr = ADD ? residual + row * r_stride : nullptr;
    T* yr = y + row * y_stride;
    const T* w_e = static_cast<const T*>(weight);
    const float* w_f = static_cast<const float*>(weight);

    float ss = 0.f;
    if (VEC) {
        // The first NORM_KEEP vectors of 8 per thread stay in registers between the two passes; what
        // a wider row has beyond them (width > threads * 8 * NORM_KEEP) is read again.
        float kept[NORM_KEEP][8];
#pragma unroll
        for (int v = 0; v < NORM_KEEP; ++v) {
            const int i = (v * blockDim.x + threadIdx.x) * 8;
            if (i < width) {
                float a[8];
                if (part.sums) partial_value8<T>(part, row, width, i, a); else load8(xr + i, a);
                if (ADD) {
                    float b[8];
                    load8(rr + i, b);
#pragma unroll
                    for (int j = 0; j < 8; ++j) a[j] += b[j];
                }
#pragma unroll
                for (int j = 0; j < 8; ++j) {
                    ss += a[j] * a[j];
                    kept[v][j] = a[j];
                }
            }
        }
        for (int i = (NORM_KEEP * blockDim.x + threadIdx.x) * 8; i < width; i += blockDim.x * 8) {
            float a[8];
            if (part.sums) partial_value8<T>(part, row, width, i, a); else load8(xr + i, a);
            if (ADD) {
                float b[8];
                load8(rr + i, b);
#pragma unroll
                for (int j = 0; j < 8; ++j) a[j] += b[j];
            }
#pragma unroll
            for (int j = 0; j < 8; ++j) ss += a[j] * a[j];
        }
        ss = block_sum(ss, scratch);
        const float scale = rsqrtf(ss / (float)width + eps);
#pragma unroll
        for (int v = 0; v < NORM_KEEP; ++v) {
            const int i = (v * blockDim.x + threadIdx.x) * 8;
            if (i < width) {
                float a[8], w[8];
#pragma unroll
                for (int j = 0; j < 8; ++j) a[j] = kept[v][j];
                if (ADD) store8(rr + i, a);
                if (w_is_f32) load8(w_f + i, w); else load8(w_e + i, w);
#pragma unroll
                for (int j = 0; j < 8; ++j) a[j] = round_through<T>(a[j] * scale) * w[j];
                store8(yr + i, a);
            }
        }
        for (int i = (NORM_KEEP * blockDim.x + threadIdx.x) * 8; i < width; i += blockDim.x * 8) {
            float a[8], w[8];
            if (part.sums) partial_value8<T>(part, row, width, i, a); else load8(xr + i, a);
            if (ADD) {
                float b[8];
                load8(rr + i, b);
#pragma unroll
                for (int j = 0; j < 8; ++j) a[j] += b[j];
                store8(rr + i, a);
            }
            if (w_is_f32) load8(w_f + i, w); else load8(w_e + i, w);
#pragma unroll
            for (int j = 0; j < 8; ++j) a[j] = round_through<T>(a[j] * scale) * w[j];
            store8(yr + i, a);
        }
    } else {
        for (int i = threadIdx.x; i < width; i += blockDim.x) {
            float a = part.sums ? partial_value<T>(part, row, width, i) : to_float(xr[i]);
            if (ADD) a += to_float(rr[i]);
            ss += a * a;
        }
        ss = block_sum(ss, scratch);
        const float scale = rsqrtf(ss / (float)width + eps);
        for (int i = threadIdx.x; i < width; i += blockDim.x) {
            float a = part.sums ? partial_value<T>(part, row, width, i) : to_float(xr[i]);
            if (ADD) {
                a += to_float(rr[i]);
                rr[i] = from_float<T>(a);
            }
            const float w = w_is_f32 ? w_f[i] : to_float(w_e[i]);
            yr[i] = from_float<T>(round_through<T>(a * scale) * w);
        }
    }
}

template <bool ADD>
static int launch(const elem_t* x, int64_t x_stride, PartialInput part, elem_t* residual, int64_t r_stride,
                  const void* weight, int w_is_f32, elem_t* y, int64_t y_stride,
                  int64_t rows, int width, float eps, hipStream_t stream) {
    if (rows == 0) return 0;
    if (rows < 0 || width <= 0) return nva_fail("rms_norm: bad shape rows=%lld width=%d", (long long)rows, width);
    if (rows > 0x7fffffff) return nva_fail("rms_norm: too many rows (%lld)", (long long)rows);
    const size_t vec_bytes = 8 * sizeof(elem_t);
    if (part.sums && (part.splits <= 0 || part.split_stride < rows * (int64_t)width))
        return nva_fail("rms_norm: bad partial sums (splits %d)", part.splits);
    const bool x_vec = part.sums ? (nva_aligned(part.sums, 16) && (!part.bias || nva_aligned(part.bias, vec_bytes)) &&
                                    part.split_stride % 4 == 0)
                                 : (x_stride % 8 == 0 && nva_aligned(x, vec_bytes));
    const bool vec = width % 8 == 0 && x_vec && y_stride % 8 == 0 && r_stride % 8 == 0 &&
                     nva_aligned(y, vec_bytes) &&
                     (!ADD || nva_aligned(residual, vec_bytes)) &&
                     nva_aligned(weight, w_is_f32 ? 32 : vec_bytes);
    // few wide rows: one vector of 8 per thread, so that a row of partial sums is read in one round of loads
    const int threads = width >= 4096 && rows <= 256 ? 512 : width >= 2048 ? 256 : (width >= 512 ? 128 : 64);
    if (vec)
        hipLaunchKernelGGL((rms_norm_kernel<elem_t, ADD, true>), dim3((unsigned)rows), dim3(threads), 0, stream,
                           x, x_stride, part, residual, r_stride, weight, w_is_f32, y, y_stride, width, eps);
    else
        hipLaunchKernelGGL((rms_norm_kernel<elem_t, ADD, false>), dim3((unsigned)rows), dim3(threads), 0, stream,
                           x, x_stride, part, residual, r_stride, weight, w_is_f32, y, y_stride, width, eps);
    return nva_check_launch("rms_norm");
}

// y may be x.  Strides are in elements between rows.
NVA_EXPORT int NVA_NAME(nva_rms_norm)(const void* x, int64_t x_stride, const void* weight, int w_is_f32,
                                      void* y, int64_t y_stride, int64_t rows, int width, float eps,
                                      hipStream_t stream) {
    return launch<false>((const elem_t*)x, x_stride, PartialInput{nullptr, 0, 0, nullptr}, nullptr, 0, weight, w_is_f32,
                         (elem_t*)y, y_stride, rows, width, eps, stream);
}

// residual is updated in place with the sum; y may be x.
NVA_EXPORT int NVA_NAME(nva_add_rms_norm)(const void* x, int64_t x_stride, void* residual, int64_t r_stride,
                                          const void* weight, int w_is_f32, void* y, int64_t y_stride,
                                          int64_t rows, int width, float eps, hipStream_t stream) {
    return launch<true>((const elem_t*)x, x_stride, PartialInput{nullptr, 0, 0, nullptr}, (elem_t*)residual, r_stride,
                        weight, w_is_f32, (elem_t*)y, y_stride, rows, width, eps, stream);
}

// As nva_add_rms_norm with x = round(sum over splits of sums[s][row][:] (+ bias)); residual may be
// null, then there is no residual sum (the first layer's norm).
NVA_EXPORT int NVA_NAME(nva_rms_norm_of_partials)(const float* sums, int splits, int64_t split_stride, const void* bias,
                                                  void* residual, int64_t r_stride, const void* weight, int w_is_f32,
                                                  void* y, int64_t y_stride, int64_t rows, int width, float eps,
                                                  hipStream_t stream) {
    const PartialInput part{sums, splits, split_stride, bias};
    if (!sums) return nva_fail("rms_norm_of_partials: no partial sums");
    if (residual)
        return launch<true>(nullptr, 0, part, (elem_t*)residual, r_stride, weight, w_is_f32, (elem_t*)y, y_stride, rows,
                            width, eps, stream);
    return launch<false>(nullptr, 0, part, nullptr, 0, weight, w_is_f32, (elem_t*)y, y_stride, rows, width, eps, stream);
}

// ---------------------------------------------------------------------------- float residual stream
// The residual stream kept in float whatever the element type, with up to two addends a layer
// (a block whose mixer and feed-forward read the same norm output and are added together):
//     r <- a + b            (first: the stream starts here, r is not read)
//     r <- r + a + b        (else; a and b may each be absent)
//     y = r * rsqrt(mean(r^2) + eps) * (offset + w)        rounded once, to the element type
// All arithmetic in float.  offset 1 is the weight stored around zero, offset 0 the plain weight.
// An addend may be given as the float partial sums of a product whose k range was split (pa, pb): they
// are added, with the bias, and rounded to the element type as the product's own finishing pass would.
template <typename T>
__global__ void __launch_bounds__(1024)
stream_rms_norm_kernel(const T* __restrict__ a, int64_t a_stride, PartialInput pa, const T* __restrict__ b,
                       int64_t b_stride, PartialInput pb, float* residual, int64_t r_stride, int first,
                       const void* __restrict__ weight, int w_is_f32, float offset, T* __restrict__ y,
                       int64_t y_stride, int width, float eps) {
    __shared__ float scratch[16];
    const int64_t row = blockIdx.x;
    const T* ar = a ? a + row * a_stride : nullptr;
    const T* br = b ? b + row * b_stride : nullptr;
    float* rr = residual + row * r_stride;
    T* yr = y + row * y_stride;
    const T* w_e = static_cast<const T*>(weight);
    const float* w_f = static_cast<const float*>(weight);
    constexpr int KEEP = 4;                       // elements a thread keeps between the two passes
    float kept[KEEP];
    float ss = 0.f;
    int n = 0;
    for (int i = threadIdx.x; i < width; i += blockDim.x, ++n) {
        float s = first ? 0.f : rr[i];
        // the two sublayers are added to each other first, then to the stream
        float add = 0.f;
        if (pa.sums) add = partial_value<T>(pa, row, width, i); else if (ar) add = to_float(ar[i]);
        if (pb.sums) add += partial_value<T>(pb, row, width, i); else if (br) add += to_float(br[i]);
        s += add;
        if (ar || br || pa.sums || pb.sums || first) rr[i] = s;
        if (n < KEEP) kept[n] = s;
        ss += s * s;
    }
    ss = block_sum(ss, scratch);
    const float scale = rsqrtf(ss / (float)width + eps);
    n = 0;
    for (int i = threadIdx.x; i < width; i += blockDim.x, ++n) {
        const float s = n < KEEP ? kept[n] : rr[i];
        const float w = offset + (w_is_f32 ? w_f[i] : to_float(w_e[i]));
        yr[i] = from_float<T>(s * scale * w);
    }
}

// residual: float [rows, width] in place.  a, b: elements or null.  first != 0: the stream starts with a (+ b).
// a_sums / b_sums (with splits, the stride between splits and an optional bias): the addend as partial sums
// [splits][rows][width] instead of elements.
NVA_EXPORT int NVA_NAME(nva_stream_rms_norm)(const void* a, int64_t a_stride, const float* a_sums, int a_splits,
                                             int64_t a_split_stride, const void* a_bias, const void* b, int64_t b_stride,
                                             const float* b_sums, int b_splits, int64_t b_split_stride, const void* b_bias,
                                             float* residual, int64_t r_stride, int first, const void* weight,
                                             int w_is_f32, float offset, void* y, int64_t y_stride, int64_t rows,
                                             int width, float eps, hipStream_t stream) {
    if (rows == 0) return 0;
    if (rows < 0 || rows > 0x7fffffff || width <= 0)
        return nva_fail("stream_rms_norm: bad shape rows=%lld width=%d", (long long)rows, width);
    if (!residual || !y || !weight) return nva_fail("stream_rms_norm: residual, output and weight are needed");
    if (first && !a && !a_sums) return nva_fail("stream_rms_norm: the stream starts with an addend");
    const PartialInput pa{a_sums, a_splits, a_split_stride, a_bias}, pb{b_sums, b_splits, b_split_stride, b_bias};
    if ((a_sums && (a_splits <= 0 || a_split_stride < rows * (int64_t)width)) ||
        (b_sums && (b_splits <= 0 || b_split_stride < rows * (int64_t)width)))
        return nva_fail("stream_rms_norm: bad partial sums");
    // (partial sums of few rows: an element a thread, so that a row's sums are asked for at once)
    const int threads = (a_sums || b_sums) && rows <= 64 && width >= 1024 ? 1024
                        : width >= 2048 ? 512 : width >= 1024 ? 256 : width >= 256 ? 128 : 64;
    hipLaunchKernelGGL((stream_rms_norm_kernel<elem_t>), dim3((unsigned)rows), dim3(threads), 0, stream,
                       (const elem_t*)a, a_stride, pa, (const elem_t*)b, b_stride, pb, residual, r_stride, first, weight,
                       w_is_f32, offset, (elem_t*)y, y_stride, width, eps);
    return nva_check_launch("stream_rms_norm");
}

// ---------------------------------------------------------------------------- scaled addends, two norms of one stream
// A block whose two sublayers read norms of their own of the same stream, and whose outputs are multiplied,
// channel by channel, with learned vectors before they are added (layer scale):
//     r <- r + sa * a + sb * b          (first: r <- a, unscaled: the embedding; a, b, sa, sb may each be absent)
//     y1 = r * rsqrt(mean(r^2) + eps) * w1;   y2 = r * rsqrt(mean(r^2) + eps) * w2      (y2, w2 may be absent)
// All arithmetic in float, each output rounded once.  One row sum serves both norms.  An addend may come as the
// float partial sums of a split product.
template <typename T>
__global__ void __launch_bounds__(1024)
stream_scaled_norm_kernel(const T* __restrict__ a, int64_t a_stride, PartialInput pa, const void* __restrict__ sa,
                          const T* __restrict__ b, int64_t b_stride, PartialInput pb, const void* __restrict__ sb,
                          int s_is_f32, float* residual, int64_t r_stride, int first,
                          const void* __restrict__ w1, const void* __restrict__ w2, int w_is_f32,
                          T* __restrict__ y1, T* __restrict__ y2, int64_t y_stride, int width, float eps) {
    __shared__ float scratch[16];
    const int64_t row = blockIdx.x;
    const T* ar = a ? a + row * a_stride : nullptr;
    const T* br = b ? b + row * b_stride : nullptr;
    float* rr = residual + row * r_stride;
    auto vec = [&](const void* v, int is_f32, int i) -> float {
        return !v ? 1.f : is_f32 ? static_cast<const float*>(v)[i] : to_float(static_cast<const T*>(v)[i]);
    };
    constexpr int KEEP = 4;
    float kept[KEEP];
    float ss = 0.f;
    int n = 0;
    const bool adds = ar || br || pa.sums || pb.sums;
    for (int i = threadIdx.x; i < width; i += blockDim.x, ++n) {
        float s = first ? 0.f : rr[i];
        float add = 0.f;
        if (pa.sums) add = partial_value<T>(pa, row, width, i) * vec(sa, s_is_f32, i);
        else if (ar) add = to_float(ar[i]) * vec(sa, s_is_f32, i);
        if (pb.sums) add += partial_value<T>(pb, row, width, i) * vec(sb, s_is_f32, i);
        else if (br) add += to_float(br[i]) * vec(sb, s_is_f32, i);
        s += add;
        if (adds || first) rr[i] = s;
        if (n < KEEP) kept[n] = s;
        ss += s * s;
    }
    ss = block_sum(ss, scratch);
    const float scale = rsqrtf(ss / (float)width + eps);
    n = 0;
    for (int i = threadIdx.x; i < width; i += blockDim.x, ++n) {
        const float s = (n < KEEP ? kept[n] : rr[i]) * scale;
        y1[row * y_stride + i] = from_float<T>(s * vec(w1, w_is_f32, i));
        if (y2) y2[row * y_stride + i] = from_float<T>(s * vec(w2, w_is_f32, i));
    }
}

// a, b: elements [rows, width], partial sums, or null; sa, sb: vectors [width] (float when s_is_f32, else elements) or
// null (1); residual float [rows, width] in place; y1 and (optional) y2 [rows, width] with rows y_stride apart.
NVA_EXPORT int NVA_NAME(nva_stream_scaled_norm)(const void* a, int64_t a_stride, const float* a_sums, int a_splits,
                                                int64_t a_split_stride, const void* a_bias, const void* sa, const void* b,
                                                int64_t b_stride, const float* b_sums, int b_splits, int64_t b_split_stride,
                                                const void* b_bias, const void* sb, int s_is_f32, float* residual,
                                                int64_t r_stride, int first, const void* w1, const void* w2, int w_is_f32,
                                                void* y1, void* y2, int64_t y_stride, int64_t rows, int width, float eps,
                                                hipStream_t stream) {
    if (rows == 0) return 0;
    if (rows < 0 || rows > 0x7fffffff || width <= 0)
        return nva_fail("stream_scaled_norm: bad shape rows=%lld width=%d", (long long)rows, width);
    if (!residual || !y1 || !w1 || (y2 && !w2)) return nva_fail("stream_scaled_norm: residual, output and weight are needed");
    if (first && !a && !a_sums) return nva_fail("stream_scaled_norm: the stream starts with an addend");
    const PartialInput pa{a_sums, a_splits, a_split_stride, a_bias}, pb{b_sums, b_splits, b_split_stride, b_bias};
    if ((a_sums && (a_splits <= 0 || a_split_stride < rows * (int64_t)width)) ||
        (b_sums && (b_splits <= 0 || b_split_stride < rows * (int64_t)width)))
        return nva_fail("stream_scaled_norm: bad partial sums");
    const int threads = (a_sums || b_sums) && rows <= 64 && width >= 1024 ? 1024
                        : width >= 2048 ? 512 : width >= 1024 ? 256 : width >= 256 ? 128 : 64;
    hipLaunchKernelGGL((stream_scaled_norm_kernel<elem_t>), dim3((unsigned)rows), dim3(threads), 0, stream,
                       (const elem_t*)a, a_stride, pa, sa, (const elem_t*)b, b_stride, pb, sb, s_is_f32, residual, r_stride,
                       first, w1, w2, w_is_f32, (elem_t*)y1, (elem_t*)y2, y_stride, width, eps);
    return nva_check_launch("stream_scaled_norm");
}

// ---------------------------------------------------------------------------- a normed addend into the float stream
// A sublayer's output enters the stream through a norm of its own and a constant, and the stream is normed
// for the next sublayer, all in one pass over the row:
//     u = a / sqrt(mean(a^2) + eps_a) * wa            a elements, or a split product's partial sums
//     r <- r + mult * u
//     y = r / sqrt(mean(r^2) + eps) * w               rounded once, to the element type
// All arithmetic in float; r float, in place.  One workgroup a row, which keeps its entries between the sums.
template <typename T>
__global__ void __launch_bounds__(1024)
stream_post_norm_kernel(const T* __restrict__ a, int64_t a_stride, PartialInput pa, const void* __restrict__ a_weight,
                        int aw_is_f32, float a_eps, float mult, float* residual, int64_t r_stride,
                        const void* __restrict__ weight, int w_is_f32, T* __restrict__ y, int64_t y_stride, int width,
                        float eps) {
    __shared__ float scratch[16];
    const int64_t row = blockIdx.x;
    const T* ar = a ? a + row * a_stride : nullptr;
    float* rr = residual + row * r_stride;
    T* yr = y + row * y_stride;
    constexpr int KEEP = 8;                       // entries a thread keeps between the passes
    float kept[KEEP];
    float ss = 0.f;
    int n = 0;
    for (int i = threadIdx.x; i < width; i += blockDim.x, ++n) {
        const float v = pa.sums ? partial_value<T>(pa, row, width, i) : to_float(ar[i]);
        if (n < KEEP) kept[n] = v;
        ss += v * v;
    }
    ss = block_sum(ss, scratch);
    const float a_scale = rsqrtf(ss / (float)width + a_eps) * mult;
    float ss2 = 0.f;
    n = 0;
    for (int i = threadIdx.x; i < width; i += blockDim.x, ++n) {
        const float v = n < KEEP ? kept[n] : (pa.sums ? partial_value<T>(pa, row, width, i) : to_float(ar[i]));
        const float wa = aw_is_f32 ? static_cast<const float*>(a_weight)[i] : to_float(static_cast<const T*>(a_weight)[i]);
        const float s = rr[i] + v * a_scale * wa;
        rr[i] = s;
        if (n < KEEP) kept[n] = s;
        ss2 += s * s;
    }
    ss2 = block_sum(ss2, scratch);
    const float scale = rsqrtf(ss2 / (float)width + eps);
    n = 0;
    for (int i = threadIdx.x; i < width; i += blockDim.x, ++n) {
        const float s = n < KEEP ? kept[n] : rr[i];
        const float w = w_is_f32 ? static_cast<const float*>(weight)[i] : to_float(static_cast<const T*>(weight)[i]);
        yr[i] = from_float<T>(s * scale * w);
    }
}

// a: elements [rows, width], or (a_sums) partial sums [splits][rows][width] with an optional bias.
NVA_EXPORT int NVA_NAME(nva_stream_post_norm)(const void* a, int64_t a_stride, const float* a_sums, int a_splits,
                                              int64_t a_split_stride, const void* a_bias, const void* a_weight,
                                              int aw_is_f32, float a_eps, float mult, float* residual, int64_t r_stride,
                                              const void* weight, int w_is_f32, void* y, int64_t y_stride, int64_t rows,
                                              int width, float eps, hipStream_t stream) {
    if (rows == 0) return 0;
    if (rows < 0 || rows > 0x7fffffff || width <= 0)
        return nva_fail("stream_post_norm: bad shape rows=%lld width=%d", (long long)rows, width);
    if (!residual || !y || !weight || !a_weight || (!a && !a_sums))
        return nva_fail("stream_post_norm: the addend, its weight, the stream, the weight and the output are needed");
    if (a_sums && (a_splits <= 0 || a_split_stride < rows * (int64_t)width)) return nva_fail("stream_post_norm: bad partial sums");
    const PartialInput pa{a_sums, a_splits, a_split_stride, a_bias};
    const int threads = a_sums && rows <= 64 && width >= 1024 ? 1024
                        : width >= 2048 ? 512 : width >= 1024 ? 256 : width >= 256 ? 128 : 64;
    hipLaunchKernelGGL((stream_post_norm_kernel<elem_t>), dim3((unsigned)rows), dim3(threads), 0, stream,
                       (const elem_t*)a, a_stride, pa, a_weight, aw_is_f32, a_eps, mult, residual, r_stride, weight, w_is_f32,
                       (elem_t*)y, y_stride, width, eps);
    return nva_check_launch("stream_post_norm");
}

// ---------------------------------------------------------------------------- Dynamic Tanh on the float stream
//     r <- r + a + b   (first: r <- a + b)        a, b elements or absent
//     y = tanh(alpha * r) * w + c                  alpha one float read on the device, w and c float vectors
// No mean and no variance: every entry by itself.  All float, rounded once.
template <typename T>
__global__ void __launch_bounds__(256)
stream_dyt_kernel(const T* __restrict__ a, int64_t a_stride, const T* __restrict__ b, int64_t b_stride, float* residual,
                  int64_t r_stride, int first, const float* __restrict__ weight, const float* __restrict__ bias,
                  const float* __restrict__ alpha, T* __restrict__ y, int64_t y_stride, int width) {
    const int64_t row = blockIdx.y;
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= width) return;
    float* rr = residual + row * r_stride;
    float s = first ? 0.f : rr[i];
    float add = 0.f;
    if (a) add = to_float(a[row * a_stride + i]);
    if (b) add += to_float(b[row * b_stride + i]);
    s += add;
    if (a || b || first) rr[i] = s;
    y[row * y_stride + i] = from_float<T>(tanhf(alpha[0] * s) * weight[i] + bias[i]);
}

NVA_EXPORT int NVA_NAME(nva_stream_dyt)(const void* a, int64_t a_stride, const void* b, int64_t b_stride, float* residual,
                                        int64_t r_stride, int first, const float* weight, const float* bias,
                                        const float* alpha, void* y, int64_t y_stride, int64_t rows, int width,
                                        hipStream_t stream) {
    if (rows == 0) return 0;
    if (rows < 0 || width <= 0) return nva_fail("stream_dyt: bad shape rows=%lld width=%d", (long long)rows, width);
    if (!residual || !y || !weight || !bias || !alpha) return nva_fail("stream_dyt: residual, output, weight, bias and alpha are needed");
    if (first && !a) return nva_fail("stream_dyt: the stream starts with an addend");
    for (int64_t r0 = 0; r0 < rows; r0 += 65535) {
        const unsigned nr = (unsigned)((rows - r0) < 65535 ? (rows - r0) : 65535);
        hipLaunchKernelGGL((stream_dyt_kernel<elem_t>), dim3((width + 255) / 256, nr), dim3(256), 0, stream,
                           a ? (const elem_t*)a + r0 * a_stride : nullptr, a_stride,
                           b ? (const elem_t*)b + r0 * b_stride : nullptr, b_stride, residual + r0 * r_stride, r_stride, first,
                           weight, bias, alpha, (elem_t*)y + r0 * y_stride, y_stride, width);
    }
    return nva_check_launch("stream_dyt");
}

// ---------------------------------------------------------------------------- two normed inputs, averaged
//     y = ( a * rsqrt(mean(a^2) + eps) * wa  +  b * rsqrt(mean(b^2) + eps) * wb ) / 2
// a, b elements [rows, width] (each may come as the partial sums of a split product), wa, wb float [width].
template <typename T>
__global__ void __launch_bounds__(1024)
pair_norm_mean_kernel(const T* __restrict__ a, int64_t a_stride, PartialInput pa, const float* __restrict__ wa,
                      const T* __restrict__ b, int64_t b_stride, PartialInput pb, const float* __restrict__ wb,
                      T* __restrict__ y, int64_t y_stride, int width, float eps) {
    extern __shared__ __attribute__((aligned(16))) float row_s[];       // a's row, then b's
    __shared__ float scratch[16];
    const int64_t row = blockIdx.x;
    float sa = 0.f, sb = 0.f;
    for (int i = threadIdx.x; i < width; i += blockDim.x) {
        const float x = pa.sums ? partial_value<T>(pa, row, width, i) : to_float(a[row * a_stride + i]);
        const float z = pb.sums ? partial_value<T>(pb, row, width, i) : to_float(b[row * b_stride + i]);
        row_s[i] = x;
        row_s[width + i] = z;
        sa += x * x;
        sb += z * z;
    }
    sa = block_sum(sa, scratch);
    sb = block_sum(sb, scratch);
    const float ra = rsqrtf(sa / (float)width + eps), rb = rsqrtf(sb / (float)width + eps);
    for (int i = threadIdx.x; i < width; i += blockDim.x)
        y[row * y_stride + i] = from_float<T>(0.5f * (row_s[i] * ra * wa[i] + row_s[width + i] * rb * wb[i]));
}

NVA_EXPORT int NVA_NAME(nva_pair_norm_mean)(const void* a, int64_t a_stride, const float* a_sums, int a_splits,
                                            int64_t a_split_stride, const void* a_bias, const float* wa, const void* b,
                                            int64_t b_stride, const float* b_sums, int b_splits, int64_t b_split_stride,
                                            const void* b_bias, const float* wb, void* y, int64_t y_stride, int64_t rows,
                                            int width, float eps, hipStream_t stream) {
    if (rows == 0) return 0;
    if (rows < 0 || rows > 0x7fffffff || width <= 0 || width > 16 * 1024)
        return nva_fail("pair_norm_mean: bad shape rows=%lld width=%d", (long long)rows, width);
    if ((!a && !a_sums) || (!b && !b_sums) || !wa || !wb || !y) return nva_fail("pair_norm_mean: both inputs, both weights and the output are needed");
    const PartialInput pa{a_sums, a_splits, a_split_stride, a_bias}, pb{b_sums, b_splits, b_split_stride, b_bias};
    const int threads = width >= 2048 ? 512 : width >= 512 ? 256 : 128;
    auto kernel = pair_norm_mean_kernel<elem_t>;
    const size_t lds = 2 * (size_t)width * sizeof(float);
    static bool raised = false;
    if (!raised && lds > 48 * 1024) {
        if (hipFuncSetAttribute((const void*)kernel, hipFuncAttributeMaxDynamicSharedMemorySize, 128 * 1024) != hipSuccess)
            return nva_fail("pair_norm_mean: cannot have %zu bytes of LDS", lds);
        raised = true;
    }
    hipLaunchKernelGGL(kernel, dim3((unsigned)rows), dim3(threads), lds, stream, (const elem_t*)a, a_stride, pa, wa,
                       (const elem_t*)b, b_stride, pb, wb, (elem_t*)y, y_stride, width, eps);
    return nva_check_launch("pair_norm_mean");
}

NVA_DEFINE_LAST_ERROR(nva_norm)
