// Layer norm with weight and bias over rows of the float32 residual stream, and the step between two sublayers
// whose input and result are both normed:
//
//     LN(u)[c] = (u[c] - mean u) / sqrt(var u + eps) * w[c] + b[c],   var u = mean (u - mean u)^2
//
//     norm   out = scale * LN(sum of the slabs of u)                                  (any output type)
//     step   x <- x + mult * LN_post(sum of the slabs of delta) [+ extra];  out = LN_next(x)   (out optional)
//
// One workgroup a row; the row stays in registers (a lane holds every 256th column), so a row is read once.  The
// mean is taken first and the variance from the deviations, both summed over the workgroup in an order that the
// width alone fixes: a row's result does not depend on what else is in the launch.  All arithmetic is float32.
#include "common.h"
#include <math.h>

#define LN_THREADS 256
#define LN_ITEMS 32     // columns a lane holds: rows of up to 8,192 numbers

struct RowStats {
    float mean, inv;
};

__device__ __forceinline__ RowStats row_stats(const float (&v)[LN_ITEMS], int width, float eps, float* scratch) {
    float s = 0.0f;
#pragma unroll
    for (int i = 0; i < LN_ITEMS; ++i)
        if ((int)threadIdx.x + i * LN_THREADS < width) s += v[i];
    const float mean = block_sum(s, scratch) / (float)width;
    float ss = 0.0f;
#pragma unroll
    for (int i = 0; i < LN_ITEMS; ++i)
        if ((int)threadIdx.x + i * LN_THREADS < width) {
            const float dlt = v[i] - mean;
            ss = fmaf(dlt, dlt, ss);
        }
    const float var = block_sum(ss, scratch) / (float)width;
    RowStats r;
    r.mean = mean;
    r.inv = 1.0f / sqrtf(var + eps);
    return r;
}

__device__ __forceinline__ void load_slabs(float (&v)[LN_ITEMS], const float* __restrict__ src, int parts, size_t part_stride, int width) {
#pragma unroll
    for (int i = 0; i < LN_ITEMS; ++i) {
        const int c = (int)threadIdx.x + i * LN_THREADS;
        float a = 0.0f;
        if (c < width) {
            a = src[c];
            for (int p = 1; p < parts; ++p) a += src[p * part_stride + c];
        }
        v[i] = a;
    }
}

template <typename TO>
__global__ void __launch_bounds__(LN_THREADS)
layer_norm_kernel(const float* __restrict__ u, int parts, size_t part_stride, const float* __restrict__ w,
                  const float* __restrict__ b, float eps, float scale, TO* __restrict__ out, int width) {
    __shared__ float scratch[16];
    const size_t row = blockIdx.x;
    float v[LN_ITEMS];
    load_slabs(v, u + row * width, parts, part_stride, width);
    const RowStats st = row_stats(v, width, eps, scratch);
    TO* dst = out + row * width;
#pragma unroll
    for (int i = 0; i < LN_ITEMS; ++i) {
        const int c = (int)threadIdx.x + i * LN_THREADS;
        if (c < width) store_f(dst, c, ((v[i] - st.mean) * st.inv * w[c] + b[c]) * scale);
    }
}

template <typename TO>
__global__ void __launch_bounds__(LN_THREADS)
sandwich_step_kernel(float* __restrict__ x, const float* __restrict__ delta, int parts, size_t part_stride,
                     const float* __restrict__ post_w, const float* __restrict__ post_b, float post_eps, float mult,
                     const float* __restrict__ extra, const float* __restrict__ next_w, const float* __restrict__ next_b,
                     float next_eps, TO* __restrict__ out, int width) {
    __shared__ float scratch[16];
    const size_t row = blockIdx.x;
    float v[LN_ITEMS];
    load_slabs(v, delta + row * width, parts, part_stride, width);
    const RowStats st = row_stats(v, width, post_eps, scratch);
    float* xr = x + row * width;
#pragma unroll
    for (int i = 0; i < LN_ITEMS; ++i) {
        const int c = (int)threadIdx.x + i * LN_THREADS;
        if (c < width) {
            float nx = xr[c] + mult * ((v[i] - st.mean) * st.inv * post_w[c] + post_b[c]);
            if (extra != nullptr) nx += extra[row * width + c];
            xr[c] = nx;
            v[i] = nx;
        }
    }
    if (out == nullptr) return;
    const RowStats nt = row_stats(v, width, next_eps, scratch);
    TO* dst = out + row * width;
#pragma unroll
    for (int i = 0; i < LN_ITEMS; ++i) {
        const int c = (int)threadIdx.x + i * LN_THREADS;
        if (c < width) store_f(dst, c, (v[i] - nt.mean) * nt.inv * next_w[c] + next_b[c]);
    }
}

extern "C" int kipp_layer_norm(const float* u, int parts, const float* w, const float* b, float eps, float scale, void* out,
                               int out_dtype, int rows, int width, hipStream_t stream) {
    if (rows <= 0) return 0;
    if (width <= 0 || width > LN_THREADS * LN_ITEMS || parts <= 0) return -1;
    const size_t part_stride = (size_t)rows * width;
    if (out_dtype == KIPP_F32)
        hipLaunchKernelGGL((layer_norm_kernel<float>), dim3(rows), dim3(LN_THREADS), 0, stream, u, parts, part_stride, w, b, eps, scale,
                           (float*)out, width);
    else if (out_dtype == KIPP_BF16)
        hipLaunchKernelGGL((layer_norm_kernel<bf16_t>), dim3(rows), dim3(LN_THREADS), 0, stream, u, parts, part_stride, w, b, eps, scale,
                           (bf16_t*)out, width);
    else
        return -2;
    return KIPP_LAUNCH_CHECK();
}

extern "C" int kipp_sandwich_step(float* x, const float* delta, int parts, const float* post_w, const float* post_b, float post_eps,
                                  float mult, const float* extra, const float* next_w, const float* next_b, float next_eps,
                                  void* out, int out_dtype, int rows, int width, hipStream_t stream) {
    if (rows <= 0) return 0;
    if (width <= 0 || width > LN_THREADS * LN_ITEMS || parts <= 0) return -1;
    if (out != nullptr && (next_w == nullptr || next_b == nullptr)) return -1;
    const size_t part_stride = (size_t)rows * width;
    if (out == nullptr || out_dtype == KIPP_F32)
        hipLaunchKernelGGL((sandwich_step_kernel<float>), dim3(rows), dim3(LN_THREADS), 0, stream, x, delta, parts, part_stride, post_w,
                           post_b, post_eps, mult, extra, next_w, next_b, next_eps, (float*)out, width);
    else if (out_dtype == KIPP_BF16)
        hipLaunchKernelGGL((sandwich_step_kernel<bf16_t>), dim3(rows), dim3(LN_THREADS), 0, stream, x, delta, parts, part_stride, post_w,
                           post_b, post_eps, mult, extra, next_w, next_b, next_eps, (bf16_t*)out, width);
    else
        return -2;
    return KIPP_LAUNCH_CHECK();
}
