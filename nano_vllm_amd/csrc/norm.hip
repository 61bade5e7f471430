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

NVA_DEFINE_LAST_ERROR(nva_norm)
