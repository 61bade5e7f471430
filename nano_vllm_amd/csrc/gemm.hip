// y[M, N] = x[M, K] * W[N, K]^T (+ bias[N]): the linear layer of
// nanovllm/layers/linear.py:51,73,153 and the output head of embed_head.py:61, with the weight
// in its stored [out, in] layout.
//
// This is the tiled kernel on the vector units: inputs are read as they are stored, every
// product and sum is a float operation (no matrix-core instruction, no reduced-precision
// input format), and each output is summed over k in ascending order in 16-wide tiles,
// whatever M is.  It is the matrix product of the 32-bit path and accepts any M, N, K.
// The result is written as elements or, for logits, as float.
#include "common.h"

#define TILE_M 64
#define TILE_N 64
#define TILE_K 16

template <typename T>
__device__ __forceinline__ void load_tile(const T* __restrict__ src, int64_t stride, int rows_left, int k_left,
                                          bool vec, float (*dst)[TILE_M + 4], int tid) {
    // 64 rows x 16 k: each of the 256 threads takes 4 consecutive k of one row
    const int r = tid / 4, kq = (tid % 4) * 4;
    float v[4] = {0.f, 0.f, 0.f, 0.f};
    if (r < rows_left) {
        const T* p = src + (int64_t)r * stride + kq;
        if (vec && kq + 4 <= k_left) {
            if (sizeof(T) == 4) {
                const float4 f = *reinterpret_cast<const float4*>(p);
                v[0] = f.x; v[1] = f.y; v[2] = f.z; v[3] = f.w;
            } else {
                typedef __attribute__((ext_vector_type(4))) __bf16 b4;
                const b4 f = *reinterpret_cast<const b4*>(p);
#pragma unroll
                for (int e = 0; e < 4; ++e) v[e] = static_cast<float>(f[e]);
            }
        } else {
#pragma unroll
            for (int e = 0; e < 4; ++e)
                if (kq + e < k_left) v[e] = to_float(p[e]);
        }
    }
#pragma unroll
    for (int e = 0; e < 4; ++e) dst[kq + e][r] = v[e];
}

template <typename T, typename OutT>
__global__ void __launch_bounds__(256)
linear_tiled_kernel(const T* __restrict__ x, int64_t x_stride, const T* __restrict__ w, int64_t w_stride,
                    const T* __restrict__ bias, OutT* __restrict__ y, int64_t y_stride, int M, int N, int K,
                    int vec) {
    __shared__ float xs[TILE_K][TILE_M + 4];
    __shared__ float ws[TILE_K][TILE_N + 4];
    const int tid = threadIdx.x;
    const int m0 = blockIdx.y * TILE_M, n0 = blockIdx.x * TILE_N;
    const int ty = tid / 16, tx = tid % 16;
    float acc[4][4];
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[i][j] = 0.f;

    for (int k0 = 0; k0 < K; k0 += TILE_K) {
        load_tile<T>(x + (int64_t)m0 * x_stride + k0, x_stride, M - m0, K - k0, vec, xs, tid);
        load_tile<T>(w + (int64_t)n0 * w_stride + k0, w_stride, N - n0, K - k0, vec, ws, tid);
        __syncthreads();
#pragma unroll
        for (int k = 0; k < TILE_K; ++k) {
            const float4 a = *reinterpret_cast<const float4*>(&xs[k][ty * 4]);
            const float4 b = *reinterpret_cast<const float4*>(&ws[k][tx * 4]);
            const float av[4] = {a.x, a.y, a.z, a.w}, bv[4] = {b.x, b.y, b.z, b.w};
#pragma unroll
            for (int i = 0; i < 4; ++i)
#pragma unroll
                for (int j = 0; j < 4; ++j) acc[i][j] += av[i] * bv[j];
        }
        __syncthreads();
    }
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const int m = m0 + ty * 4 + i;
        if (m >= M) continue;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int n = n0 + tx * 4 + j;
            if (n >= N) continue;
            float v = acc[i][j];
            if (bias) v += to_float(bias[n]);
            y[(int64_t)m * y_stride + n] = from_float<OutT>(v);
        }
    }
}

NVA_EXPORT int NVA_NAME(nva_linear_tiled)(const void* x, int64_t x_stride, const void* w, int64_t w_stride,
                                          const void* bias, void* y, int64_t y_stride, int out_is_f32, int64_t M,
                                          int64_t N, int64_t K, hipStream_t stream) {
    if (M == 0 || N == 0) return 0;
    if (M < 0 || N < 0 || K <= 0 || M > 0x7fffffff || N > 0x7fffffff || K > 0x7fffffff)
        return nva_fail("linear: bad shape M=%lld N=%lld K=%lld", (long long)M, (long long)N, (long long)K);
    const int64_t grid_m = (M + TILE_M - 1) / TILE_M, grid_n = (N + TILE_N - 1) / TILE_N;
    if (grid_m > 65535) return nva_fail("linear: M=%lld exceeds %d rows per call", (long long)M, 65535 * TILE_M);
    const size_t vb = 4 * sizeof(elem_t);
    const int vec = x_stride % 4 == 0 && w_stride % 4 == 0 && nva_aligned(x, vb) && nva_aligned(w, vb);
    dim3 grid((unsigned)grid_n, (unsigned)grid_m);
    if (out_is_f32)
        hipLaunchKernelGGL((linear_tiled_kernel<elem_t, float>), grid, dim3(256), 0, stream, (const elem_t*)x, x_stride,
                           (const elem_t*)w, w_stride, (const elem_t*)bias, (float*)y, y_stride, (int)M, (int)N,
                           (int)K, vec);
    else
        hipLaunchKernelGGL((linear_tiled_kernel<elem_t, elem_t>), grid, dim3(256), 0, stream, (const elem_t*)x,
                           x_stride, (const elem_t*)w, w_stride, (const elem_t*)bias, (elem_t*)y, y_stride, (int)M,
                           (int)N, (int)K, vec);
    return nva_check_launch("linear_tiled");
}

NVA_DEFINE_LAST_ERROR(nva_gemm)
