// SwiGLU gating: out[t, i] = silu(x[t, i]) * x[t, inner + i], silu(g) = g * sigmoid(g)
// (nanovllm/layers/activation.py:8-11).  Computed in float and rounded once.
#include "common.h"

template <typename T, bool VEC>
__global__ void __launch_bounds__(256)
silu_mul_kernel(const T* __restrict__ x, int64_t x_stride, T* __restrict__ out, int64_t out_stride, int inner) {
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
        for (int j = 0; j < 8; ++j) g[j] = g[j] / (1.f + nva_exp(-g[j])) * u[j];
        store8(o + i, g);
    } else {
        const int i = blockIdx.x * blockDim.x + threadIdx.x;
        if (i >= inner) return;
        const float g = to_float(gate[i]);
        o[i] = from_float<T>(g / (1.f + nva_exp(-g)) * to_float(up[i]));
    }
}

NVA_EXPORT int NVA_NAME(nva_silu_mul)(const void* x, int64_t x_stride, void* out, int64_t out_stride,
                                      int64_t rows, int inner, hipStream_t stream) {
    if (rows == 0) return 0;
    if (rows < 0 || rows > 65535LL * 65535LL || inner <= 0)
        return nva_fail("silu_mul: bad shape rows=%lld inner=%d", (long long)rows, inner);
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
            hipLaunchKernelGGL((silu_mul_kernel<elem_t, true>), grid, dim3(256), 0, stream, xp + r0 * x_stride,
                               x_stride, op + r0 * out_stride, out_stride, inner);
        } else {
            dim3 grid((inner + 255) / 256, nr);
            hipLaunchKernelGGL((silu_mul_kernel<elem_t, false>), grid, dim3(256), 0, stream, xp + r0 * x_stride,
                               x_stride, op + r0 * out_stride, out_stride, inner);
        }
    }
    return nva_check_launch("silu_mul");
}

NVA_DEFINE_LAST_ERROR(nva_activation)
