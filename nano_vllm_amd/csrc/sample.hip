// Next-token choice from float logits, one block per row.
//
// temperature == 0: the argmax of the logits, the lowest index on ties.
// temperature  > 0: the reference draws argmax(softmax(l / T) / E) with E ~ Exp(1) i.i.d. per
// entry (nanovllm/layers/sampler.py:8-12), a categorical draw from softmax(l / T).  The
// softmax's normaliser does not move the argmax, so this takes argmax(l / T - log E) instead.
// E comes from a counter-based generator, a pure function of (row key, entry), so that a
// request's draw does not depend on what else is in the batch:
//   bits = mix64(key ^ entry);  u = ((bits >> 40) + 0.5) / 2^24;  E = -log(u)
// with mix64 the splitmix64 finaliser; the key is made on the host from (seed, request,
// position).  Noise and scores are computed in double.
#include "common.h"

__device__ __forceinline__ uint64_t mix64(uint64_t z) {
    z += 0x9E3779B97F4A7C15ull;
    z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
    z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
    return z ^ (z >> 31);
}

#define SAMPLE_THREADS 1024

__device__ __forceinline__ void take(double s, int i, double& best, int& best_idx) {
    // a NaN score never wins; a row of only NaN yields index 0
    if (s == s && (best_idx == 0x7fffffff || s > best || (s == best && i < best_idx))) {
        best = s;
        best_idx = i;
    }
}

__global__ void __launch_bounds__(SAMPLE_THREADS)
sample_kernel(const float* __restrict__ logits, int64_t row_stride, int vocab,
              const float* __restrict__ temperatures, const uint64_t* __restrict__ keys,
              int32_t* __restrict__ out) {
    __shared__ double best_s[SAMPLE_THREADS / NVA_WAVE];
    __shared__ int best_i[SAMPLE_THREADS / NVA_WAVE];
    const int64_t row = blockIdx.x;
    const float* l = logits + row * row_stride;
    const float temp = temperatures ? temperatures[row] : 0.f;
    const uint64_t key = keys ? keys[row] : 0;
    double best = -INFINITY;
    int best_idx = 0x7fffffff;
    const bool vec = (row_stride % 4 == 0) && ((uintptr_t)logits % 16 == 0);
    const int vec_end = vec ? (vocab & ~3) : 0;
    for (int i = threadIdx.x * 4; i < vec_end; i += blockDim.x * 4) {
        const float4 v4 = *reinterpret_cast<const float4*>(l + i);
        const float v[4] = {v4.x, v4.y, v4.z, v4.w};
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            double s = (double)v[e];
            if (temp > 0.f) {
                const uint64_t bits = mix64(key ^ (uint64_t)(i + e));
                const double u = ((double)(bits >> 40) + 0.5) * (1.0 / 16777216.0);
                s = s / (double)temp - log(-log(u));
            }
            take(s, i + e, best, best_idx);
        }
    }
    for (int i = vec_end + threadIdx.x; i < vocab; i += blockDim.x) {
        double s = (double)l[i];
        if (temp > 0.f) {
            const uint64_t bits = mix64(key ^ (uint64_t)i);
            const double u = ((double)(bits >> 40) + 0.5) * (1.0 / 16777216.0);
            s = s / (double)temp - log(-log(u));
        }
        take(s, i, best, best_idx);
    }
    // within the wave, then across the waves
#pragma unroll
    for (int off = NVA_WAVE / 2; off > 0; off >>= 1) {
        const double os = __shfl_xor(best, off, NVA_WAVE);
        const int oi = __shfl_xor(best_idx, off, NVA_WAVE);
        if (oi != 0x7fffffff && (best_idx == 0x7fffffff || os > best || (os == best && oi < best_idx))) {
            best = os;
            best_idx = oi;
        }
    }
    const int wave = threadIdx.x / NVA_WAVE, lane = threadIdx.x % NVA_WAVE;
    if (lane == 0) {
        best_s[wave] = best;
        best_i[wave] = best_idx;
    }
    __syncthreads();
    if (threadIdx.x == 0) {
        for (int w = 1; w < blockDim.x / NVA_WAVE; ++w) {
            const double os = best_s[w];
            const int oi = best_i[w];
            if (oi != 0x7fffffff && (best_idx == 0x7fffffff || os > best || (os == best && oi < best_idx))) {
                best = os;
                best_idx = oi;
            }
        }
        out[row] = best_idx == 0x7fffffff ? 0 : best_idx;
    }
}

NVA_EXPORT int nva_sample(const float* logits, int64_t row_stride, int64_t rows, int vocab,
                          const float* temperatures, const uint64_t* keys, int32_t* out, hipStream_t stream) {
    if (rows == 0) return 0;
    if (rows < 0 || rows > 0x7fffffff || vocab <= 0) return nva_fail("sample: bad shape rows=%lld vocab=%d", (long long)rows, vocab);
    hipLaunchKernelGGL(sample_kernel, dim3((unsigned)rows), dim3(SAMPLE_THREADS), 0, stream, logits, row_stride, vocab,
                       temperatures, keys, out);
    return nva_check_launch("sample");
}

NVA_DEFINE_LAST_ERROR(nva_sample)
