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

__global__ void __launch_bounds__(256)
sample_kernel(const float* __restrict__ logits, int64_t row_stride, int vocab,
              const float* __restrict__ temperatures, const uint64_t* __restrict__ keys,
              int32_t* __restrict__ out) {
    __shared__ double best_s[256];
    __shared__ int best_i[256];
    const int64_t row = blockIdx.x;
    const float* l = logits + row * row_stride;
    const float temp = temperatures ? temperatures[row] : 0.f;
    const uint64_t key = keys ? keys[row] : 0;
    double best = -INFINITY;
    int best_idx = 0x7fffffff;
    for (int i = threadIdx.x; i < vocab; i += blockDim.x) {
        double s = (double)l[i];
        if (temp > 0.f) {
            const uint64_t bits = mix64(key ^ (uint64_t)i);
            const double u = ((double)(bits >> 40) + 0.5) * (1.0 / 16777216.0);
            s = s / (double)temp - log(-log(u));
        }
        // a NaN score never wins; a row of only NaN yields index 0
        if (s == s && (best_idx == 0x7fffffff || s > best || (s == best && i < best_idx))) {
            best = s;
            best_idx = i;
        }
    }
    best_s[threadIdx.x] = best;
    best_i[threadIdx.x] = best_idx;
    __syncthreads();
    for (int step = blockDim.x / 2; step > 0; step >>= 1) {
        if (threadIdx.x < step) {
            const double a = best_s[threadIdx.x], b = best_s[threadIdx.x + step];
            const int ia = best_i[threadIdx.x], ib = best_i[threadIdx.x + step];
            if (b > a || (b == a && ib < ia)) {
                best_s[threadIdx.x] = b;
                best_i[threadIdx.x] = ib;
            }
        }
        __syncthreads();
    }
    if (threadIdx.x == 0) out[row] = best_i[0] == 0x7fffffff ? 0 : best_i[0];
}

NVA_EXPORT int nva_sample(const float* logits, int64_t row_stride, int64_t rows, int vocab,
                          const float* temperatures, const uint64_t* keys, int32_t* out, hipStream_t stream) {
    if (rows == 0) return 0;
    if (rows < 0 || rows > 0x7fffffff || vocab <= 0) return nva_fail("sample: bad shape rows=%lld vocab=%d", (long long)rows, vocab);
    hipLaunchKernelGGL(sample_kernel, dim3((unsigned)rows), dim3(256), 0, stream, logits, row_stride, vocab,
                       temperatures, keys, out);
    return nva_check_launch("sample");
}

NVA_DEFINE_LAST_ERROR(nva_sample)
