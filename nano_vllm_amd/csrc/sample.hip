// Next-token choice from float logits: one block per chunk of 8192 entries of a row, then one
// wave per row over the chunks' results.
//
// temperature == 0: the argmax of the logits, the lowest index on ties.
// temperature  > 0: the reference draws argmax(softmax(l / T) / E) with E ~ Exp(1) i.i.d. per
// entry (nanovllm/layers/sampler.py:8-12), a categorical draw from softmax(l / T).  The
// softmax's normaliser does not move the argmax, so this takes argmax(l / T - log E) instead.
// E comes from a counter-based generator, a pure function of (row key, entry), so that a
// request's draw does not depend on what else is in the batch:
//   bits = mix64(key ^ entry);  u = ((bits >> 40) + 0.5) / 2^24;  E = -log(u)
// with mix64 the splitmix64 finaliser; the key is made on the host from (seed, request,
// position).  Noise and scores are computed in double.  Two logarithms in double for every entry
// are most of that work, and only the largest score matters: a workgroup first takes all scores of
// its chunk in float, with the fast logarithm, keeps them in registers and finds their maximum; then only
// the entries whose float score lies within SAMPLE_WINDOW of that maximum (a few), and those whose u
// lies in the far tails, where the float score is poor, are taken in double.  The float score is off
// by a few thousandths at most (below), the window is a hundred times that, so the entry with the
// largest score in double is always among them, and it is the one chosen.
#include "common.h"

__device__ __forceinline__ uint64_t mix64(uint64_t z) {
    z += 0x9E3779B97F4A7C15ull;
    z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
    z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
    return z ^ (z >> 31);
}

#define SAMPLE_THREADS 256
#define SAMPLE_CHUNK 8192         // entries of a row per workgroup
#define SAMPLE_WINDOW 0.5f        // float scores this far below the largest are still taken in double
#define SAMPLE_TAIL 1024u         // u below SAMPLE_TAIL / 2^24 or above 1 - SAMPLE_TAIL / 2^24: always in double

__device__ __forceinline__ bool better(double s, int i, double best, int best_idx) {
    // a NaN score never wins (its index stays 0x7fffffff); the lowest index wins a tie
    return i != 0x7fffffff && (best_idx == 0x7fffffff || s > best || (s == best && i < best_idx));
}

__device__ __forceinline__ double score(float logit, float temp, uint64_t key, int entry) {
    double s = (double)logit;
    if (temp > 0.f) {
        const uint64_t bits = mix64(key ^ (uint64_t)entry);
        const double u = ((double)(bits >> 40) + 0.5) * (1.0 / 16777216.0);
        s = s / (double)temp - log(-log(u));
    }
    return s;
}

// The score in float, or +inf for an entry that is to be taken in double whatever the others' scores.
// Between the tails |d log(-log u) / du| is at most 2^24 / SAMPLE_TAIL, the float u is off by 2^-25
// (it has no bit for the half) and the fast logarithm by a few units in the last place, also of the
// small -log u near u = 1: together under 2e-3; the quotient logit / T adds 2e-7 of itself.
__device__ __forceinline__ float float_score(float logit, float inv_temp, uint64_t key, int entry) {
    const uint32_t k24 = (uint32_t)(mix64(key ^ (uint64_t)entry) >> 40);
    if (k24 < SAMPLE_TAIL || k24 >= (1u << 24) - SAMPLE_TAIL) return INFINITY;
    const float u = ((float)k24 + 0.5f) * (1.f / 16777216.f);
    return logit * inv_temp - __logf(-__logf(u));
}

// The best entry of a block's threads: within the waves, then across them (thread 0 holds it).
__device__ __forceinline__ void block_best(double& best, int& best_idx) {
    __shared__ double best_s[SAMPLE_THREADS / NVA_WAVE];
    __shared__ int best_i[SAMPLE_THREADS / NVA_WAVE];
#pragma unroll
    for (int off = NVA_WAVE / 2; off > 0; off >>= 1) {
        const double os = __shfl_xor(best, off, NVA_WAVE);
        const int oi = __shfl_xor(best_idx, off, NVA_WAVE);
        if (better(os, oi, best, best_idx)) {
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
    if (threadIdx.x == 0)
        for (int w = 1; w < (int)blockDim.x / NVA_WAVE; ++w)
            if (better(best_s[w], best_i[w], best, best_idx)) {
                best = best_s[w];
                best_idx = best_i[w];
            }
}

// First pass: the best entry of one chunk of one row -> part_s / part_i [rows][chunks].
__global__ void __launch_bounds__(SAMPLE_THREADS)
sample_chunk_kernel(const float* __restrict__ logits, int64_t row_stride, int vocab,
                    const float* __restrict__ temperatures, const uint64_t* __restrict__ keys,
                    double* __restrict__ part_s, int32_t* __restrict__ part_i) {
    const int64_t row = blockIdx.y;
    const int chunk = blockIdx.x, chunks = gridDim.x;
    const float* l = logits + row * row_stride;
    const float temp = temperatures ? temperatures[row] : 0.f;
    const uint64_t key = keys ? keys[row] : 0;
    const int begin = chunk * SAMPLE_CHUNK, end = min(vocab, begin + SAMPLE_CHUNK);
    double best = -INFINITY;
    int best_idx = 0x7fffffff;
    const bool vec = (row_stride % 4 == 0) && ((uintptr_t)logits % 16 == 0);
    const int vec_end = vec ? begin + ((end - begin) & ~3) : begin;
    if (temp > 0.f) {
        // ---- every score in float, kept in registers (a thread walks SAMPLE_CHUNK / SAMPLE_THREADS
        // entries); their maximum over the chunk (the tails and NaN aside)
        constexpr int PER = SAMPLE_CHUNK / SAMPLE_THREADS;
        __shared__ float max_s[SAMPLE_THREADS / NVA_WAVE];
        const float inv_temp = 1.f / temp;
        // entry j of this thread: four in a row per turn where rows can be read in vectors
        auto entry = [&](int j) { return vec ? begin + (j / 4) * (SAMPLE_THREADS * 4) + threadIdx.x * 4 + j % 4
                                             : begin + j * SAMPLE_THREADS + threadIdx.x; };
        float f[PER], top = -INFINITY;
#pragma unroll
        for (int j = 0; j < PER; j += 4) {
            float v[4];
            if (vec && entry(j) + 3 < end) {
                const float4 v4 = *reinterpret_cast<const float4*>(l + entry(j));
                v[0] = v4.x; v[1] = v4.y; v[2] = v4.z; v[3] = v4.w;
            } else {
#pragma unroll
                for (int e = 0; e < 4; ++e) v[e] = entry(j + e) < end ? l[entry(j + e)] : 0.f;
            }
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                f[j + e] = entry(j + e) < end ? float_score(v[e], inv_temp, key, entry(j + e)) : -INFINITY;
                if (f[j + e] < INFINITY) top = fmaxf(top, f[j + e]);      // not for a NaN either
            }
        }
        top = wave_max(top);
        if (threadIdx.x % NVA_WAVE == 0) max_s[threadIdx.x / NVA_WAVE] = top;
        __syncthreads();
        top = max_s[0];
#pragma unroll
        for (int w = 1; w < SAMPLE_THREADS / NVA_WAVE; ++w) top = fmaxf(top, max_s[w]);
        // ---- in double: what may be the largest.  (No finite float score at all: everything.)
        const float least = top - (SAMPLE_WINDOW + 4e-6f * fabsf(top));
#pragma unroll
        for (int j = 0; j < PER; ++j) {
            if (f[j] < least || entry(j) >= end) continue;        // the comparison is false for +inf and for a NaN
            const double s = score(l[entry(j)], temp, key, entry(j));
            if (s == s && better(s, entry(j), best, best_idx)) {
                best = s;
                best_idx = entry(j);
            }
        }
    } else {
    for (int i = begin + threadIdx.x * 4; i < vec_end; i += SAMPLE_THREADS * 4) {
        const float4 v4 = *reinterpret_cast<const float4*>(l + i);
        const float v[4] = {v4.x, v4.y, v4.z, v4.w};
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            const double s = score(v[e], temp, key, i + e);
            if (s == s && better(s, i + e, best, best_idx)) {
                best = s;
                best_idx = i + e;
            }
        }
    }
    for (int i = vec_end + threadIdx.x; i < end; i += SAMPLE_THREADS) {
        const double s = score(l[i], temp, key, i);
        if (s == s && better(s, i, best, best_idx)) {
            best = s;
            best_idx = i;
        }
    }
    }
    block_best(best, best_idx);
    if (threadIdx.x == 0) {
        part_s[row * chunks + chunk] = best;
        part_i[row * chunks + chunk] = best_idx;
    }
}

// Second pass: the best of a row's chunks; a row of only NaN yields index 0.
__global__ void __launch_bounds__(NVA_WAVE)
sample_merge_kernel(const double* __restrict__ part_s, const int32_t* __restrict__ part_i, int chunks,
                    int32_t* __restrict__ out) {
    const int64_t row = blockIdx.x;
    double best = -INFINITY;
    int best_idx = 0x7fffffff;
    for (int c = threadIdx.x; c < chunks; c += NVA_WAVE) {
        const double s = part_s[row * chunks + c];
        const int i = part_i[row * chunks + c];
        if (better(s, i, best, best_idx)) {
            best = s;
            best_idx = i;
        }
    }
#pragma unroll
    for (int off = NVA_WAVE / 2; off > 0; off >>= 1) {
        const double os = __shfl_xor(best, off, NVA_WAVE);
        const int oi = __shfl_xor(best_idx, off, NVA_WAVE);
        if (better(os, oi, best, best_idx)) {
            best = os;
            best_idx = oi;
        }
    }
    if (threadIdx.x == 0) out[row] = best_idx == 0x7fffffff ? 0 : best_idx;
}

// scratch: rows * ceil(vocab / 8192) * 12 bytes, 8-byte aligned (nva_sample_scratch_bytes).
NVA_EXPORT int64_t nva_sample_scratch_bytes(int64_t rows, int vocab) {
    const int64_t chunks = (vocab + SAMPLE_CHUNK - 1) / SAMPLE_CHUNK;
    return rows * chunks * 12;
}

NVA_EXPORT int nva_sample(const float* logits, int64_t row_stride, int64_t rows, int vocab,
                          const float* temperatures, const uint64_t* keys, int32_t* out, void* scratch,
                          hipStream_t stream) {
    if (rows == 0) return 0;
    if (rows < 0 || rows > 65535 || vocab <= 0) return nva_fail("sample: bad shape rows=%lld vocab=%d", (long long)rows, vocab);
    if (!scratch || !nva_aligned(scratch, 8)) return nva_fail("sample: needs 8-byte aligned scratch memory");
    const int chunks = (vocab + SAMPLE_CHUNK - 1) / SAMPLE_CHUNK;
    double* part_s = (double*)scratch;
    int32_t* part_i = (int32_t*)(part_s + rows * chunks);
    hipLaunchKernelGGL(sample_chunk_kernel, dim3((unsigned)chunks, (unsigned)rows), dim3(SAMPLE_THREADS), 0, stream, logits,
                       row_stride, vocab, temperatures, keys, part_s, part_i);
    int rc = nva_check_launch("sample_chunk");
    if (rc) return rc;
    hipLaunchKernelGGL(sample_merge_kernel, dim3((unsigned)rows), dim3(NVA_WAVE), 0, stream, part_s, part_i, chunks, out);
    return nva_check_launch("sample_merge");
}

// After a decode step whose tokens were just sampled: the step's own metadata, in place, becomes
// that of the next decode step of the same requests (the reference rebuilds it on the host,
// nanovllm/engine/model_runner.py:166-188; here several steps run without the host in between).
// Request i < n_real takes its sampled token at the next position, whose slot comes from its block
// tables (the page must be there already); rows n_real.. are padding: copies of request 0 that
// write nothing.  out_row receives the sampled tokens.
#define ADVANCE_MAX_GROUPS 4
struct AdvanceGroups {
    int32_t* slots[ADVANCE_MAX_GROUPS];
    const int32_t* tables[ADVANCE_MAX_GROUPS];
    int width[ADVANCE_MAX_GROUPS];
};

__global__ void advance_decode_kernel(int32_t* __restrict__ input_ids, int32_t* __restrict__ positions,
                                      int32_t* __restrict__ kv_lens, int32_t* __restrict__ starts,
                                      const int32_t* __restrict__ sampled,
                                      int32_t* __restrict__ out_row, int n_real, int n_total, int page_size,
                                      AdvanceGroups groups, int num_groups, int32_t* error_flag) {
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n_total) return;
    const int tok = sampled[i < n_real ? i : 0];
    if (i < n_real) out_row[i] = tok;
    const int pos = positions[i] + 1;
    positions[i] = pos;
    kv_lens[i] = pos + 1;
    starts[i] = pos;
    input_ids[i] = tok;
    for (int g = 0; g < num_groups; ++g) {
        int slot = -1;
        if (i < n_real) {
            const int page = pos / page_size < groups.width[g] ? groups.tables[g][(int64_t)i * groups.width[g] + pos / page_size] : -1;
            if (page < 0) {
                if (error_flag) atomicOr(error_flag, 2);
            } else {
                slot = page * page_size + pos % page_size;
            }
        }
        groups.slots[g][i] = slot;
    }
}

NVA_EXPORT int nva_advance_decode(int32_t* input_ids, int32_t* positions, int32_t* kv_lens, int32_t* starts,
                                  const int32_t* sampled, int32_t* out_row, int n_real, int n_total,
                                  int page_size, int num_groups, int32_t* const* slots, const int32_t* const* tables,
                                  const int* widths, int32_t* error_flag, hipStream_t stream) {
    if (n_real <= 0 || n_total < n_real || page_size <= 0 || num_groups < 0 || num_groups > ADVANCE_MAX_GROUPS)
        return nva_fail("advance_decode: bad sizes (%d of %d requests, %d cache groups)", n_real, n_total, num_groups);
    AdvanceGroups groups;
    for (int g = 0; g < num_groups; ++g) {
        groups.slots[g] = slots[g];
        groups.tables[g] = tables[g];
        groups.width[g] = widths[g];
    }
    hipLaunchKernelGGL(advance_decode_kernel, dim3((unsigned)((n_total + 255) / 256)), dim3(256), 0, stream, input_ids,
                       positions, kv_lens, starts, sampled, out_row, n_real, n_total, page_size, groups, num_groups,
                       error_flag);
    return nva_check_launch("advance_decode");
}

NVA_DEFINE_LAST_ERROR(nva_sample)
