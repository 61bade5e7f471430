// Causal attention of a step's tokens over the paged cache: the general kernel.
//
// It takes any head size up to 512, any number of heads and groups, any page size and an
// optional window, in float arithmetic with an online softmax (scores, running maximum and
// sum, and the output accumulator in float).  It is the attention of the 32-bit path and the
// fallback of the bfloat16 path for shapes the matrix-core kernels refuse.
//
// Semantics (nanovllm/layers/attention.py:64-75 with causal=True): the query of a token at
// absolute position p of its request, head h, reads the keys of kv head h / (Hq / Hkv) at
// positions j <= p (and j > p - window if window > 0) through the request's block table:
// s_j = scale * <q, k_j>, P = softmax(s), o = sum_j P_j v_j.  The step's own keys are in the
// cache already when this runs.
// Layouts: K [pages, Hkv, page, D], V transposed in tiles of keys (common.h).  One wave per (token, q head).
#include "common.h"

#define ATT_MAX_D 512
#define ATT_ACC (ATT_MAX_D / NVA_WAVE)

template <typename T>
__global__ void __launch_bounds__(NVA_WAVE)
paged_attention_generic_kernel(const T* __restrict__ q, int64_t q_stride, T* __restrict__ out, int64_t out_stride,
                               const T* __restrict__ k_cache, const T* __restrict__ v_cache,
                               const int32_t* __restrict__ block_tables, int table_stride,
                               const int32_t* __restrict__ token_seq, const int32_t* __restrict__ positions,
                               int num_q_heads, int num_kv_heads, int head_dim, int page_size, float scale,
                               int window, int32_t* error_flag) {
    __shared__ float q_s[ATT_MAX_D];
    __shared__ float p_s[NVA_WAVE];
    __shared__ int64_t v_off_s[NVA_WAVE];

    const int64_t t = blockIdx.x;
    const int h = blockIdx.y;
    const int lane = threadIdx.x;
    const int kvh = h / (num_q_heads / num_kv_heads);
    const int seq = token_seq[t];
    const int pos = positions[t];
    const int first = window > 0 && pos - window + 1 > 0 ? pos - window + 1 : 0;
    const int32_t* table = block_tables + (int64_t)seq * table_stride;

    const T* qrow = q + t * q_stride + (int64_t)h * head_dim;
    for (int d = lane; d < head_dim; d += NVA_WAVE) q_s[d] = to_float(qrow[d]);
    __syncthreads();

    float acc[ATT_ACC];
#pragma unroll
    for (int i = 0; i < ATT_ACC; ++i) acc[i] = 0.f;
    float m_run = -INFINITY, l_run = 0.f;
    const bool vec = head_dim % 8 == 0;
    const int vt = nva_v_tile(page_size);

    for (int base = first; base <= pos; base += NVA_WAVE) {
        const int j = base + lane;
        float s = -INFINITY;
        int64_t v_off = 0;
        if (j <= pos) {
            const int page = table[j / page_size];
            const int off = j % page_size;
            if (page < 0) {
                if (error_flag) atomicOr(error_flag, 2);      // a visible key has no page
            } else {
                const int64_t head_base = (int64_t)page * num_kv_heads + kvh;
                const T* krow = k_cache + (head_base * page_size + off) * head_dim;
                v_off = head_base * head_dim * (int64_t)page_size + nva_v_offset(off, 0, head_dim, vt);
                float dot = 0.f;
                if (vec) {
                    for (int d = 0; d < head_dim; d += 8) {
                        float kk[8];
                        load8(krow + d, kk);
#pragma unroll
                        for (int e = 0; e < 8; ++e) dot += q_s[d + e] * kk[e];
                    }
                } else {
                    for (int d = 0; d < head_dim; ++d) dot += q_s[d] * to_float(krow[d]);
                }
                s = dot * scale;
            }
        }
        const float m_new = fmaxf(m_run, wave_max(s));
        // m_new is finite: the key at `pos` itself is always visible in the first chunk that holds it;
        // a chunk of only faulty keys leaves m_new at -inf, guarded below.
        const float p = (s == -INFINITY) ? 0.f : nva_exp(s - m_new);
        const float correction = (m_run == -INFINITY) ? 0.f : nva_exp(m_run - m_new);
        l_run = l_run * correction + wave_sum(p);
        m_run = m_new;
        __syncthreads();
        p_s[lane] = p;
        v_off_s[lane] = v_off;
        __syncthreads();
        const int valid = pos - base + 1 < NVA_WAVE ? pos - base + 1 : NVA_WAVE;
#pragma unroll
        for (int i = 0; i < ATT_ACC; ++i) {
            const int d = lane + i * NVA_WAVE;
            if (d < head_dim) {
                float a = acc[i] * correction;
                const T* vcol = v_cache + (int64_t)d * vt;
                for (int jj = 0; jj < valid; ++jj) {
                    const float pj = p_s[jj];
                    if (pj != 0.f) a += pj * to_float(vcol[v_off_s[jj]]);
                }
                acc[i] = a;
            }
        }
    }
    const float inv = l_run > 0.f ? 1.f / l_run : 0.f;
    T* orow = out + t * out_stride + (int64_t)h * head_dim;
#pragma unroll
    for (int i = 0; i < ATT_ACC; ++i) {
        const int d = lane + i * NVA_WAVE;
        if (d < head_dim) orow[d] = from_float<T>(acc[i] * inv);
    }
}

NVA_EXPORT int NVA_NAME(nva_paged_attention_generic)(
    const void* q, int64_t q_stride, void* out, int64_t out_stride, const void* k_cache, const void* v_cache,
    const int32_t* block_tables, int table_stride, const int32_t* token_seq, const int32_t* positions,
    int64_t tokens, int num_q_heads, int num_kv_heads, int head_dim, int page_size, float scale, int window,
    int32_t* error_flag, hipStream_t stream) {
    if (tokens == 0) return 0;
    if (tokens < 0 || tokens > 0x7fffffff) return nva_fail("paged_attention: bad token count %lld", (long long)tokens);
    if (num_q_heads <= 0 || num_kv_heads <= 0 || num_q_heads % num_kv_heads || num_q_heads > 65535)
        return nva_fail("paged_attention: %d query heads do not divide into %d kv heads", num_q_heads, num_kv_heads);
    if (head_dim <= 0 || head_dim > ATT_MAX_D)
        return nva_fail("paged_attention: head_dim %d is outside 1..%d", head_dim, ATT_MAX_D);
    if (page_size <= 0 || table_stride <= 0) return nva_fail("paged_attention: bad page size or table width");
    if (window < 0) return nva_fail("paged_attention: negative window");
    dim3 grid((unsigned)tokens, (unsigned)num_q_heads);
    hipLaunchKernelGGL(paged_attention_generic_kernel<elem_t>, grid, dim3(NVA_WAVE), 0, stream, (const elem_t*)q,
                       q_stride, (elem_t*)out, out_stride, (const elem_t*)k_cache, (const elem_t*)v_cache,
                       block_tables, table_stride, token_seq, positions, num_q_heads, num_kv_heads, head_dim,
                       page_size, scale, window, error_flag);
    return nva_check_launch("paged_attention_generic");
}

NVA_DEFINE_LAST_ERROR(nva_attn_generic)
