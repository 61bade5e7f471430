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
//
// Portions of prompts have a second kernel with the same arithmetic, operation for operation (the
// results are the same bits): a workgroup takes 32 query rows of one request and one head, and the
// chunks of 64 keys that the per-token kernel would fetch for every row by itself are staged in LDS
// once for all of them (without a window every row's chunks start at key 0, so the rows share them).
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
                    int d = 0;
                    for (; d + 32 <= head_dim; d += 32) {           // four loads on their way at once; the sum stays one chain
                        float kk[4][8];
#pragma unroll
                        for (int u = 0; u < 4; ++u) load8(krow + d + 8 * u, kk[u]);
#pragma unroll
                        for (int u = 0; u < 4; ++u)
#pragma unroll
                            for (int e = 0; e < 8; ++e) dot += q_s[d + 8 * u + e] * kk[u][e];
                    }
                    for (; d < head_dim; d += 8) {
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
                int jj = 0;
                for (; jj + 8 <= valid; jj += 8) {                   // eight loads on their way at once
                    float vv[8];
#pragma unroll
                    for (int u = 0; u < 8; ++u) vv[u] = to_float(vcol[v_off_s[jj + u]]);
#pragma unroll
                    for (int u = 0; u < 8; ++u) {
                        const float pj = p_s[jj + u];
                        const float with = a + pj * vv[u];
                        a = pj != 0.f ? with : a;                    // a key of weight zero adds nothing, whatever V holds
                    }
                }
                for (; jj < valid; ++jj) {
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

template <int N> struct Count { static constexpr int value = N; };

#define ATT_ROWS 32              // query rows of a workgroup of the tiled kernel
#define ATT_TILED_MAX_D 128      // its head sizes: two accumulators per lane, the tiles in LDS
#define ATT_TILED_WAVES 8

// floats of LDS the tiled kernel needs: the queries, a chunk of K (rows of an odd length: a lane per
// key reads them side by side) and of V (channel-major, rows of 65)
__host__ __device__ inline size_t att_tiled_lds(int head_dim) {
    return ((size_t)ATT_ROWS * head_dim + (size_t)NVA_WAVE * (head_dim | 1) + (size_t)head_dim * (NVA_WAVE + 1)) * sizeof(float);
}

template <typename T>
__global__ void __launch_bounds__(ATT_TILED_WAVES * NVA_WAVE)
paged_attention_tiled_kernel(const T* __restrict__ q, int64_t q_stride, T* __restrict__ out, int64_t out_stride,
                             const T* __restrict__ k_cache, const T* __restrict__ v_cache,
                             const int32_t* __restrict__ block_tables, int table_stride,
                             const int32_t* __restrict__ cu_seqlens_q, const int32_t* __restrict__ kv_lens,
                             const int32_t* __restrict__ tiles, int num_q_heads, int num_kv_heads, int head_dim,
                             int page_size, float scale, int32_t* error_flag) {
    extern __shared__ __attribute__((aligned(16))) float lds[];
    __shared__ int64_t k_off_s[NVA_WAVE], v_off_s[NVA_WAVE];       // of a chunk's keys; -1: the key has no page
    constexpr int ROWS_PER_WAVE = ATT_ROWS / ATT_TILED_WAVES;
    constexpr int ACC = ATT_TILED_MAX_D / NVA_WAVE;
    const int DS = head_dim | 1;
    float* const q_s = lds;                                         // [ATT_ROWS][head_dim]
    float* const k_s = q_s + ATT_ROWS * head_dim;                   // [64 keys][DS]
    float* const v_s = k_s + NVA_WAVE * DS;                         // [head_dim][65]

    const int seq = tiles[2 * blockIdx.x], tile = tiles[2 * blockIdx.x + 1];
    const int h = blockIdx.y;
    const int kvh = h / (num_q_heads / num_kv_heads);
    const int q_begin = cu_seqlens_q[seq];
    const int q_len = cu_seqlens_q[seq + 1] - q_begin;
    const int start = kv_lens[seq] - q_len;                          // position of the request's first query of this step
    const int q0 = tile * ATT_ROWS;
    const int rows = min(ATT_ROWS, q_len - q0);
    const int last_pos = start + q0 + rows - 1;
    const int32_t* table = block_tables + (int64_t)seq * table_stride;
    const int tid = threadIdx.x, lane = tid % NVA_WAVE, wave = tid / NVA_WAVE;
    const int vt = nva_v_tile(page_size);
    const bool vec = head_dim % 8 == 0;

    for (int i = tid; i < rows * head_dim; i += blockDim.x) {
        const int r = i / head_dim, d = i % head_dim;
        q_s[i] = to_float(q[(int64_t)(q_begin + q0 + r) * q_stride + (int64_t)h * head_dim + d]);
    }

    float acc[ROWS_PER_WAVE][ACC], m_run[ROWS_PER_WAVE], l_run[ROWS_PER_WAVE];
#pragma unroll
    for (int r = 0; r < ROWS_PER_WAVE; ++r) {
#pragma unroll
        for (int i = 0; i < ACC; ++i) acc[r][i] = 0.f;
        m_run[r] = -INFINITY, l_run[r] = 0.f;
    }

    for (int base = 0; base <= last_pos; base += NVA_WAVE) {
        __syncthreads();                                             // the chunk before is done with (and q_s is written)
        if (tid < NVA_WAVE) {
            const int j = base + tid;
            int64_t k_off = -1, v_off = -1;
            if (j <= last_pos) {
                const int page = table[j / page_size];
                const int off = j % page_size;
                if (page < 0) {
                    if (error_flag) atomicOr(error_flag, 2);          // a visible key has no page
                } else {
                    const int64_t head_base = (int64_t)page * num_kv_heads + kvh;
                    k_off = (head_base * page_size + off) * head_dim;
                    v_off = head_base * head_dim * (int64_t)page_size + nva_v_offset(off, 0, head_dim, vt);
                }
            }
            k_off_s[tid] = k_off;
            v_off_s[tid] = v_off;
        }
        __syncthreads();
        // (loads in batches, so that a thread has several on their way at once)
        if (vec) {
            constexpr int B = 4;
            for (int i0 = tid; i0 < NVA_WAVE * head_dim / 8; i0 += B * blockDim.x) {
                float kk[B][8];
#pragma unroll
                for (int u = 0; u < B; ++u) {
                    const int i = i0 + u * blockDim.x;
                    const int j = i / (head_dim / 8), d = (i % (head_dim / 8)) * 8;
                    if (i < NVA_WAVE * head_dim / 8 && k_off_s[j] >= 0) load8(k_cache + k_off_s[j] + d, kk[u]);
                    else {
#pragma unroll
                        for (int e = 0; e < 8; ++e) kk[u][e] = 0.f;
                    }
                }
#pragma unroll
                for (int u = 0; u < B; ++u) {
                    const int i = i0 + u * blockDim.x;
                    const int j = i / (head_dim / 8), d = (i % (head_dim / 8)) * 8;
                    if (i < NVA_WAVE * head_dim / 8) {
#pragma unroll
                        for (int e = 0; e < 8; ++e) k_s[j * DS + d + e] = kk[u][e];
                    }
                }
            }
        } else {
            for (int i = tid; i < NVA_WAVE * head_dim; i += blockDim.x) {
                const int j = i / head_dim, d = i % head_dim;
                k_s[j * DS + d] = k_off_s[j] >= 0 ? to_float(k_cache[k_off_s[j] + d]) : 0.f;
            }
        }
        {
            // a thread's key is the same in every turn (256 is a multiple of 64): j = tid % 64, channels tid / 64 + 4 n
            constexpr int B = 8;
            const int j = tid % NVA_WAVE;
            const int64_t v_off = v_off_s[j];
            for (int d0 = tid / NVA_WAVE; d0 < head_dim; d0 += B * ATT_TILED_WAVES) {
                float vv[B];
#pragma unroll
                for (int u = 0; u < B; ++u) {
                    const int d = d0 + u * ATT_TILED_WAVES;
                    vv[u] = d < head_dim && v_off >= 0 ? to_float(v_cache[v_off + (int64_t)d * vt]) : 0.f;
                }
#pragma unroll
                for (int u = 0; u < B; ++u) {
                    const int d = d0 + u * ATT_TILED_WAVES;
                    if (d < head_dim) v_s[d * (NVA_WAVE + 1) + j] = vv[u];
                }
            }
        }
        __syncthreads();

        // A wave's rows four at a time: their sums are chains of their own, which fill each other's
        // waits, and what is read of K and V serves all four.  A row that sees nothing of the chunk (or
        // is past the portion's end: position -1) goes through it with every score masked, which leaves
        // its maximum, sum and accumulators as they are, bit for bit.
#pragma unroll
        for (int quad = 0; quad < ROWS_PER_WAVE / 4; ++quad) {
            int pos4[4], last4 = -1;
#pragma unroll
            for (int t = 0; t < 4; ++t) {
                const int r = wave + ATT_TILED_WAVES * (4 * quad + t);
                pos4[t] = r < rows ? start + q0 + r : -1;
                last4 = max(last4, pos4[t]);
            }
            if (base > last4) continue;                              // (the same for the whole wave)
            const float* kr = k_s + lane * DS;
            const float* qr = q_s + (wave + ATT_TILED_WAVES * 4 * quad) * head_dim;      // row t of the quad: + 4 t head_dim
            float dot[4] = {0.f, 0.f, 0.f, 0.f};
            int d = 0;
            for (; d + 8 <= head_dim; d += 8) {
                float kk[8], qq[4][8];
#pragma unroll
                for (int e = 0; e < 8; ++e) kk[e] = kr[d + e];
#pragma unroll
                for (int t = 0; t < 4; ++t) {
                    const float* qt = qr + ATT_TILED_WAVES * t * head_dim + d;           // the same address in every lane
                    if (head_dim % 4 == 0) {
                        const float4 lo = *reinterpret_cast<const float4*>(qt), hi = *reinterpret_cast<const float4*>(qt + 4);
                        qq[t][0] = lo.x, qq[t][1] = lo.y, qq[t][2] = lo.z, qq[t][3] = lo.w;
                        qq[t][4] = hi.x, qq[t][5] = hi.y, qq[t][6] = hi.z, qq[t][7] = hi.w;
                    } else {
#pragma unroll
                        for (int e = 0; e < 8; ++e) qq[t][e] = qt[e];
                    }
                }
#pragma unroll
                for (int e = 0; e < 8; ++e)
#pragma unroll
                    for (int t = 0; t < 4; ++t) dot[t] += qq[t][e] * kk[e];
            }
            for (; d < head_dim; ++d)
#pragma unroll
                for (int t = 0; t < 4; ++t) dot[t] += qr[ATT_TILED_WAVES * t * head_dim + d] * kr[d];
            const bool key_ok = k_off_s[lane] >= 0;
            float p[4];
#pragma unroll
            for (int t = 0; t < 4; ++t) {
                const int rr = 4 * quad + t;
                const float s = base + lane <= pos4[t] && key_ok ? dot[t] * scale : -INFINITY;
                const float m_new = fmaxf(m_run[rr], wave_max(s));
                p[t] = (s == -INFINITY) ? 0.f : nva_exp(s - m_new);
                const float correction = (m_run[rr] == -INFINITY) ? 0.f : nva_exp(m_run[rr] - m_new);
                l_run[rr] = l_run[rr] * correction + wave_sum(p[t]);
                m_run[rr] = m_new;
#pragma unroll
                for (int i = 0; i < ACC; ++i) acc[rr][i] *= correction;
            }
            // channel d = lane + 64 i adds its keys in ascending order, as in the per-token kernel; a key
            // of weight zero (masked, or beyond the row's position) adds nothing, whatever V holds
            const int valid = last4 - base + 1 < NVA_WAVE ? last4 - base + 1 : NVA_WAVE;
            auto add_keys = [&](int jj, auto count) __attribute__((always_inline)) {
                constexpr int N = decltype(count)::value;
                float pj[4][N], vv[ACC][N];
#pragma unroll
                for (int u = 0; u < N; ++u) {
#pragma unroll
                    for (int t = 0; t < 4; ++t) pj[t][u] = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(p[t]), jj + u));
#pragma unroll
                    for (int i = 0; i < ACC; ++i) {
                        const int dd = lane + i * NVA_WAVE;
                        vv[i][u] = dd < head_dim ? v_s[dd * (NVA_WAVE + 1) + jj + u] : 0.f;
                    }
                }
#pragma unroll
                for (int u = 0; u < N; ++u)
#pragma unroll
                    for (int t = 0; t < 4; ++t)
#pragma unroll
                        for (int i = 0; i < ACC; ++i) {
                            const float with = acc[4 * quad + t][i] + pj[t][u] * vv[i][u];
                            acc[4 * quad + t][i] = pj[t][u] != 0.f ? with : acc[4 * quad + t][i];
                        }
            };
            int jj = 0;
            for (; jj + 8 <= valid; jj += 8) add_keys(jj, Count<8>());
            for (; jj < valid; ++jj) add_keys(jj, Count<1>());
        }
    }
#pragma unroll
    for (int rr = 0; rr < ROWS_PER_WAVE; ++rr) {
        const int r = wave + ATT_TILED_WAVES * rr;
        if (r >= rows) continue;
        const float inv = l_run[rr] > 0.f ? 1.f / l_run[rr] : 0.f;
        T* orow = out + (int64_t)(q_begin + q0 + r) * out_stride + (int64_t)h * head_dim;
#pragma unroll
        for (int i = 0; i < ACC; ++i) {
            const int d = lane + i * NVA_WAVE;
            if (d < head_dim) orow[d] = from_float<T>(acc[rr][i] * inv);
        }
    }
}

// The same attention for portions of prompts, 32 rows of a request to a workgroup: tiles is int32
// [num_tiles][2] = (request, row tile of 32 queries), requests described by cu_seqlens_q and kv_lens as
// for the matrix-core kernel.  No window, head sizes up to 128; returns 1 for what it does not take.
NVA_EXPORT int NVA_NAME(nva_paged_attention_tiled)(
    const void* q, int64_t q_stride, void* out, int64_t out_stride, const void* k_cache, const void* v_cache,
    const int32_t* block_tables, int table_stride, const int32_t* cu_seqlens_q, const int32_t* kv_lens,
    const int32_t* tiles, int64_t num_tiles, int num_q_heads, int num_kv_heads, int head_dim, int page_size,
    float scale, int32_t* error_flag, hipStream_t stream) {
    if (num_tiles == 0) return 0;
    if (head_dim <= 0 || head_dim > ATT_TILED_MAX_D) {
        nva_fail("paged_attention_tiled: head_dim %d is outside 1..%d", head_dim, ATT_TILED_MAX_D);
        return 1;
    }
    if (!tiles || num_tiles < 0 || num_tiles > 0x7fffffff) return nva_fail("paged_attention_tiled: bad tile count %lld", (long long)num_tiles);
    if (num_q_heads <= 0 || num_kv_heads <= 0 || num_q_heads % num_kv_heads || num_q_heads > 65535)
        return nva_fail("paged_attention_tiled: %d query heads do not divide into %d kv heads", num_q_heads, num_kv_heads);
    if (page_size <= 0 || table_stride <= 0) return nva_fail("paged_attention_tiled: bad page size or table width");
    const size_t lds = att_tiled_lds(head_dim);
    auto kernel = paged_attention_tiled_kernel<elem_t>;
    static bool raised = false;              // the kernel's LDS limit, lifted once to what the largest head size needs
    if (!raised) {
        if (hipFuncSetAttribute((const void*)kernel, hipFuncAttributeMaxDynamicSharedMemorySize, (int)att_tiled_lds(ATT_TILED_MAX_D)) != hipSuccess)
            return nva_fail("paged_attention_tiled: cannot have %zu bytes of LDS", att_tiled_lds(ATT_TILED_MAX_D));
        raised = true;
    }
    dim3 grid((unsigned)num_tiles, (unsigned)num_q_heads);
    hipLaunchKernelGGL(kernel, grid, dim3(ATT_TILED_WAVES * NVA_WAVE), lds, stream, (const elem_t*)q, q_stride,
                       (elem_t*)out, out_stride, (const elem_t*)k_cache, (const elem_t*)v_cache, block_tables,
                       table_stride, cu_seqlens_q, kv_lens, tiles, num_q_heads, num_kv_heads, head_dim, page_size,
                       scale, error_flag);
    return nva_check_launch("paged_attention_tiled");
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
