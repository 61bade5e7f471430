// Position encoding and the write into the paged cache, in one pass over a step's q, k and v.
//
// For every token and head of the packed projection row [q heads | k heads | v heads]:
//   q, k:  optional per-head RMS norm over the head (nanovllm/models/qwen3.py:68-70,82-84),
//          then the rotation of pairs (i, i + rot/2) by the angle table's row of the token's
//          position (nanovllm/layers/rotary_embedding.py:6-14,44-47), in float, one rounding;
//          rot, the table's width, is the head size there; a smaller even rot rotates the first
//          rot channels of the head and leaves the others as they are;
//          q is written back in place, k in place and into its page slot;
//   v:     copied into its page slot (nanovllm/layers/attention.py:10-30), stored transposed.
// Cache layouts: K [pages, kv_heads, page_size, head_dim], V transposed in tiles of keys (common.h).
// slot = page * page_size + offset; slot -1 writes nothing into the cache.
#include "common.h"

// table[p, 0:half] = cos(p * inv_freq), table[p, half:2*half] = sin(p * inv_freq); the product
// p * inv_freq is one float multiplication, as the reference's outer product
// (rotary_embedding.py:30-31).
__global__ void rotary_table_kernel(const float* __restrict__ inv_freq, int half, int64_t positions,
                                    float* __restrict__ table) {
    const int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (idx >= positions * half) return;
    const int64_t p = idx / half;
    const int i = (int)(idx % half);
    const float angle = (float)p * inv_freq[i];
    table[p * 2 * half + i] = cosf(angle);
    table[p * 2 * half + half + i] = sinf(angle);
}

NVA_EXPORT int NVA_NAME(nva_rotary_table)(const float* inv_freq, int half, int64_t positions, float* table,
                                          hipStream_t stream) {
    if (half <= 0 || positions <= 0) return nva_fail("rotary_table: bad shape half=%d positions=%lld", half, (long long)positions);
    const int64_t n = positions * half;
    hipLaunchKernelGGL(rotary_table_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, stream, inv_freq, half,
                       positions, table);
    return nva_check_launch("rotary_table");
}

#define NVA_MAX_PER_LANE 4   // head_dim / 2 <= 64 * 4

template <typename T>
__global__ void __launch_bounds__(256)
qk_norm_rope_store_kernel(T* qkv, int64_t row_stride, PartialInput part, T* q_out, int64_t q_out_stride,
                          int num_q_heads, int num_kv_heads, int head_dim,
                          const void* __restrict__ q_weight, const void* __restrict__ k_weight, int w_is_f32,
                          float eps, const float* __restrict__ table, int rot_dim,
                          const int32_t* __restrict__ positions, const int32_t* __restrict__ slots,
                          T* k_cache, T* v_cache, int page_size) {
    const int64_t t = blockIdx.x;
    const int lane = threadIdx.x % NVA_WAVE;
    const int head = blockIdx.y * (blockDim.x / NVA_WAVE) + threadIdx.x / NVA_WAVE;
    const int total_heads = num_q_heads + 2 * num_kv_heads;
    if (head >= total_heads) return;
    // The row comes from qkv, or (a product left as partial sums) from `part`; then q goes to q_out
    // and k only into the cache.
    T* row = part.sums ? nullptr : qkv + t * row_stride + (int64_t)head * head_dim;
    const int row_width = (num_q_heads + 2 * num_kv_heads) * head_dim;
    const int col0 = head * head_dim;
    const int64_t slot = slots ? slots[t] : -1;
    // A lane holds pairs of channels (a, b): pair i < rot/2 is (i, i + rot/2), which the rotation
    // turns; the channels from rot on are paired among themselves, (rot + i', rot + i' + rest/2),
    // and only normed.  With rot = head_dim these are the pairs (i, i + head_dim/2).
    const int half = head_dim / 2, rot_half = rot_dim / 2, rest_half = (head_dim - rot_dim) / 2;
#define PAIR_A(i) ((i) < rot_half ? (i) : rot_dim + (i) - rot_half)
#define PAIR_B(i) ((i) < rot_half ? (i) + rot_half : rot_dim + (i) - rot_half + rest_half)

    if (head >= num_q_heads + num_kv_heads) {                       // a v head: copy, transposed
        if (slot < 0 || !v_cache) return;
        const int h = head - num_q_heads - num_kv_heads;
        const int64_t page = slot / page_size, off = slot % page_size;
        T* dst = v_cache + ((page * num_kv_heads + h) * (int64_t)head_dim) * page_size;
        const int vt = nva_v_tile(page_size);
        for (int d = lane; d < head_dim; d += NVA_WAVE)
            dst[nva_v_offset((int)off, d, head_dim, vt)] = part.sums ? from_float<T>(partial_value<T>(part, t, row_width, col0 + d)) : row[d];
        return;
    }

    const bool is_q = head < num_q_heads;
    const void* weight = is_q ? q_weight : k_weight;
    float x1[NVA_MAX_PER_LANE], x2[NVA_MAX_PER_LANE];
    float ss = 0.f;
#pragma unroll
    for (int j = 0; j < NVA_MAX_PER_LANE; ++j) {
        const int i = lane + j * NVA_WAVE;
        x1[j] = x2[j] = 0.f;
        if (i < half) {
            const int a = PAIR_A(i), b = PAIR_B(i);
            x1[j] = part.sums ? partial_value<T>(part, t, row_width, col0 + a) : to_float(row[a]);
            x2[j] = part.sums ? partial_value<T>(part, t, row_width, col0 + b) : to_float(row[b]);
            ss += x1[j] * x1[j] + x2[j] * x2[j];
        }
    }
    if (weight) {
        ss = wave_sum(ss);
        const float scale = rsqrtf(ss / (float)head_dim + eps);
#pragma unroll
        for (int j = 0; j < NVA_MAX_PER_LANE; ++j) {
            const int i = lane + j * NVA_WAVE;
            if (i < half) {
                const int a = PAIR_A(i), b = PAIR_B(i);
                const float w1 = w_is_f32 ? ((const float*)weight)[a] : to_float(((const T*)weight)[a]);
                const float w2 = w_is_f32 ? ((const float*)weight)[b] : to_float(((const T*)weight)[b]);
                x1[j] = round_through<T>(round_through<T>(x1[j] * scale) * w1);
                x2[j] = round_through<T>(round_through<T>(x2[j] * scale) * w2);
            }
        }
    }
    // Rotation of the pair (i, i + rot/2), which is exactly (x1, x2).  The table row holds
    // rot/2 cosines, then rot/2 sines.
    const float* angles = table ? table + (int64_t)positions[t] * rot_dim : nullptr;
    T* k_dst = nullptr;
    if (!is_q && slot >= 0 && k_cache) {
        const int h = head - num_q_heads;
        const int64_t page = slot / page_size, off = slot % page_size;
        k_dst = k_cache + ((page * num_kv_heads + h) * (int64_t)page_size + off) * head_dim;
    }
    if (angles) {
#pragma unroll
        for (int j = 0; j < NVA_MAX_PER_LANE; ++j) {
            const int i = lane + j * NVA_WAVE;
            if (i < rot_half) {
                const float c = angles[i], s = angles[rot_half + i];
                const float y1 = x1[j] * c - x2[j] * s;
                const float y2 = x2[j] * c + x1[j] * s;
                x1[j] = y1;
                x2[j] = y2;
            }
        }
    }
#pragma unroll
    for (int j = 0; j < NVA_MAX_PER_LANE; ++j) {
        const int i = lane + j * NVA_WAVE;
        if (i < half) {
            const T a = from_float<T>(x1[j]), b = from_float<T>(x2[j]);
            const int ia = PAIR_A(i), ib = PAIR_B(i);
            if (!part.sums) {
                row[ia] = a;
                row[ib] = b;
            } else if (is_q) {
                T* qo = q_out + t * q_out_stride + col0;
                qo[ia] = a;
                qo[ib] = b;
            }
            if (k_dst) {
                k_dst[ia] = a;
                k_dst[ib] = b;
            }
        }
    }
#undef PAIR_A
#undef PAIR_B
}

// The same work for many tokens at once (portions of prompts).  A workgroup of 256 threads takes
// one head of 256 / LPH consecutive tokens, LPH = head_dim / 16 lanes per token: a lane holds the
// eight elements 8p.. of the head's first half and the eight of its second half that pair with them,
// so every access is a 16-byte (32-byte in float) vector and the norm's sum crosses LPH lanes only.
// A v head goes through LDS, and where 32 tokens in a row have 32 slots in a row that start a key
// tile of the V cache, a lane writes eight keys of one channel at once.
template <typename T, int LPH>
__global__ void __launch_bounds__(256)
qk_norm_rope_store_tile_kernel(T* qkv, int64_t row_stride, int tokens, int num_q_heads, int num_kv_heads,
                               const void* __restrict__ q_weight, const void* __restrict__ k_weight, int w_is_f32,
                               float eps, const float* __restrict__ table, const int32_t* __restrict__ positions,
                               const int32_t* __restrict__ slots, T* k_cache, T* v_cache, int page_size) {
    constexpr int D = 16 * LPH, HALF = 8 * LPH, TB = 256 / LPH, VS = TB + 8 / (int)sizeof(T) * 2;
    __shared__ __attribute__((aligned(16))) T v_s[D * VS];
    __shared__ int run_ok[(TB + 31) / 32];
    const int tid = threadIdx.x, r = tid / LPH, p = tid % LPH;
    const int head = blockIdx.y;
    const int t0 = blockIdx.x * TB, t = t0 + r;
    const bool live = t < tokens;
    T* row = qkv + (int64_t)(live ? t : 0) * row_stride + (int64_t)head * D;
    const int64_t slot = live && slots ? slots[t] : -1;
    float x1[8], x2[8];
    load8(row + 8 * p, x1);
    load8(row + HALF + 8 * p, x2);

    if (head >= num_q_heads + num_kv_heads) {                       // a v head
        if (!v_cache) return;
        const int h = head - num_q_heads - num_kv_heads;
        const int vt = nva_v_tile(page_size);
        // runs of 32 tokens whose slots are 32 in a row from the start of a key tile
        if (tid < (TB + 31) / 32) run_ok[tid] = vt == 32 ? 1 : 0;
        __syncthreads();
        const int run = r / 32;
        const int64_t run_slot = (t0 + run * 32 < tokens && slots) ? slots[t0 + run * 32] : -1;
        if (!(live && run_slot >= 0 && run_slot % 32 == 0 && slot == run_slot + r % 32)) run_ok[run] = 0;
#pragma unroll
        for (int e = 0; e < 8; ++e) {
            v_s[(8 * p + e) * VS + r] = from_float<T>(x1[e]);
            v_s[(HALF + 8 * p + e) * VS + r] = from_float<T>(x2[e]);
        }
        __syncthreads();
        // pieces of eight keys of one channel: TB / 8 per channel
        for (int idx = tid; idx < D * (TB / 8); idx += 256) {
            const int d = idx / (TB / 8), piece = idx % (TB / 8);
            const int tok = piece * 8;                               // first token of the piece within the block
            if (run_ok[tok / 32]) {
                const int64_t s0 = slots[t0 + (tok & ~31)];
                const int64_t page = s0 / page_size, off = s0 % page_size + (tok & 31);
                T* dst = v_cache + ((page * num_kv_heads + h) * (int64_t)D) * page_size + nva_v_offset((int)off, d, D, vt);
                float v[8];
                load8(&v_s[d * VS + tok], v);
                store8(dst, v);
            } else {
                for (int e = 0; e < 8; ++e) {
                    const int tt = t0 + tok + e;
                    const int64_t se = tt < tokens && slots ? slots[tt] : -1;
                    if (se < 0) continue;
                    const int64_t page = se / page_size, off = se % page_size;
                    v_cache[((page * num_kv_heads + h) * (int64_t)D) * page_size + nva_v_offset((int)off, d, D, vt)] =
                        v_s[d * VS + tok + e];
                }
            }
        }
        return;
    }

    const bool is_q = head < num_q_heads;
    const void* weight = is_q ? q_weight : k_weight;
    if (weight) {
        float ss = 0.f;
#pragma unroll
        for (int e = 0; e < 8; ++e) ss += x1[e] * x1[e] + x2[e] * x2[e];
#pragma unroll
        for (int o = LPH / 2; o > 0; o >>= 1) ss += __shfl_xor(ss, o, NVA_WAVE);
        const float scale = rsqrtf(ss / (float)D + eps);
        float w1[8], w2[8];
        if (w_is_f32) {
            load8((const float*)weight + 8 * p, w1);
            load8((const float*)weight + HALF + 8 * p, w2);
        } else {
            load8((const T*)weight + 8 * p, w1);
            load8((const T*)weight + HALF + 8 * p, w2);
        }
#pragma unroll
        for (int e = 0; e < 8; ++e) {
            x1[e] = round_through<T>(round_through<T>(x1[e] * scale) * w1[e]);
            x2[e] = round_through<T>(round_through<T>(x2[e] * scale) * w2[e]);
        }
    }
    if (table) {
        const float* angles = table + (int64_t)(live ? positions[t] : 0) * D;
        float c[8], sn[8];
        load8(angles + 8 * p, c);
        load8(angles + HALF + 8 * p, sn);
#pragma unroll
        for (int e = 0; e < 8; ++e) {
            const float y1 = x1[e] * c[e] - x2[e] * sn[e];
            const float y2 = x2[e] * c[e] + x1[e] * sn[e];
            x1[e] = y1;
            x2[e] = y2;
        }
    }
    if (!live) return;
    store8(row + 8 * p, x1);
    store8(row + HALF + 8 * p, x2);
    if (!is_q && slot >= 0 && k_cache) {
        const int h = head - num_q_heads;
        const int64_t page = slot / page_size, off = slot % page_size;
        T* dst = k_cache + ((page * num_kv_heads + h) * (int64_t)page_size + off) * D;
        store8(dst + 8 * p, x1);
        store8(dst + HALF + 8 * p, x2);
    }
}

static int launch_qk(elem_t* qkv, int64_t row_stride, PartialInput part, elem_t* q_out, int64_t q_out_stride,
                     int64_t tokens, int num_q_heads, int num_kv_heads, int head_dim, const void* q_weight,
                     const void* k_weight, int w_is_f32, float eps, const float* table, int rot_dim,
                     const int32_t* positions, const int32_t* slots, void* k_cache, void* v_cache, int page_size,
                     hipStream_t stream) {
    if (tokens == 0) return 0;
    if (tokens < 0 || tokens > 0x7fffffff) return nva_fail("qk_norm_rope_store: bad token count %lld", (long long)tokens);
    if (num_q_heads < 0 || num_kv_heads < 0 || num_q_heads + num_kv_heads == 0 || head_dim <= 0)
        return nva_fail("qk_norm_rope_store: bad heads q=%d kv=%d head_dim=%d", num_q_heads, num_kv_heads, head_dim);
    if (head_dim % 2 || head_dim / 2 > NVA_WAVE * NVA_MAX_PER_LANE)
        return nva_fail("qk_norm_rope_store: head_dim %d must be even and at most %d", head_dim,
                        2 * NVA_WAVE * NVA_MAX_PER_LANE);
    if ((k_cache || v_cache) && (page_size <= 0 || !slots))
        return nva_fail("qk_norm_rope_store: a cache needs a page size and slots");
    if (table && !positions) return nva_fail("qk_norm_rope_store: a rotation table needs positions");
    if (!table) rot_dim = head_dim;
    if (rot_dim <= 0 || rot_dim % 2 || rot_dim > head_dim)
        return nva_fail("qk_norm_rope_store: a rotation of %d channels of a head of %d: it must be even and at most the head",
                        rot_dim, head_dim);
    const int total = num_q_heads + 2 * num_kv_heads;
    // many tokens of a finished projection: the tiled kernel, where the head size has an instance
    // and the rows can be read in vectors
    const int lph = head_dim / 16;
    if (!part.sums && tokens >= 64 && rot_dim == head_dim && head_dim % 16 == 0 && (lph & (lph - 1)) == 0 && lph <= 16 && total <= 65535 &&
        row_stride % 8 == 0 && nva_aligned(qkv, 32) && (!q_weight || nva_aligned(q_weight, 32)) &&
        (!k_weight || nva_aligned(k_weight, 32)) && nva_aligned(table, 32) && nva_aligned(k_cache, 32) &&
        nva_aligned(v_cache, 32)) {
        const int tb = 256 / lph;
        dim3 tgrid((unsigned)((tokens + tb - 1) / tb), (unsigned)total);
#define TILE(LPH)                                                                                                      \
    hipLaunchKernelGGL((qk_norm_rope_store_tile_kernel<elem_t, LPH>), tgrid, dim3(256), 0, stream, qkv, row_stride,   \
                       (int)tokens, num_q_heads, num_kv_heads, q_weight, k_weight, w_is_f32, eps, table, positions,  \
                       slots, (elem_t*)k_cache, (elem_t*)v_cache, page_size)
        switch (lph) {
            case 1: TILE(1); break;
            case 2: TILE(2); break;
            case 4: TILE(4); break;
            case 8: TILE(8); break;
            default: TILE(16); break;
        }
#undef TILE
        return nva_check_launch("qk_norm_rope_store_tile");
    }
    const int waves = 4;
    dim3 grid((unsigned)tokens, (total + waves - 1) / waves);
    hipLaunchKernelGGL(qk_norm_rope_store_kernel<elem_t>, grid, dim3(waves * NVA_WAVE), 0, stream, qkv, row_stride, part,
                       q_out, q_out_stride, num_q_heads, num_kv_heads, head_dim, q_weight, k_weight, w_is_f32, eps, table, rot_dim,
                       positions, slots, (elem_t*)k_cache, (elem_t*)v_cache, page_size);
    return nva_check_launch("qk_norm_rope_store");
}

// qkv rows hold [q heads | k heads | v heads] of head_dim each.  q_weight / k_weight may be null
// (no norm), table may be null (no rotation), the caches may be null (nothing is stored).
// table rows are rot_dim wide (cosines, then sines), rot_dim even and at most head_dim.
// The kernels read table + positions[t] * rot_dim unchecked: the host wrapper takes the largest
// position of the step and refuses one that is not a row of the table.
NVA_EXPORT int NVA_NAME(nva_qk_norm_rope_store)(void* qkv, int64_t row_stride, int64_t tokens, int num_q_heads,
                                                int num_kv_heads, int head_dim, const void* q_weight,
                                                const void* k_weight, int w_is_f32, float eps, const float* table,
                                                int rot_dim, const int32_t* positions, const int32_t* slots,
                                                void* k_cache, void* v_cache, int page_size, hipStream_t stream) {
    return launch_qk((elem_t*)qkv, row_stride, PartialInput{nullptr, 0, 0, nullptr}, nullptr, 0, tokens, num_q_heads,
                     num_kv_heads, head_dim, q_weight, k_weight, w_is_f32, eps, table, rot_dim, positions, slots, k_cache,
                     v_cache, page_size, stream);
}

// The same with the packed projection given as float partial sums [splits][tokens][row width]
// (+ bias): q is written to q_out [tokens, q heads * head_dim], k and v only into the cache.
NVA_EXPORT int NVA_NAME(nva_qk_norm_rope_store_of_partials)(
    const float* sums, int splits, int64_t split_stride, const void* bias, void* q_out, int64_t q_out_stride,
    int64_t tokens, int num_q_heads, int num_kv_heads, int head_dim, const void* q_weight, const void* k_weight,
    int w_is_f32, float eps, const float* table, int rot_dim, const int32_t* positions, const int32_t* slots,
    void* k_cache, void* v_cache, int page_size, hipStream_t stream) {
    if (!sums || splits <= 0 || !q_out) return nva_fail("qk_norm_rope_store_of_partials: no partial sums or no output");
    return launch_qk(nullptr, 0, PartialInput{sums, splits, split_stride, bias}, (elem_t*)q_out, q_out_stride, tokens,
                     num_q_heads, num_kv_heads, head_dim, q_weight, k_weight, w_is_f32, eps, table, rot_dim, positions,
                     slots, k_cache, v_cache, page_size, stream);
}

NVA_DEFINE_LAST_ERROR(nva_rope)
