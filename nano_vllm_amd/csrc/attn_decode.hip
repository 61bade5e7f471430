// Decode attention on the matrix cores (bfloat16): one query token per request against the
// request's keys in the paged cache, split over the context.
//
// Semantics as in attn_generic.hip (nanovllm/layers/attention.py:71-74, causal).  The token at
// position p reads keys first..p, first = max(0, p - window + 1) with a window, else 0.
//
// Work split: an item is (split of a token's context, kv head); persistent waves take the items in
// turn (see decode_plan below).  The G = Hq / Hkv query heads of a kv head share its keys: they are
// the 16 columns of a 16x16x32 MFMA (columns >= G idle).  A wave walks its split in chunks of 32 keys:
//   S^T[32 keys x 16 heads] = K[32 x D] Q^T          2 tiles x D/32 MFMAs, K rows straight from global
//   online softmax over keys (in-lane, then across the 4 lane groups)
//   O^T[D x 16 heads] += V^T[D x 32 keys] P^T        D/16 MFMAs; P stays in registers
// The transposed V cache (tiles [D, 32 keys], common.h) makes 8 consecutive keys of one channel one
// 16-byte load and a chunk's values one contiguous block; the rows of the two S tiles are interleaved (tile a: keys 8g..8g+3, tile b: 8g+4..8g+7 for
// lane group g) so that a lane's eight probabilities are exactly the eight keys of that load.
// Each split writes an unnormalised partial result (max, sum, O); a second kernel merges them.
// A token with a single split is written by the first kernel itself.
//
// Requires head_dim % 32 == 0 (32..256), G <= 16, page_size % 8 == 0; the launcher refuses
// anything else and the caller falls back to the general kernel.
#include "common.h"

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(4))) float f32x4;

#define DEC_CHUNK 32

// One chunk of 32 keys for one lane: its two K rows (keys base + row_key and + 4, the channels of
// lane group g) and, per 16-channel tile, eight consecutive keys of channel `col` of V.  Every load
// is unconditional: a key outside [first, kv_len) is replaced by the nearest visible one, so that
// no loaded value has to pass through a select (which would make each load wait for the one
// before).  What such lanes hold is masked where it is used: scores by the key index, and V in the
// chunks at the two ends of the visible range.
template <int D>
__device__ __forceinline__ void load_chunk(int base, bf16x8* ka, bf16x8* kb, bf16x8* vf,
                                           const __bf16* __restrict__ k_cache, const __bf16* __restrict__ v_cache,
                                           int table_window, int window_page0, int first, int kv_len, int num_kv_heads,
                                           int kvh, int page_size, int row_key, int col, int g, int32_t* error_flag) {
    constexpr int KP = D / 32, DT = D / 16;
    const int key_a = min(max(base + row_key, first), kv_len - 1);
    const int key_b = min(max(base + row_key + 4, first), kv_len - 1);
    // the group of 8 keys of V, moved to the nearest group that holds a visible key
    const int key0 = min(max(base + 8 * g, first & ~7), (kv_len - 1) & ~7);
    // block table entries come from the wave's register window (lane i holds page window_page0 + i)
    const int page_a = __shfl(table_window, (key_a / page_size - window_page0) & (NVA_WAVE - 1), NVA_WAVE);
    const int page_b = __shfl(table_window, (key_b / page_size - window_page0) & (NVA_WAVE - 1), NVA_WAVE);
    const int page_v = __shfl(table_window, (key0 / page_size - window_page0) & (NVA_WAVE - 1), NVA_WAVE);
    if (page_a < 0 || page_b < 0 || page_v < 0) {
        if (error_flag) atomicOr(error_flag, 2);
    }
    const __bf16* pa = k_cache + (((int64_t)max(page_a, 0) * num_kv_heads + kvh) * page_size + key_a % page_size) * D + g * (D / 4);
    const __bf16* pb = k_cache + (((int64_t)max(page_b, 0) * num_kv_heads + kvh) * page_size + key_b % page_size) * D + g * (D / 4);
#pragma unroll
    for (int c = 0; c < KP; ++c) {
        ka[c] = *reinterpret_cast<const bf16x8*>(pa + 8 * c);
        kb[c] = *reinterpret_cast<const bf16x8*>(pb + 8 * c);
    }
    // V: channel 16*dt + col, keys key0 .. key0 + 7 (one page: page_size % 8 == 0)
    const int vt = nva_v_tile(page_size);           // a multiple of 8: the group lies in one tile
    const __bf16* pv = v_cache + ((int64_t)max(page_v, 0) * num_kv_heads + kvh) * D * (int64_t)page_size +
                       nva_v_offset(key0 % page_size, col, D, vt);
#pragma unroll
    for (int dt = 0; dt < DT; ++dt) vf[dt] = *reinterpret_cast<const bf16x8*>(pv + (int64_t)dt * 16 * vt);
}

// waves the GPU holds at once: the kernel's registers allow two per SIMD, eight per CU, on 256 CUs
#define DEC_RESIDENT_WAVES 2048
#define DEC_MAX_TOKENS 1024        // tokens of one launch: their split counts are summed in LDS by every wave

// The plan of a step's decode attention, made on the device from the tokens' positions by one small
// kernel per step and cache group (so a captured step follows the lengths of the step it is replayed
// for), and read by the attention kernels of all the group's layers:
//   keys per split  = mean visible length / wanted, a multiple of 32, at least 64 (32 with tiny
//                     pages: a wave keeps its split's block table entries in one register per lane,
//                     at most 62 pages); wanted = ceil(waves / (tokens * kv_heads)) with `waves` the
//                     waves the GPU holds at once, four times that where the longest request is
//                     more than 1.25 times the mean (finer items then level the load);
//   a token's splits are cut at multiples of that length of the absolute position;
//   the splits of all tokens, counted through, times the kv heads are the launch's items; wave w
//   of the W persistent waves (as many as the GPU holds at once) takes items w, w + W, ...
// Sum over tokens of splits <= tokens * (wanted + 2) (or the page limit's count): the size of the
// partial results, which the launcher checks through nva_attn_decode_plan.
// plan: [0] keys per split, [1] total splits, [2 .. 2 + tokens] where each token's splits begin,
// then per split (token << 16) | index of the split within the token's absolute positions.
__global__ void __launch_bounds__(NVA_WAVE)
attn_decode_plan_kernel(const int32_t* __restrict__ positions, int tokens, int kv_heads, int page_size, int window,
                        int max_total_splits, int32_t* __restrict__ plan, int32_t* error_flag) {
    const int lane = threadIdx.x;
    // every lane's tokens' positions, loaded at once (-1: no such token)
    int pos_r[DEC_MAX_TOKENS / NVA_WAVE];
#pragma unroll
    for (int i = 0; i < DEC_MAX_TOKENS / NVA_WAVE; ++i) {
        const int t = i * NVA_WAVE + lane;
        pos_r[i] = t < tokens ? positions[t] : -1;
    }
    int64_t sum = 0;
    int longest = 0;
#pragma unroll
    for (int i = 0; i < DEC_MAX_TOKENS / NVA_WAVE; ++i)
        if (pos_r[i] >= 0) {
            const int visible = window > 0 && pos_r[i] + 1 > window ? window : pos_r[i] + 1;
            sum += visible;
            longest = max(longest, visible);
        }
#pragma unroll
    for (int off = NVA_WAVE / 2; off > 0; off >>= 1) {
        sum += __shfl_xor(sum, off, NVA_WAVE);
        longest = max(longest, __shfl_xor(longest, off, NVA_WAVE));
    }
    const int mean = (int)((sum + tokens - 1) / tokens);
    const int64_t rows = (int64_t)tokens * kv_heads;
    const int64_t target = (int64_t)longest * 4 > (int64_t)mean * 5 ? 4 * DEC_RESIDENT_WAVES : DEC_RESIDENT_WAVES;
    const int wanted = (int)((target + rows - 1) / rows);
    int len = ((mean + wanted - 1) / wanted + DEC_CHUNK - 1) / DEC_CHUNK * DEC_CHUNK;
    if (len < 2 * DEC_CHUNK) len = 2 * DEC_CHUNK;
    const int cap = (62 * page_size) / DEC_CHUNK * DEC_CHUNK;
    if (len > cap) len = cap;
    if (len < DEC_CHUNK) len = DEC_CHUNK;
    int32_t* begin = plan + 2;
    int32_t* items = plan + 2 + tokens + 1;
    int carry = 0;
#pragma unroll
    for (int i = 0; i < DEC_MAX_TOKENS / NVA_WAVE; ++i) {
        if (i * NVA_WAVE >= tokens) break;
        const int t = i * NVA_WAVE + lane;
        int c = 0, s0 = 0;
        if (pos_r[i] >= 0) {
            const int pos = pos_r[i];
            const int first = window > 0 && pos - window + 1 > 0 ? pos - window + 1 : 0;
            s0 = first / len;
            c = pos / len - s0 + 1;
        }
        int incl = c;
#pragma unroll
        for (int off = 1; off < NVA_WAVE; off <<= 1) {
            const int up = __shfl_up(incl, off, NVA_WAVE);
            if (lane >= off) incl += up;
        }
        const int mine = carry + incl - c;
        if (t < tokens) {
            begin[t] = min(mine, max_total_splits);
            for (int k = 0; k < c; ++k)
                if (mine + k < max_total_splits) items[mine + k] = (t << 16) | (s0 + k);
        }
        carry += __shfl(incl, NVA_WAVE - 1, NVA_WAVE);
    }
    if (lane == 0) {
        if (carry > max_total_splits && error_flag) atomicOr(error_flag, 4);   // cannot be, by the launcher's bound
        plan[0] = len;
        plan[1] = min(carry, max_total_splits);
        begin[tokens] = min(carry, max_total_splits);
    }
}

template <int D>
__global__ void __launch_bounds__(NVA_WAVE)
attn_decode_kernel(const __bf16* __restrict__ q, int64_t q_stride, __bf16* __restrict__ out, int64_t out_stride,
                   float* __restrict__ part_o, float* __restrict__ part_ml, const int32_t* __restrict__ plan,
                   const __bf16* __restrict__ k_cache, const __bf16* __restrict__ v_cache,
                   const int32_t* __restrict__ block_tables, int table_stride,
                   const int32_t* __restrict__ token_seq, const int32_t* __restrict__ positions, int tokens,
                   int num_q_heads, int num_kv_heads, int page_size, float scale, int window,
                   int32_t* error_flag) {
    constexpr int KP = D / 32;          // 16-byte pieces of a key row per lane = MFMAs per S tile
    constexpr int DT = D / 16;          // 16-channel tiles of the output
    const int lane = threadIdx.x, col = lane & 15, g = lane >> 4;
    const int G = num_q_heads / num_kv_heads;
    const int split_len = plan[0], total_splits = plan[1];
    const int32_t* begin = plan + 2;
    const int32_t* items = plan + 2 + tokens + 1;
    // row r of S tile a is key 8*(r/4) + r%4 of the chunk, of tile b the same + 4
    const int row_key = 8 * (col >> 2) + (col & 3);

    for (int item = blockIdx.x; item < total_splits * num_kv_heads; item += gridDim.x) {
    // neighbouring waves take neighbouring splits of one kv head: the kv heads of a page lie a power of
    // two apart in the cache, and waves that stream them side by side meet in the same memory channels
    const int flat = item % total_splits, kvh = item / total_splits;
    const int packed = items[flat];
    const int64_t t = packed >> 16;
    const int split = packed & 0xffff;
    const int splits_of_t = begin[t + 1] - begin[t];
    const int pos = positions[t];
    const int first = window > 0 && pos - window + 1 > 0 ? pos - window + 1 : 0;
    const int kv_len = pos + 1;
    // the splits are cut at multiples of split_len of the absolute position
    const int lo = max(split * split_len, first & ~(DEC_CHUNK - 1));
    const int hi = min((split + 1) * split_len, kv_len);
    const int32_t* table = block_tables + (int64_t)token_seq[t] * table_stride;

    // Q: column `col` is query head kvh*G + col; lane group g holds channels [g*D/4, (g+1)*D/4)
    bf16x8 qf[KP];
    {
        const __bf16* qrow = q + t * q_stride + (int64_t)(kvh * G + (col < G ? col : 0)) * D + g * (D / 4);
#pragma unroll
        for (int c = 0; c < KP; ++c) {
            bf16x8 v = *reinterpret_cast<const bf16x8*>(qrow + 8 * c);
            if (col >= G) {
#pragma unroll
                for (int e = 0; e < 8; ++e) v[e] = (__bf16)0.f;
            }
            qf[c] = v;
        }
    }

    f32x4 acc[DT];
#pragma unroll
    for (int i = 0; i < DT; ++i) acc[i] = (f32x4){0.f, 0.f, 0.f, 0.f};
    float m_run = -INFINITY, l_run = 0.f;
    // The loads of chunk i + 1 are issued before the products of chunk i, so that a wave always has
    // a chunk (16 KiB at head_dim 128) in flight.
    // Lane i of the wave keeps block table entry window_page0 + i: a split spans at most 64 pages
    // (the launcher checks it), so no chunk needs the table again.
    const int last_page = (kv_len - 1) / page_size;
    const int window_page0 = lo / page_size;
    const int table_window = window_page0 + lane <= last_page ? table[window_page0 + lane] : -1;
    // The loads of the next chunk are issued, unconditionally, before the products of the current
    // one (after the last chunk the same chunk is read once more and dropped): one path through the
    // loop, so that the wait before the products covers exactly the current chunk's loads.
    const int last_base = lo + ((hi - lo - 1) / DEC_CHUNK) * DEC_CHUNK;
    bf16x8 ka_n[KP], kb_n[KP], vf_n[DT];
    load_chunk<D>(lo, ka_n, kb_n, vf_n, k_cache, v_cache, table_window, window_page0, first, kv_len, num_kv_heads, kvh,
                  page_size, row_key, col, g, error_flag);
    for (int base = lo; base < hi; base += DEC_CHUNK) {
        bf16x8 ka[KP], kb[KP], vf[DT];
#pragma unroll
        for (int c = 0; c < KP; ++c) {
            ka[c] = ka_n[c];
            kb[c] = kb_n[c];
        }
#pragma unroll
        for (int dt = 0; dt < DT; ++dt) vf[dt] = vf_n[dt];
        load_chunk<D>(min(base + DEC_CHUNK, last_base), ka_n, kb_n, vf_n, k_cache, v_cache, table_window, window_page0,
                      first, kv_len, num_kv_heads, kvh, page_size, row_key, col, g, error_flag);
        if (base < first || base + DEC_CHUNK > kv_len) {
            // a chunk at an end of the visible range: what V holds outside the range may be anything
            const int key0 = base + 8 * g;
#pragma unroll
            for (int dt = 0; dt < DT; ++dt)
#pragma unroll
                for (int e = 0; e < 8; ++e)
                    if (key0 + e >= kv_len || key0 + e < first) vf[dt][e] = (__bf16)0.f;
        }
        // ---- scores
        f32x4 sa = {0.f, 0.f, 0.f, 0.f}, sb = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int c = 0; c < KP; ++c) {
            sa = __builtin_amdgcn_mfma_f32_16x16x32_bf16(ka[c], qf[c], sa, 0, 0, 0);
            sb = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kb[c], qf[c], sb, 0, 0, 0);
        }
        // this lane: head `col`, keys base + 8g + i (tile a) and base + 8g + 4 + i (tile b)
        float s[8];
        float m_new = m_run;
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            const int key = base + 8 * g + i;
            const float v = (i < 4 ? sa[i] : sb[i - 4]) * scale;
            s[i] = (key >= first && key < kv_len) ? v : -INFINITY;
            m_new = fmaxf(m_new, s[i]);
        }
        m_new = fmaxf(m_new, __shfl_xor(m_new, 16, NVA_WAVE));
        m_new = fmaxf(m_new, __shfl_xor(m_new, 32, NVA_WAVE));
        float psum = 0.f;
        bf16x8 pf;
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            const float p = (s[i] == -INFINITY) ? 0.f : __expf(s[i] - m_new);
            const __bf16 pb16 = (__bf16)p;
            pf[i] = pb16;
            psum += (float)pb16;           // the sum of what the product below really uses
        }
        psum += __shfl_xor(psum, 16, NVA_WAVE);
        psum += __shfl_xor(psum, 32, NVA_WAVE);
        const float alpha = (m_run == -INFINITY) ? 0.f : __expf(m_run - m_new);
        l_run = l_run * alpha + psum;
        m_run = m_new;
        // ---- O^T += V^T P^T
#pragma unroll
        for (int dt = 0; dt < DT; ++dt) {
            f32x4 a = acc[dt];
            a[0] *= alpha; a[1] *= alpha; a[2] *= alpha; a[3] *= alpha;
            acc[dt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vf[dt], pf, a, 0, 0, 0);
        }
    }

    // acc[dt][i] = O[head col][channel 16*dt + 4*g + i]
    if (col < G) {
        const int head = kvh * G + col;
        if (splits_of_t == 1) {
            const float inv = l_run > 0.f ? 1.f / l_run : 0.f;
            __bf16* orow = out + t * out_stride + (int64_t)head * D;
#pragma unroll
            for (int dt = 0; dt < DT; ++dt)
#pragma unroll
                for (int i = 0; i < 4; ++i) orow[16 * dt + 4 * g + i] = (__bf16)(acc[dt][i] * inv);
        } else {
            const int64_t slot = (int64_t)flat * num_q_heads + head;
            float* po = part_o + slot * D;
#pragma unroll
            for (int dt = 0; dt < DT; ++dt)
                *reinterpret_cast<f32x4*>(po + 16 * dt + 4 * g) = acc[dt];
            if (g == 0) {
                part_ml[slot * 2] = m_run;
                part_ml[slot * 2 + 1] = l_run;
            }
        }
    }
    }
}

// Merges the splits of one (token, head): o = sum_s o_s e^(m_s - m) / sum_s l_s e^(m_s - m); a
// token with one split was written by the attention kernel itself.  One workgroup of four waves per
// (token, head).  Every wave finds the maximum m over the splits, then takes every fourth group of
// four splits (their loads overlap) and the four partial sums meet in LDS; the order of the sum
// depends on the number of splits only.
#define MERGE_WAVES 4
__global__ void __launch_bounds__(MERGE_WAVES * NVA_WAVE)
attn_decode_merge_kernel(const float* __restrict__ part_o, const float* __restrict__ part_ml,
                         const int32_t* __restrict__ plan, __bf16* __restrict__ out, int64_t out_stride,
                         int num_q_heads, int head_dim) {
    __shared__ float acc_s[MERGE_WAVES][4 * NVA_WAVE];
    __shared__ float l_s[MERGE_WAVES];
    const int64_t t = blockIdx.x;
    const int head = blockIdx.y, lane = threadIdx.x % NVA_WAVE, wave = threadIdx.x / NVA_WAVE;
    const int s_lo = plan[2 + t], s_hi = plan[2 + t + 1] - 1;             // the token's splits, counted through
    if (s_hi <= s_lo) return;
    auto slot_of = [&](int s) { return (int64_t)s * num_q_heads + head; };
    float m = -INFINITY;
    for (int s = s_lo + lane; s <= s_hi; s += NVA_WAVE) m = fmaxf(m, part_ml[slot_of(s) * 2]);
    m = wave_max(m);
    float l = 0.f;
    float acc[4] = {0.f, 0.f, 0.f, 0.f};
    for (int s0 = s_lo + 4 * wave; s0 <= s_hi; s0 += 4 * MERGE_WAVES) {
        float wj[4], v[4][4];
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int s = min(s0 + j, s_hi);                              // a split past the end: read again, weight 0
            const float ms = part_ml[slot_of(s) * 2];
            wj[j] = (s0 + j > s_hi || ms == -INFINITY) ? 0.f : __expf(ms - m);
            l += part_ml[slot_of(s) * 2 + 1] * wj[j];
            const float* po = part_o + slot_of(s) * head_dim;
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const int d = lane + i * NVA_WAVE;
                v[j][i] = d < head_dim ? po[d] : 0.f;
            }
        }
#pragma unroll
        for (int j = 0; j < 4; ++j)
#pragma unroll
            for (int i = 0; i < 4; ++i) acc[i] += v[j][i] * wj[j];
    }
#pragma unroll
    for (int i = 0; i < 4; ++i) acc_s[wave][lane + i * NVA_WAVE] = acc[i];
    if (lane == 0) l_s[wave] = l;
    __syncthreads();
    if (wave != 0) return;
    l = 0.f;
#pragma unroll
    for (int w = 0; w < MERGE_WAVES; ++w) l += l_s[w];
    const float inv = l > 0.f ? 1.f / l : 0.f;
    __bf16* orow = out + t * out_stride + (int64_t)head * head_dim;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const int d = lane + i * NVA_WAVE;
        float o = 0.f;
#pragma unroll
        for (int w = 0; w < MERGE_WAVES; ++w) o += acc_s[w][d];
        if (d < head_dim) orow[d] = (__bf16)(o * inv);
    }
}

// What the decode attention of `tokens` single tokens needs when no request holds more than `longest`
// keys: the bound of the splits of all tokens together, the number of persistent waves, and the size
// of the plan (int32).  Partial results: max_total_splits * num_q_heads * (head_dim + 2) floats.
NVA_EXPORT int nva_attn_decode_plan_size_bf16(int longest, int64_t tokens, int num_kv_heads, int page_size,
                                              int* max_total_splits, int* waves, int64_t* plan_ints) {
    if (longest <= 0 || tokens <= 0 || tokens > DEC_MAX_TOKENS || num_kv_heads <= 0 || page_size <= 0 ||
        !max_total_splits || !waves || !plan_ints)
        return nva_fail("attn_decode_plan_size: bad arguments (at most %d tokens a launch)", DEC_MAX_TOKENS);
    const int64_t rows = tokens * num_kv_heads;
    const int64_t wanted = (4 * DEC_RESIDENT_WAVES + rows - 1) / rows;
    // sum of the tokens' counts <= total / len + 2 * tokens; len >= mean / wanted unless the page limit cuts it
    const int cap = (62 * page_size) / DEC_CHUNK * DEC_CHUNK > DEC_CHUNK ? (62 * page_size) / DEC_CHUNK * DEC_CHUNK : DEC_CHUNK;
    int64_t per_token = wanted;
    if ((longest + cap - 1) / cap > per_token) per_token = (longest + cap - 1) / cap;
    if (per_token > (longest + DEC_CHUNK - 1) / DEC_CHUNK) per_token = (longest + DEC_CHUNK - 1) / DEC_CHUNK;
    const int64_t bound = tokens * (per_token + 2);
    if (bound * num_kv_heads > 0x7fffffff || (longest + DEC_CHUNK - 1) / DEC_CHUNK > 0xffff)
        return nva_fail("attn_decode_plan_size: too many splits");
    *max_total_splits = (int)bound;
    const int64_t items = bound * num_kv_heads;
    *waves = (int)(items < DEC_RESIDENT_WAVES ? items : DEC_RESIDENT_WAVES);
    *plan_ints = 2 + tokens + 1 + bound;
    return 0;
}

// Makes the plan of a step (once per step and cache group; every layer's attention reads it).
NVA_EXPORT int nva_attn_decode_plan_bf16(const int32_t* positions, int64_t tokens, int num_kv_heads, int page_size,
                                         int window, int max_total_splits, int32_t* plan, int32_t* error_flag,
                                         hipStream_t stream) {
    if (!positions || !plan || tokens <= 0 || tokens > DEC_MAX_TOKENS || num_kv_heads <= 0 || page_size <= 0 ||
        window < 0 || max_total_splits <= 0)
        return nva_fail("attn_decode_plan: bad arguments");
    hipLaunchKernelGGL(attn_decode_plan_kernel, dim3(1), dim3(NVA_WAVE), 0, stream, positions, (int)tokens, num_kv_heads,
                       page_size, window, max_total_splits, plan, error_flag);
    return nva_check_launch("attn_decode_plan");
}

// Returns 1 (and leaves a message) for shapes this kernel does not take; the caller then uses the
// general kernel.  plan: made by nva_attn_decode_plan for these tokens, kv heads, page size and
// window; max_total_splits and waves from nva_attn_decode_plan_size.
NVA_EXPORT int nva_attn_decode_bf16(const void* q, int64_t q_stride, void* out, int64_t out_stride, float* scratch,
                                    const int32_t* plan, const void* k_cache, const void* v_cache,
                                    const int32_t* block_tables, int table_stride, const int32_t* token_seq,
                                    const int32_t* positions, int64_t tokens, int num_q_heads, int num_kv_heads,
                                    int head_dim, int page_size, float scale, int window, int max_total_splits,
                                    int waves, int32_t* error_flag, hipStream_t stream) {
    if (tokens == 0) return 0;
    if (num_q_heads <= 0 || num_kv_heads <= 0 || num_q_heads % num_kv_heads)
        return nva_fail("attn_decode: %d query heads do not divide into %d kv heads", num_q_heads, num_kv_heads);
    const int G = num_q_heads / num_kv_heads;
    if (G > 16 || head_dim % 32 || head_dim < 32 || head_dim > 256 || page_size % 8 || page_size <= 0) {
        nva_fail("attn_decode: needs head_dim %% 32 == 0 in 32..256, at most 16 query heads per kv head and "
                 "page_size %% 8 == 0 (got head_dim %d, group %d, page %d)", head_dim, G, page_size);
        return 1;
    }
    if (tokens < 0 || tokens > DEC_MAX_TOKENS || num_q_heads > 65535)
        return nva_fail("attn_decode: %lld tokens (at most %d a launch) or %d heads exceed the grid", (long long)tokens,
                        DEC_MAX_TOKENS, num_q_heads);
    if (max_total_splits <= 0 || waves <= 0 || window < 0 || table_stride <= 0 || !scratch || !plan)
        return nva_fail("attn_decode: bad plan (%d splits, %d waves), window %d or no scratch", max_total_splits, waves,
                        window);
    float* part_o = scratch;
    float* part_ml = scratch + (int64_t)max_total_splits * num_q_heads * head_dim;
#define LAUNCH(DD)                                                                                              \
    hipLaunchKernelGGL(attn_decode_kernel<DD>, dim3((unsigned)waves), dim3(NVA_WAVE), 0, stream, (const __bf16*)q, \
                       q_stride, (__bf16*)out, out_stride, part_o, part_ml, plan, (const __bf16*)k_cache,         \
                       (const __bf16*)v_cache, block_tables, table_stride, token_seq, positions, (int)tokens,     \
                       num_q_heads, num_kv_heads, page_size, scale, window, error_flag)
    switch (head_dim) {
        case 32: LAUNCH(32); break;
        case 64: LAUNCH(64); break;
        case 96: LAUNCH(96); break;
        case 128: LAUNCH(128); break;
        case 160: LAUNCH(160); break;
        case 192: LAUNCH(192); break;
        case 224: LAUNCH(224); break;
        case 256: LAUNCH(256); break;
        default: return nva_fail("attn_decode: head_dim %d has no instance", head_dim);
    }
#undef LAUNCH
    int rc = nva_check_launch("attn_decode");
    if (rc) return rc;
    dim3 mgrid((unsigned)tokens, (unsigned)num_q_heads);
    hipLaunchKernelGGL(attn_decode_merge_kernel, mgrid, dim3(MERGE_WAVES * NVA_WAVE), 0, stream, part_o, part_ml, plan,
                       (__bf16*)out, out_stride, num_q_heads, head_dim);
    return nva_check_launch("attn_decode_merge");
}

NVA_DEFINE_LAST_ERROR(nva_attn_decode)
