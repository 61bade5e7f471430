// Decode attention on the matrix cores (bfloat16): one query token per request against the
// request's keys in the paged cache, split over the context.
//
// Semantics as in attn_generic.hip (nanovllm/layers/attention.py:71-74, causal).  The token at
// position p reads keys first..p, first = max(0, p - window + 1) with a window, else 0.
//
// Work split: the keys that the step's tokens see are cut into equal quotas, one per wave and kv
// head (see the plan below).  The G = Hq / Hkv query heads of a kv head share its keys: they are
// the 16 columns of a 16x16x32 MFMA (columns >= G idle).  A wave walks its keys in chunks of 32:
//   S^T[32 keys x 16 heads] = K[32 x D] Q^T          2 tiles x D/32 MFMAs, K rows straight from global
//   online softmax over keys (in-lane, then across the 4 lane groups)
//   O^T[D x 16 heads] += V^T[D x 32 keys] P^T        D/16 MFMAs; P stays in registers
// The transposed V cache (tiles [D, 32 keys], common.h) makes 8 consecutive keys of one channel one
// 16-byte load and a chunk's values one contiguous block; the rows of the two S tiles are interleaved (tile a: keys 8g..8g+3, tile b: 8g+4..8g+7 for
// lane group g) so that a lane's eight probabilities are exactly the eight keys of that load.
// A token whose keys lie in several quotas gets an unnormalised partial result (max, sum, O) from
// each; a second kernel merges them.  A token inside one quota is written by the first kernel itself.
//
// Requires head_dim % 32 == 0 (32..256), G <= 16, page_size % 8 == 0.  The launcher refuses anything
// else with an error; the host wrapper knows these limits and runs the general kernel instead.
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
    // block table entries come from the wave's register window (lane i holds page window_page0 + i);
    // a chunk begins at a multiple of its 32 keys, so where pages hold whole chunks it lies in one
    // page, which one instruction reads from the window (a shuffle per key goes through LDS)
    int page_a, page_b, page_v;
    if (page_size % DEC_CHUNK == 0) {
        page_a = page_b = page_v = __builtin_amdgcn_readlane(
            table_window, __builtin_amdgcn_readfirstlane(base / page_size - window_page0) & (NVA_WAVE - 1));
    } else {
        page_a = __shfl(table_window, (key_a / page_size - window_page0) & (NVA_WAVE - 1), NVA_WAVE);
        page_b = __shfl(table_window, (key_b / page_size - window_page0) & (NVA_WAVE - 1), NVA_WAVE);
        page_v = __shfl(table_window, (key0 / page_size - window_page0) & (NVA_WAVE - 1), NVA_WAVE);
    }
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

#define DEC_MAX_TOKENS 1024        // tokens of one launch: one wave plans them, 16 to a lane

// The plan of a step's decode attention, made on the device from the tokens' positions by one small
// kernel per step and cache group (so a captured step follows the lengths of the step it is replayed
// for), and read by the attention kernels of all the group's layers.
//
// Every wave gets the same amount of work, whatever the lengths of the requests: the chunks (32
// keys) that the tokens see are counted through, token after token, and cut into quotas of equal
// size, one quota for each of the W waves that work on a kv head (W = waves of the launch / kv
// heads, as many as the GPU holds at once); at least two chunks a quota (four for a few long
// requests, see nva_attn_decode_plan_size), and at most what 62 pages
// hold (a wave keeps the block table entries of what it reads in one register per lane), in which
// case a wave takes several quotas in turn.  A quota is one or more segments: (token, keys lo..hi).
// A token cut by a quota's edge has several segments, which a second kernel merges; a token with
// one segment is written by the attention kernel itself.  Segments <= tokens + quotas.
//
// plan (int32): [0] number of quotas, [1] number of segments, [2 .. 2 + tokens] where each token's
// segments begin; from decode_plan_quotas_at on, the first segment of every quota (and the number
// of segments after the last); from decode_plan_segments_at on, eight ints per segment: token,
// its request's block table row, its position, 1 if it is the token's only segment; lo, hi, -, -.
__host__ __device__ inline int64_t decode_plan_quotas_at(int64_t tokens) { return (2 + tokens + 1 + 3) / 4 * 4; }
__host__ __device__ inline int64_t decode_plan_segments_at(int64_t tokens, int64_t max_segments) {
    return (decode_plan_quotas_at(tokens) + (max_segments - tokens) + 2 + 3) / 4 * 4;     // quotas <= segments - tokens
}
__host__ __device__ inline int decode_quota_cap(int page_size) {
    const int cap = (62 * page_size) / DEC_CHUNK;
    return cap > 1 ? cap : 1;
}

__global__ void __launch_bounds__(NVA_WAVE)
attn_decode_plan_kernel(const int32_t* __restrict__ positions, const int32_t* __restrict__ token_seq, int tokens,
                        int page_size, int window, int max_segments, int waves_per_head, int32_t* __restrict__ plan,
                        int32_t* error_flag) {
    const int lane = threadIdx.x;
    // every lane's tokens: position (-1: no such token) and the chunks it sees
    int pos_r[DEC_MAX_TOKENS / NVA_WAVE];
    int total = 0;
#pragma unroll
    for (int i = 0; i < DEC_MAX_TOKENS / NVA_WAVE; ++i) {
        const int t = i * NVA_WAVE + lane;
        pos_r[i] = t < tokens ? positions[t] : -1;
    }
#pragma unroll
    for (int i = 0; i < DEC_MAX_TOKENS / NVA_WAVE; ++i)
        if (pos_r[i] >= 0) {
            const int first = window > 0 && pos_r[i] - window + 1 > 0 ? pos_r[i] - window + 1 : 0;
            total += pos_r[i] / DEC_CHUNK - first / DEC_CHUNK + 1;
        }
#pragma unroll
    for (int off = NVA_WAVE / 2; off > 0; off >>= 1) total += __shfl_xor(total, off, NVA_WAVE);
    int quota = (total + waves_per_head - 1) / waves_per_head;
    if (quota < 2) quota = 2;
    if (quota > decode_quota_cap(page_size)) quota = decode_quota_cap(page_size);
    int num_quotas = (total + quota - 1) / quota;
    const int max_quotas = max_segments - tokens;
    if (num_quotas > max_quotas) {                       // cannot be, by the launcher's bound
        if (error_flag && lane == 0) atomicOr(error_flag, 4);
        num_quotas = 0;
    }
    int32_t* begin = plan + 2;
    int32_t* quota_first = plan + decode_plan_quotas_at(tokens);
    int4* segments = reinterpret_cast<int4*>(plan + decode_plan_segments_at(tokens, max_segments));
    int chunks_before = 0, segments_before = 0;
#pragma unroll
    for (int i = 0; i < DEC_MAX_TOKENS / NVA_WAVE; ++i) {
        if (i * NVA_WAVE >= tokens) break;
        const int t = i * NVA_WAVE + lane;
        const int pos = pos_r[i];
        const int first = window > 0 && pos - window + 1 > 0 ? pos - window + 1 : 0;
        const int c = pos >= 0 && num_quotas > 0 ? pos / DEC_CHUNK - first / DEC_CHUNK + 1 : 0;
        int incl = c;
#pragma unroll
        for (int off = 1; off < NVA_WAVE; off <<= 1) {
            const int up = __shfl_up(incl, off, NVA_WAVE);
            if (lane >= off) incl += up;
        }
        const int cum = chunks_before + incl - c;                   // the token's first chunk, counted through
        chunks_before += __shfl(incl, NVA_WAVE - 1, NVA_WAVE);
        const int n = c > 0 ? (cum + c - 1) / quota - cum / quota + 1 : 0;
        incl = n;
#pragma unroll
        for (int off = 1; off < NVA_WAVE; off <<= 1) {
            const int up = __shfl_up(incl, off, NVA_WAVE);
            if (lane >= off) incl += up;
        }
        const int mine = segments_before + incl - n;
        segments_before += __shfl(incl, NVA_WAVE - 1, NVA_WAVE);
        if (t < tokens) {
            begin[t] = mine;
            const int seq = token_seq[t];
            for (int k = 0; k < n; ++k) {
                const int qi = cum / quota + k;
                const int c_lo = max(cum, qi * quota), c_hi = min(cum + c, (qi + 1) * quota);
                const int lo = (first / DEC_CHUNK + c_lo - cum) * DEC_CHUNK;
                const int hi = min((first / DEC_CHUNK + c_hi - cum) * DEC_CHUNK, pos + 1);
                if (mine + k < max_segments) {
                    segments[2 * (mine + k)] = make_int4(t, seq, pos, n == 1);
                    segments[2 * (mine + k) + 1] = make_int4(lo, hi, 0, 0);
                    if (c_lo == qi * quota) quota_first[qi] = mine + k;
                }
            }
        }
    }
    if (lane == 0) {
        plan[0] = num_quotas;
        plan[1] = segments_before;
        begin[tokens] = segments_before;
        quota_first[num_quotas] = segments_before;
    }
}

template <int D>
__global__ void __launch_bounds__(NVA_WAVE) __attribute__((amdgpu_waves_per_eu(D <= 128 ? 2 : 1, 2)))
attn_decode_kernel(const __bf16* __restrict__ q, int64_t q_stride, __bf16* __restrict__ out, int64_t out_stride,
                   float* __restrict__ part_o, float* __restrict__ part_ml, const int32_t* __restrict__ plan,
                   const __bf16* __restrict__ k_cache, const __bf16* __restrict__ v_cache,
                   const int32_t* __restrict__ block_tables, int table_stride, int tokens, int max_segments,
                   int num_q_heads, int num_kv_heads, int page_size, float scale, int window,
                   int32_t* error_flag) {
    constexpr int KP = D / 32;          // 16-byte pieces of a key row per lane = MFMAs per S tile
    constexpr int DT = D / 16;          // 16-channel tiles of the output
    const int lane = threadIdx.x, col = lane & 15, g = lane >> 4;
    const int G = num_q_heads / num_kv_heads;
    // Neighbouring waves take neighbouring quotas of one kv head: the kv heads of a page lie a power
    // of two apart in the cache, and waves that stream them side by side meet in the same memory
    // channels.
    const int waves_per_head = gridDim.x / num_kv_heads;
    const int kvh = blockIdx.x / waves_per_head;
    int quota = blockIdx.x % waves_per_head;
    const int32_t* quota_first = plan + decode_plan_quotas_at(tokens);
    const int4* segments = reinterpret_cast<const int4*>(plan + decode_plan_segments_at(tokens, max_segments));
    int seg = quota_first[quota], seg_end = quota_first[quota + 1];      // read before it is known that the quota exists
    const int num_quotas = plan[0];
    if (quota >= num_quotas) return;
    // row r of S tile a is key 8*(r/4) + r%4 of the chunk, of tile b the same + 4
    const int row_key = 8 * (col >> 2) + (col & 3);

    // A segment's block table entries: lane i keeps the entry of page lo / page_size + i (a segment
    // spans at most 62 pages, so no chunk needs the table again).
    auto first_of = [&](const int4& r) { return window > 0 && r.z - window + 1 > 0 ? r.z - window + 1 : 0; };
    auto window_of = [&](const int4& r, int lo) {
        const int page0 = lo / page_size;
        return page0 + lane <= r.z / page_size ? block_tables[(int64_t)r.y * table_stride + page0 + lane] : -1;
    };
    auto load_q = [&](const int4& r, bf16x8* qf) {
        // column `col` is query head kvh*G + col; lane group g holds channels [g*D/4, (g+1)*D/4)
        const __bf16* qrow = q + (int64_t)r.x * q_stride + (int64_t)(kvh * G + (col < G ? col : 0)) * D + g * (D / 4);
#pragma unroll
        for (int c = 0; c < KP; ++c) qf[c] = *reinterpret_cast<const bf16x8*>(qrow + 8 * c);
    };

    for (;;) {                                                           // over the wave's quotas: as a rule, one
    // A quota's segments follow each other without a gap in the wave's loads: while it works on a
    // segment, the record, the table entries and the query of the next are on their way, and the
    // load that follows a segment's last chunk is the next segment's first chunk.  (After the
    // quota's last segment the same segment is read once more and dropped.)
    int4 rec = segments[2 * seg];
    int lo = segments[2 * seg + 1].x, hi = segments[2 * seg + 1].y;
    int table_window = window_of(rec, lo);
    bf16x8 qf[KP];
    load_q(rec, qf);
    bf16x8 ka_n[KP], kb_n[KP], vf_n[DT];
    load_chunk<D>(lo, ka_n, kb_n, vf_n, k_cache, v_cache, table_window, lo / page_size, first_of(rec), rec.z + 1,
                  num_kv_heads, kvh, page_size, row_key, col, g, error_flag);
    int seg_next = min(seg + 1, seg_end - 1);
    int4 rec_next = segments[2 * seg_next];
    int2 range_next = *reinterpret_cast<const int2*>(&segments[2 * seg_next + 1]);

    for (;;) {                                                           // over the quota's segments
    const int64_t t = rec.x;
    const int first = first_of(rec);
    const int kv_len = rec.z + 1;
    const int window_page0 = lo / page_size;
    // the next segment: its table entries and its query (asked for now, used after this segment)
    // (after the quota's last segment there is none: the loads past its end then all meet the
    // segment's last key, which is visible and whose page the wave's table entries hold)
    const bool more = seg + 1 < seg_end;
    const int lo_next = range_next.x, hi_next = range_next.y;
    const int first_next = more ? first_of(rec_next) : hi_next - 1;
    const int kv_len_next = more ? rec_next.z + 1 : hi_next;
    int table_window_next = table_window;
    bf16x8 qf_next[KP];
    int4 rec_after = rec_next;
    int2 range_after = range_next;
    const int seg_after = min(seg_next + 1, seg_end - 1);
    if (more) {
        table_window_next = window_of(rec_next, lo_next);
        load_q(rec_next, qf_next);
        rec_after = segments[2 * seg_after];
        range_after = *reinterpret_cast<const int2*>(&segments[2 * seg_after + 1]);
    }
    if (col >= G) {
#pragma unroll
        for (int c = 0; c < KP; ++c)
#pragma unroll
            for (int e = 0; e < 8; ++e) qf[c][e] = (__bf16)0.f;
    }

    f32x4 acc[DT];
#pragma unroll
    for (int i = 0; i < DT; ++i) acc[i] = (f32x4){0.f, 0.f, 0.f, 0.f};
    float m_run = -INFINITY, l_run = 0.f;      // the maximum in units of raw scores
    const float c_exp = scale * 1.4426950408889634f;      // scale * log2(e)
    // The loads of the chunk after are issued, unconditionally and on one path, before the products
    // of the current chunk, so that a wave always has a chunk (16 KiB at head_dim 128) in flight and
    // the wait before the products covers exactly the current chunk's loads.
    for (int base = lo; base < hi; base += DEC_CHUNK) {
        bf16x8 ka[KP], kb[KP], vf[DT];
#pragma unroll
        for (int c = 0; c < KP; ++c) {
            ka[c] = ka_n[c];
            kb[c] = kb_n[c];
        }
#pragma unroll
        for (int dt = 0; dt < DT; ++dt) vf[dt] = vf_n[dt];
        {
            const bool last = base + DEC_CHUNK >= hi;                 // then the chunk after is the next segment's first
            load_chunk<D>(last ? lo_next : base + DEC_CHUNK, ka_n, kb_n, vf_n, k_cache, v_cache,
                          last ? table_window_next : table_window, last ? lo_next / page_size : window_page0,
                          last ? first_next : first, last ? kv_len_next : kv_len, num_kv_heads, kvh,
                          page_size, row_key, col, g, error_flag);
        }
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
        // this lane: head `col`, keys base + 8g + i (tile a) and base + 8g + 4 + i (tile b).  The
        // maximum is taken of the raw scores (scale > 0) and the scale folded, with log2(e), into the
        // exponent: p = 2^((s - m) * scale * log2 e), one fused multiply-add per score; the four lanes
        // of a head exchange their maxima and sums without LDS.
        float s[8];
        float m_new = m_run;
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            const int key = base + 8 * g + i;
            s[i] = (key >= first && key < kv_len) ? (i < 4 ? sa[i] : sb[i - 4]) : -INFINITY;
            m_new = fmaxf(m_new, s[i]);
        }
        m_new = nva_max_over_rows(m_new);
        // a head that has seen no key yet keeps -inf as its maximum; exponents then use a finite
        // stand-in so that -inf - (-inf) never arises
        const float m_use = fmaxf(m_new, -1e30f);
        const float neg_mc = -m_use * c_exp;
        float psum = 0.f;
        bf16x8 pf;
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            const __bf16 pb16 = (__bf16)__builtin_amdgcn_exp2f(fmaf(s[i], c_exp, neg_mc));
            pf[i] = pb16;
            psum += (float)pb16;           // the sum of what the product below really uses
        }
        psum = nva_sum_over_rows(psum);
        const float alpha = __builtin_amdgcn_exp2f((fmaxf(m_run, -1e30f) - m_use) * c_exp);
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
        if (rec.w == 1) {
            const float inv = l_run > 0.f ? 1.f / l_run : 0.f;
            __bf16* orow = out + t * out_stride + (int64_t)head * D;
#pragma unroll
            for (int dt = 0; dt < DT; ++dt)
#pragma unroll
                for (int i = 0; i < 4; ++i) orow[16 * dt + 4 * g + i] = (__bf16)(acc[dt][i] * inv);
        } else {
            const int64_t slot = (int64_t)seg * num_q_heads + head;
            float* po = part_o + slot * D;
#pragma unroll
            for (int dt = 0; dt < DT; ++dt)
                *reinterpret_cast<f32x4*>(po + 16 * dt + 4 * g) = acc[dt];
            if (g == 0) {
                part_ml[slot * 2] = m_run * scale;             // as the merge takes it: of the scaled scores
                part_ml[slot * 2 + 1] = l_run;
            }
        }
    }
    if (!more) break;
    seg = seg_next;
    seg_next = seg_after;
    rec = rec_next;
    rec_next = rec_after;
    range_next = range_after;
    table_window = table_window_next;
    lo = lo_next;
    hi = hi_next;
#pragma unroll
    for (int c = 0; c < KP; ++c) qf[c] = qf_next[c];
    }
    quota += waves_per_head;
    if (quota >= num_quotas) break;
    seg = quota_first[quota];
    seg_end = quota_first[quota + 1];
    }
}

// Merges the segments of one (token, head): o = sum_s o_s e^(m_s - m) / sum_s l_s e^(m_s - m); a
// token with one segment was written by the attention kernel itself.  One workgroup of four waves per
// (token, head).  Every wave finds the maximum m over the segments, then takes every fourth group of
// four segments (their loads overlap) and the four partial sums meet in LDS; the order of the sum
// depends on the number of segments only.
#define MERGE_WAVES 4
__global__ void __launch_bounds__(MERGE_WAVES * NVA_WAVE)
attn_decode_merge_kernel(const float* __restrict__ part_o, const float* __restrict__ part_ml,
                         const int32_t* __restrict__ plan, __bf16* __restrict__ out, int64_t out_stride,
                         int num_q_heads, int head_dim) {
    __shared__ float acc_s[MERGE_WAVES][4 * NVA_WAVE];
    __shared__ float l_s[MERGE_WAVES];
    const int64_t t = blockIdx.x;
    const int head = blockIdx.y, lane = threadIdx.x % NVA_WAVE, wave = threadIdx.x / NVA_WAVE;
    const int s_lo = plan[2 + t], s_hi = plan[2 + t + 1] - 1;             // the token's segments, counted through
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
            const int s = min(s0 + j, s_hi);                              // a segment past the end: read again, weight 0
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

// The same merge with one wave per (token, head) and four pairs per workgroup: for steps of many
// tokens, where there are pairs enough to fill the GPU and a token has few segments.
__global__ void __launch_bounds__(MERGE_WAVES * NVA_WAVE)
attn_decode_merge_wave_kernel(const float* __restrict__ part_o, const float* __restrict__ part_ml,
                              const int32_t* __restrict__ plan, __bf16* __restrict__ out, int64_t out_stride,
                              int tokens, int num_q_heads, int head_dim) {
    const int lane = threadIdx.x % NVA_WAVE;
    const int64_t pair = (int64_t)blockIdx.x * MERGE_WAVES + threadIdx.x / NVA_WAVE;
    if (pair >= (int64_t)tokens * num_q_heads) return;
    const int64_t t = pair / num_q_heads;
    const int head = (int)(pair % num_q_heads);
    const int s_lo = plan[2 + t], s_hi = plan[2 + t + 1] - 1;
    if (s_hi <= s_lo) return;
    auto slot_of = [&](int s) { return (int64_t)s * num_q_heads + head; };
    float m = -INFINITY;
    for (int s = s_lo + lane; s <= s_hi; s += NVA_WAVE) m = fmaxf(m, part_ml[slot_of(s) * 2]);
    m = wave_max(m);
    float l = 0.f;
    float acc[4] = {0.f, 0.f, 0.f, 0.f};
    for (int s0 = s_lo; s0 <= s_hi; s0 += 4) {
        float wj[4], v[4][4];
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int s = min(s0 + j, s_hi);                              // a segment past the end: read again, weight 0
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
    const float inv = l > 0.f ? 1.f / l : 0.f;
    __bf16* orow = out + t * out_stride + (int64_t)head * head_dim;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const int d = lane + i * NVA_WAVE;
        if (d < head_dim) orow[d] = (__bf16)(acc[i] * inv);
    }
}

// Waves of the attention kernel for this head size that the current GPU holds at once: the CUs of
// the device times the workgroups (of one wave) of that instance a CU takes, both asked of the
// runtime once.  0 after leaving a message.
static int decode_cus = 0;                 // the CUs of the device, known once decode_resident_waves has run
static int decode_resident_waves(int head_dim) {
    static int resident[9];                 // by head_dim / 32
    if (head_dim % 32 || head_dim < 32 || head_dim > 256) {
        nva_fail("attn_decode: head_dim %d has no instance", head_dim);
        return 0;
    }
    int& r = resident[head_dim / 32];
    if (!r) {
        int dev = 0, cus = 0, per_cu = 0;
        if (hipGetDevice(&dev) != hipSuccess ||
            hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || cus <= 0) {
            nva_fail("attn_decode: cannot read the number of CUs");
            return 0;
        }
        hipError_t e = hipSuccess;
        switch (head_dim) {
#define OCC(DD) case DD: e = hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, attn_decode_kernel<DD>, NVA_WAVE, 0); break
            OCC(32); OCC(64); OCC(96); OCC(128); OCC(160); OCC(192); OCC(224); OCC(256);
#undef OCC
        }
        if (e != hipSuccess || per_cu <= 0) {
            nva_fail("attn_decode: cannot read how many waves a CU holds (%s)", hipGetErrorString(e));
            return 0;
        }
        r = per_cu * cus;
        decode_cus = cus;
    }
    return r;
}

// What the decode attention of `tokens` single tokens needs when no request holds more than `longest`
// keys: the bound of the segments of all tokens together, the number of persistent waves (a multiple
// of the kv heads), and the size of the plan (int32).  Partial results: max_segments * num_q_heads *
// (head_dim + 2) floats.
NVA_EXPORT int nva_attn_decode_plan_size_bf16(int longest, int64_t tokens, int num_kv_heads, int head_dim, int page_size,
                                              int* max_segments, int* waves, int64_t* plan_ints) {
    if (longest <= 0 || tokens <= 0 || tokens > DEC_MAX_TOKENS || num_kv_heads <= 0 || page_size <= 0 ||
        !max_segments || !waves || !plan_ints)
        return nva_fail("attn_decode_plan_size: bad arguments (at most %d tokens a launch)", DEC_MAX_TOKENS);
    // a token sees at most longest / 32 + 2 chunks (a window may begin and end inside a chunk)
    const int64_t chunks = tokens * ((int64_t)longest / DEC_CHUNK + 2);
    const int resident = decode_resident_waves(head_dim);
    if (!resident) return -1;
    int64_t per_head = resident / num_kv_heads > 0 ? resident / num_kv_heads : 1;
    // A quota has at least two chunks; four where that still leaves some 32 waves for a kv head: a few
    // long requests are served better by fewer waves of four chunks than by more of two or three (one
    // request of 4096 keys in 12.0 instead of 12.6 µs, two in 15.1 instead of 16.8, four in 22.1
    // instead of 24.8), a short one is not (1024 keys: 8.7 µs with two chunks a wave, 10.6 with four).
    {
        const int64_t by4 = (chunks + 3) / 4, by2 = (chunks + 1) / 2;
        const int64_t most = by4 >= 32 ? by4 : (by2 < 32 ? by2 : 32);
        if (per_head > most) per_head = most;
    }
    // As many waves as a whole multiple of the CUs, so that every CU streams as much as every other
    // (a CU draws its share of the memory's bandwidth and no more): four requests of 4096 keys take
    // 20.6 µs with 128 waves a kv head on 256 CUs and 8 kv heads, 22.1 with 130; six take 26.2 µs with
    // 96 and 29.4 with 195.
    if (decode_cus > 0 && decode_cus % num_kv_heads == 0 && per_head > decode_cus / num_kv_heads)
        per_head -= per_head % (decode_cus / num_kv_heads);
    const int64_t cap = decode_quota_cap(page_size);
    const int64_t quotas = per_head > (chunks + cap - 1) / cap ? per_head : (chunks + cap - 1) / cap;
    const int64_t bound = tokens + quotas;
    if (bound * num_kv_heads > 0x7fffffff || per_head * num_kv_heads > 0x7fffffff)
        return nva_fail("attn_decode_plan_size: too many segments");
    *max_segments = (int)bound;
    *waves = (int)(per_head * num_kv_heads);
    *plan_ints = decode_plan_segments_at(tokens, bound) + 8 * bound;
    return 0;
}

// Makes the plan of a step (once per step and cache group; every layer's attention reads it).
// max_segments and waves from nva_attn_decode_plan_size for the same tokens, kv heads and page size.
NVA_EXPORT int nva_attn_decode_plan_bf16(const int32_t* positions, const int32_t* token_seq, int64_t tokens,
                                         int num_kv_heads, int page_size, int window, int max_segments, int waves,
                                         int32_t* plan, int32_t* error_flag, hipStream_t stream) {
    if (!positions || !token_seq || !plan || !nva_aligned(plan, 16) || tokens <= 0 || tokens > DEC_MAX_TOKENS ||
        num_kv_heads <= 0 || page_size <= 0 || window < 0 || max_segments <= tokens || waves <= 0 || waves % num_kv_heads)
        return nva_fail("attn_decode_plan: bad arguments");
    hipLaunchKernelGGL(attn_decode_plan_kernel, dim3(1), dim3(NVA_WAVE), 0, stream, positions, token_seq, (int)tokens,
                       page_size, window, max_segments, waves / num_kv_heads, plan, error_flag);
    return nva_check_launch("attn_decode_plan");
}

// Refuses (non-zero code and a message) shapes this kernel does not take: the host wrapper checks
// the same limits first and runs the general kernel for them.  plan: made by nva_attn_decode_plan for these tokens, kv heads, page size and
// window; max_segments and waves from nva_attn_decode_plan_size.
NVA_EXPORT int nva_attn_decode_bf16(const void* q, int64_t q_stride, void* out, int64_t out_stride, float* scratch,
                                    const int32_t* plan, const void* k_cache, const void* v_cache,
                                    const int32_t* block_tables, int table_stride, int64_t tokens, int num_q_heads,
                                    int num_kv_heads, int head_dim, int page_size, float scale, int window,
                                    int max_segments, int waves, int32_t* error_flag, hipStream_t stream) {
    if (tokens == 0) return 0;
    if (num_q_heads <= 0 || num_kv_heads <= 0 || num_q_heads % num_kv_heads)
        return nva_fail("attn_decode: %d query heads do not divide into %d kv heads", num_q_heads, num_kv_heads);
    const int G = num_q_heads / num_kv_heads;
    if (!(scale > 0.f) || !(scale <= 3.0e38f)) {
        // the running maximum is taken of the raw scores and the scale folded into the exponent
        nva_fail("attn_decode: needs a positive, finite scale (got %g)", (double)scale);
        return 1;
    }
    if (G > 16 || head_dim % 32 || head_dim < 32 || head_dim > 256 || page_size % 8 || page_size <= 0) {
        nva_fail("attn_decode: needs head_dim %% 32 == 0 in 32..256, at most 16 query heads per kv head and "
                 "page_size %% 8 == 0 (got head_dim %d, group %d, page %d)", head_dim, G, page_size);
        return 1;
    }
    if (tokens < 0 || tokens > DEC_MAX_TOKENS || num_q_heads > 65535)
        return nva_fail("attn_decode: %lld tokens (at most %d a launch) or %d heads exceed the grid", (long long)tokens,
                        DEC_MAX_TOKENS, num_q_heads);
    if (max_segments <= tokens || waves <= 0 || waves % num_kv_heads || window < 0 || table_stride <= 0 || !scratch ||
        !plan || !nva_aligned(plan, 16))
        return nva_fail("attn_decode: bad plan (%d segments, %d waves), window %d or no scratch", max_segments, waves,
                        window);
    float* part_o = scratch;
    float* part_ml = scratch + (int64_t)max_segments * num_q_heads * head_dim;
#define LAUNCH(DD)                                                                                              \
    hipLaunchKernelGGL(attn_decode_kernel<DD>, dim3((unsigned)waves), dim3(NVA_WAVE), 0, stream, (const __bf16*)q, \
                       q_stride, (__bf16*)out, out_stride, part_o, part_ml, plan, (const __bf16*)k_cache,         \
                       (const __bf16*)v_cache, block_tables, table_stride, (int)tokens, max_segments, num_q_heads,  \
                       num_kv_heads, page_size, scale, window, error_flag)
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
    const int64_t pairs = tokens * num_q_heads;
    const int resident = decode_resident_waves(head_dim);
    if (!resident) return -1;
    if (pairs >= 2 * resident) {            // pairs enough for a wave each
        hipLaunchKernelGGL(attn_decode_merge_wave_kernel, dim3((unsigned)((pairs + MERGE_WAVES - 1) / MERGE_WAVES)),
                           dim3(MERGE_WAVES * NVA_WAVE), 0, stream, part_o, part_ml, plan, (__bf16*)out, out_stride,
                           (int)tokens, num_q_heads, head_dim);
        return nva_check_launch("attn_decode_merge");
    }
    dim3 mgrid((unsigned)tokens, (unsigned)num_q_heads);
    hipLaunchKernelGGL(attn_decode_merge_kernel, mgrid, dim3(MERGE_WAVES * NVA_WAVE), 0, stream, part_o, part_ml, plan,
                       (__bf16*)out, out_stride, num_q_heads, head_dim);
    return nva_check_launch("attn_decode_merge");
}

NVA_DEFINE_LAST_ERROR(nva_attn_decode)
