// Prefill attention on the matrix cores (bfloat16): portions of prompts against the paged cache.
//
// Semantics as in attn_generic.hip (nanovllm/layers/attention.py:64-70: causal, the diagonal
// aligned to the end of the keys when a request has cached tokens before this step's).  A request
// with q_len new tokens and kv_len tokens in the cache after this step has its query i at position
// kv_len - q_len + i; it reads keys first..position, first = max(0, position - window + 1) with a
// window, else 0.  The step's own keys are in the cache already.
//
// Work split: a workgroup of 4 waves takes 32 query rows of one request and up to 4 query heads of
// one kv head (one head per wave), so that a K/V tile is fetched once for the group.  Per tile of
// 64 keys, staged in LDS from the pages (K rows, and V rows of the transposed V cache):
//   S^T[64 keys x 32 queries] = K Q^T                 32x32x16 MFMAs, Q in registers
//   online softmax per query column (in-lane + one exchange between the lane halves)
//   O^T[D x 32 queries] += V^T P^T                    P never leaves registers
// The rows of the S tiles are permuted (row 8a+4h+b holds key 16(a/2)+8h+4(a%2)+b) so that the
// sixteen scores a lane holds per tile are keys 8h..8h+7 and 16+8h..16+8h+7: two operands of the
// second product as they are.
//
// Requires head_dim % 32 == 0 (32..256), page_size % 8 == 0 and block tables of at most 4096 pages
// (the table row is staged in LDS).  The launcher refuses anything else with an error; the host
// wrapper knows these limits and runs the general kernel instead.
#include "common.h"

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(4))) __bf16 bf16x4;
typedef __attribute__((ext_vector_type(16))) float f32x16;

#define PF_BM 32
#define PF_BN 64
#define PF_WAVES 4

struct Masked { static constexpr bool value = true; };     // a tile that the window's start or the diagonal cuts
struct Whole { static constexpr bool value = false; };     // a tile every row of the workgroup sees whole

template <int D>
// two waves per SIMD (at most 256 registers) up to head_dim 128; beyond that the accumulators need more
__global__ void __launch_bounds__(PF_WAVES * NVA_WAVE, D <= 128 ? 2 : 1)
attn_prefill_kernel(const __bf16* __restrict__ q, int64_t q_stride, __bf16* __restrict__ out, int64_t out_stride,
                    const __bf16* __restrict__ k_cache, const __bf16* __restrict__ v_cache,
                    const int32_t* __restrict__ block_tables, int table_stride,
                    const int32_t* __restrict__ cu_seqlens_q, const int32_t* __restrict__ kv_lens,
                    const int32_t* __restrict__ tiles, int num_tiles, int resident, int num_q_heads, int num_kv_heads,
                    int page_size, float scale, int window, int32_t* error_flag) {
    constexpr int KS = D + 8;             // K tile row stride (elements): 16 bytes of padding against bank conflicts
    constexpr int VS = PF_BN + 8;         // V tile row stride
    constexpr int DC = D / 16;            // 16-channel steps of the first product
    constexpr int MT = D / 32;            // 32-channel tiles of the output
    __shared__ __attribute__((aligned(16))) __bf16 k_s[PF_BN * KS];
    __shared__ __attribute__((aligned(16))) __bf16 v_s[D * VS];

    // ---- which request, which 32 rows of it, which heads.  `tiles` lists (request, row tile) from the
    // most keys to the fewest; a rank counts (tile, head chunk) pairs in that order.  Workgroups are
    // handed out in the order of their index, to the XCDs in turn and within an XCD to its CUs in turn:
    // with more workgroups than fit the GPU at once, the heaviest go first and the light ones fill the
    // gaps; with fewer, the first half of the indices takes the heavy ranks in order and the second half
    // the light ranks from the lightest, so that a CU's two workgroups are a heavy and a light one.
    const int ny = num_kv_heads * ((num_q_heads / num_kv_heads + PF_WAVES - 1) / PF_WAVES);
    const int total = num_tiles * ny;
    const int L = blockIdx.x;
    int rank = L;
    if (total <= resident) {
        const int heavy = 8 * ((total + 15) / 16);
        rank = L < heavy ? L : total - 1 - (L - heavy);
    }
    const int by = rank % ny;
    const int seq = tiles[2 * (rank / ny)], tile = tiles[2 * (rank / ny) + 1];
    const int q_begin = cu_seqlens_q[seq];
    const int q_len = cu_seqlens_q[seq + 1] - q_begin;
    const int kv_len = kv_lens[seq];
    const int start = kv_len - q_len;                 // position of the request's first query of this step
    const int q0 = tile * PF_BM;
    const int32_t* table = block_tables + (int64_t)seq * table_stride;

    const int vt = nva_v_tile(page_size);
    const int G = num_q_heads / num_kv_heads;
    const int chunks = (G + PF_WAVES - 1) / PF_WAVES;
    const int kvh = by / chunks, chunk = by % chunks;
    const int tid = threadIdx.x, wave = tid / NVA_WAVE, lane = tid % NVA_WAVE;
    const int col = lane & 31, h = lane >> 5;
    const int head_in_group = chunk * PF_WAVES + wave;
    const bool active = head_in_group < G;
    const int head = kvh * G + (active ? head_in_group : 0);

    const int row = q0 + col;                         // this lane's query row within the request's portion
    const bool row_ok = row < q_len;
    const int pos = start + row;

    // keys any row of the tile may see
    const int last_pos = start + min(q0 + PF_BM, q_len) - 1;
    const int first_any = window > 0 && start + q0 - window + 1 > 0 ? start + q0 - window + 1 : 0;
    const int kb_lo = first_any & ~(PF_BN - 1);
    const int kb_hi = last_pos + 1;                   // exclusive

    // ---- Q: column = query row, lane half h holds channels 16c + 8h .. + 7
    bf16x8 qf[DC];
    {
        const __bf16* qrow = q + (int64_t)(q_begin + (row_ok ? row : 0)) * q_stride + (int64_t)head * D + 8 * h;
#pragma unroll
        for (int c = 0; c < DC; ++c) {
            bf16x8 v = *reinterpret_cast<const bf16x8*>(qrow + 16 * c);
            if (!row_ok || !active) {
#pragma unroll
                for (int e = 0; e < 8; ++e) v[e] = (__bf16)0.f;
            }
            qf[c] = v;
        }
    }

    f32x16 acc[MT];
#pragma unroll
    for (int i = 0; i < MT; ++i)
#pragma unroll
        for (int e = 0; e < 16; ++e) acc[i][e] = 0.f;
    float m_run = -INFINITY, l_run = 0.f;

    // S tile row r = col holds key 16*(a/2) + 8*h' + 4*(a%2) + b with a = r/8, h' = (r/4)%2, b = r%4
    const int a_r = col >> 3, h_r = (col >> 2) & 1, b_r = col & 3;
    const int row_key = 16 * (a_r >> 1) + 8 * h_r + 4 * (a_r & 1) + b_r;
    const int first_row = window > 0 && pos - window + 1 > 0 ? pos - window + 1 : 0;
    const float c_exp = scale * 1.4426950408889634f;      // scale * log2(e)

    // ---- the request's block table entries for the keys this workgroup reads, once, into LDS
    extern __shared__ int32_t table_s[];
    const int page_lo = kb_lo / page_size;
    const int num_pages = (kb_hi - 1) / page_size - page_lo + 1;
    for (int i = tid; i < num_pages; i += PF_WAVES * NVA_WAVE) {
        const int page = table[page_lo + i];
        // pages before the first visible key may have been given back (a window): no fault
        if (page < 0 && page_lo + i >= first_any / page_size && error_flag) atomicOr(error_flag, 2);
        table_s[i] = max(page, 0);
    }
    __syncthreads();

    // Staging of a tile, per thread: PIECES 16-byte pieces of K (row r = tid / (D/8) + i * 256 / (D/8))
    // and of V (channel d = tid / 8 + 32 i, the 8 keys of group tid % 8).  Every load is unconditional:
    // a key outside the visible range is replaced by the nearest visible one (its scores are masked by
    // the key index; V is zeroed when it is written to LDS, in the tiles at the two ends only).  The
    // loads of tile t + 1 are issued before the products of tile t.
    //
    // The tiles fall into three runs: those the window's start cuts, those every row sees whole, and
    // those the diagonal cuts.  The middle run, most of a long prompt, runs without any masking, and
    // where pages hold whole tiles (page_size % 64 == 0) its loads are one base address per tile, held
    // in scalar registers, plus an offset per thread that never changes.
    constexpr int PIECES = PF_BN * (D / 8) / (PF_WAVES * NVA_WAVE);
    static_assert(PF_BN * (D / 8) % (PF_WAVES * NVA_WAVE) == 0, "the tile divides over the threads");
    const int last_key = kb_hi - 1;
    bf16x8 k_reg[PIECES], v_reg[PIECES];
    auto issue_loads = [&](int kb) {
#pragma unroll
        for (int i = 0; i < PIECES; ++i) {
            const int idx = tid + i * PF_WAVES * NVA_WAVE;
            const int r = idx / (D / 8), piece = idx % (D / 8);
            const int key = min(max(kb + r, first_any), last_key);
            const int page = table_s[key / page_size - page_lo];
            k_reg[i] = *reinterpret_cast<const bf16x8*>(
                k_cache + (((int64_t)page * num_kv_heads + kvh) * page_size + key % page_size) * D + piece * 8);
        }
        const int grp = tid % (PF_BN / 8);
        const int key0 = min(max(kb + grp * 8, first_any & ~7), last_key & ~7);
        const int page = table_s[key0 / page_size - page_lo];
        const __bf16* vb = v_cache + ((int64_t)page * num_kv_heads + kvh) * D * (int64_t)page_size;
#pragma unroll
        for (int i = 0; i < PIECES; ++i) {
            const int d = tid / (PF_BN / 8) + i * (PF_WAVES * NVA_WAVE / (PF_BN / 8));
            v_reg[i] = *reinterpret_cast<const bf16x8*>(vb + nva_v_offset(key0 % page_size, d, D, vt));
        }
    };
    // a tile that lies whole in one page and is visible whole: kb % 64 == 0, page_size % 64 == 0
    const int k_thread = (tid / (D / 8)) * D + (tid % (D / 8)) * 8;                 // + i * rows_per_pass * D
    constexpr int K_PASS = (PF_WAVES * NVA_WAVE / (D / 8)) * D;
    const int v_thread = (((tid % 8) / 4) * D + tid / 8) * 32 + ((tid % 8) % 4) * 8;   // + i * 32 channels * 32
    constexpr int V_PASS = (PF_WAVES * NVA_WAVE / (PF_BN / 8)) * 32;
    auto issue_loads_fast = [&](int kb) {
        const int page = __builtin_amdgcn_readfirstlane(table_s[kb / page_size - page_lo]);
        const int kip = kb % page_size;
        const __bf16* kbase = k_cache + (((int64_t)page * num_kv_heads + kvh) * page_size + kip) * D;
        const __bf16* vbase = v_cache + ((int64_t)page * num_kv_heads + kvh) * D * (int64_t)page_size + (int64_t)(kip / 32) * D * 32;
#pragma unroll
        for (int i = 0; i < PIECES; ++i) k_reg[i] = *reinterpret_cast<const bf16x8*>(kbase + k_thread + i * K_PASS);
#pragma unroll
        for (int i = 0; i < PIECES; ++i) v_reg[i] = *reinterpret_cast<const bf16x8*>(vbase + v_thread + i * V_PASS);
    };
    // (the split of a thread's pieces into a fixed offset and a step per pass needs 256 % (D / 8) == 0)
    const bool fast_pages = page_size % PF_BN == 0 && (PF_WAVES * NVA_WAVE) % (D / 8) == 0;

    // One tile: registers -> LDS, the next tile's loads, scores, softmax, second product.
    auto round = [&](int kb, auto masked_tag, int next_kb, bool next_fast) {
        constexpr bool MASKED = decltype(masked_tag)::value;
#pragma unroll
        for (int i = 0; i < PIECES; ++i) {
            const int idx = tid + i * PF_WAVES * NVA_WAVE;
            const int r = idx / (D / 8), piece = idx % (D / 8);
            *reinterpret_cast<bf16x8*>(&k_s[r * KS + piece * 8]) = k_reg[i];
        }
        {
            const int grp = tid % (PF_BN / 8);
            const int key0 = kb + grp * 8;
            const bool edge = MASKED && (kb < first_any || kb + PF_BN > kb_hi);  // the same for the whole workgroup
#pragma unroll
            for (int i = 0; i < PIECES; ++i) {
                const int d = tid / (PF_BN / 8) + i * (PF_WAVES * NVA_WAVE / (PF_BN / 8));
                bf16x8 v = v_reg[i];
                if (edge) {
#pragma unroll
                    for (int e = 0; e < 8; ++e)
                        if (key0 + e >= kb_hi || key0 + e < first_any) v[e] = (__bf16)0.f;
                }
                *reinterpret_cast<bf16x8*>(&v_s[d * VS + grp * 8]) = v;
            }
        }
        __syncthreads();
        if (next_fast) issue_loads_fast(next_kb);
        else issue_loads(next_kb);

        if (active) {
            // ---- scores of 2 x 32 keys
            f32x16 s[2];
#pragma unroll
            for (int kt = 0; kt < 2; ++kt) {
#pragma unroll
                for (int e = 0; e < 16; ++e) s[kt][e] = 0.f;
                const __bf16* krow = &k_s[(kt * 32 + row_key) * KS + 8 * h];
#pragma unroll
                for (int c = 0; c < DC; ++c) {
                    const bf16x8 a = *reinterpret_cast<const bf16x8*>(krow + 16 * c);
                    s[kt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, qf[c], s[kt], 0, 0, 0);
                }
            }
            // this lane: query `col`; register e of tile kt is key kb + 32*kt + 16*(e/8) + 8*h + e%8.
            // The maximum is taken of the raw scores (scale > 0) and the scale folded, with log2(e),
            // into the exponent: p = 2^((s - m) * scale * log2 e), one fused multiply-add per score.
            float m_new = m_run;
            if (MASKED) {
#pragma unroll
                for (int kt = 0; kt < 2; ++kt)
#pragma unroll
                    for (int e = 0; e < 16; ++e) {
                        const int key = kb + 32 * kt + 16 * (e >> 3) + 8 * h + (e & 7);
                        if (key > pos || key < first_row) s[kt][e] = -INFINITY;
                    }
            }
#pragma unroll
            for (int kt = 0; kt < 2; ++kt)
#pragma unroll
                for (int e = 0; e < 16; ++e) m_new = fmaxf(m_new, s[kt][e]);
            m_new = fmaxf(m_new, __shfl_xor(m_new, 32, NVA_WAVE));
            // a row that has seen no key yet keeps -inf as its maximum; exponents then use a finite
            // stand-in so that -inf - (-inf) never arises
            const float m_use = fmaxf(m_new, -1e30f);
            const float neg_mc = -m_use * c_exp;
            float psum = 0.f;
            bf16x8 pf[2][2];
#pragma unroll
            for (int kt = 0; kt < 2; ++kt)
#pragma unroll
                for (int e = 0; e < 16; ++e) {
                    const float p = __builtin_amdgcn_exp2f(fmaf(s[kt][e], c_exp, neg_mc));
                    pf[kt][e >> 3][e & 7] = (__bf16)p;
                    psum += p;
                }
            psum += __shfl_xor(psum, 32, NVA_WAVE);
            // The accumulators are rescaled only when some row of the wave has a new maximum (after the
            // first tiles of a row that is rare): alpha is exactly 1 otherwise.
            const float alpha = __builtin_amdgcn_exp2f((fmaxf(m_run, -1e30f) - m_use) * c_exp);
            const bool rescale = __any(m_new > m_run);
            l_run = l_run * alpha + psum;
            m_run = m_new;
            // ---- O^T += V^T P^T
#pragma unroll
            for (int mt = 0; mt < MT; ++mt) {
                f32x16 o = acc[mt];
                if (rescale) {
#pragma unroll
                    for (int e = 0; e < 16; ++e) o[e] *= alpha;
                }
                const __bf16* vrow = &v_s[(mt * 32 + col) * VS + 8 * h];
#pragma unroll
                for (int kt = 0; kt < 2; ++kt)
#pragma unroll
                    for (int ks = 0; ks < 2; ++ks) {
                        const bf16x8 a = *reinterpret_cast<const bf16x8*>(vrow + kt * 32 + ks * 16);
                        o = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, pf[kt][ks], o, 0, 0, 0);
                    }
                acc[mt] = o;
            }
        }
        __syncthreads();
    };

    // whole tiles: kb in [whole_lo, whole_hi)
    const int whole_lo = window > 0 ? (first_any + PF_BM + PF_BN - 1) & ~(PF_BN - 1) : kb_lo;
    const int whole_hi = (start + q0 + 1) & ~(PF_BN - 1);
    const int a_end = min(max(whole_lo, kb_lo), (kb_hi + PF_BN - 1) & ~(PF_BN - 1));
    const int b_end = max(a_end, min(whole_hi, kb_hi));
    const int after_last = last_key & ~(PF_BN - 1);                      // after the last tile: read again, dropped
    if (a_end < b_end && fast_pages && kb_lo == a_end) issue_loads_fast(kb_lo);
    else issue_loads(kb_lo);
    int kb = kb_lo;
    for (; kb < a_end; kb += PF_BN) round(kb, Masked(), min(kb + PF_BN, after_last), false);
    for (; kb < b_end - PF_BN; kb += PF_BN) round(kb, Whole(), kb + PF_BN, fast_pages);
    if (kb < b_end) {
        round(kb, Whole(), min(kb + PF_BN, after_last), false);
        kb += PF_BN;
    }
    for (; kb < kb_hi; kb += PF_BN) round(kb, Masked(), min(kb + PF_BN, after_last), false);

    // acc[mt][4a + b] = O[query col][channel 32*mt + 8a + 4h + b]
    if (!active || !row_ok) return;
    const float inv = l_run > 0.f ? 1.f / l_run : 0.f;
    __bf16* orow = out + (int64_t)(q_begin + row) * out_stride + (int64_t)head * D;
#pragma unroll
    for (int mt = 0; mt < MT; ++mt)
#pragma unroll
        for (int a = 0; a < 4; ++a) {
            bf16x4 v;
#pragma unroll
            for (int b = 0; b < 4; ++b) v[b] = (__bf16)(acc[mt][4 * a + b] * inv);
            *reinterpret_cast<bf16x4*>(orow + 32 * mt + 8 * a + 4 * h) = v;
        }
}

// tiles: int32 [num_tiles][2] = (request, row tile of 32 queries) for every tile of the step's
// portions, ordered from the most visible keys to the fewest (the caller builds it once per step).
// Refuses (non-zero code and a message) shapes this kernel does not take.
NVA_EXPORT int nva_attn_prefill_bf16(const void* q, int64_t q_stride, void* out, int64_t out_stride,
                                     const void* k_cache, const void* v_cache, const int32_t* block_tables,
                                     int table_stride, const int32_t* cu_seqlens_q, const int32_t* kv_lens,
                                     const int32_t* tiles, int64_t num_tiles, int num_q_heads,
                                     int num_kv_heads, int head_dim, int page_size, float scale, int window,
                                     int32_t* error_flag, hipStream_t stream) {
    if (num_tiles == 0) return 0;
    if (num_q_heads <= 0 || num_kv_heads <= 0 || num_q_heads % num_kv_heads)
        return nva_fail("attn_prefill: %d query heads do not divide into %d kv heads", num_q_heads, num_kv_heads);
    if (head_dim % 32 || head_dim < 32 || head_dim > 256 || page_size % 8 || page_size <= 0) {
        nva_fail("attn_prefill: needs head_dim %% 32 == 0 in 32..256 and page_size %% 8 == 0 (got %d, %d)", head_dim,
                 page_size);
        return 1;
    }
    const int G = num_q_heads / num_kv_heads;
    const int64_t grid_y = (int64_t)num_kv_heads * ((G + PF_WAVES - 1) / PF_WAVES);
    if (!tiles || num_tiles < 0 || num_tiles * grid_y > 0x7fffffff || window < 0 || table_stride <= 0)
        return nva_fail("attn_prefill: bad sizes (tiles %lld, heads %lld)", (long long)num_tiles, (long long)grid_y);
    if (table_stride > 4096) {
        nva_fail("attn_prefill: block tables of %d pages do not fit the kernel's staging buffer", table_stride);
        return 1;
    }
    const size_t table_bytes = (size_t)table_stride * sizeof(int32_t);
    // workgroups the GPU holds at once: two per CU (the kernel's registers allow no more)
    static int resident = 0;
    if (!resident) {
        int dev = 0, cus = 0;
        if (hipGetDevice(&dev) != hipSuccess || hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess)
            return nva_fail("attn_prefill: cannot read the number of CUs");
        resident = 2 * cus;
    }
    dim3 grid((unsigned)(num_tiles * grid_y));
#define LAUNCH(DD)                                                                                                 \
    hipLaunchKernelGGL(attn_prefill_kernel<DD>, grid, dim3(PF_WAVES * NVA_WAVE), table_bytes, stream, (const __bf16*)q, \
                       q_stride, (__bf16*)out, out_stride, (const __bf16*)k_cache, (const __bf16*)v_cache,           \
                       block_tables, table_stride, cu_seqlens_q, kv_lens, tiles, (int)num_tiles, resident,           \
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
        default: return nva_fail("attn_prefill: head_dim %d has no instance", head_dim);
    }
#undef LAUNCH
    return nva_check_launch("attn_prefill");
}

NVA_DEFINE_LAST_ERROR(nva_attn_prefill)
