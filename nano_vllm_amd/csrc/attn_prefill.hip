// Prefill attention on the matrix cores (bfloat16): portions of prompts against the paged cache.
//
// Semantics as in attn_generic.hip (nanovllm/layers/attention.py:64-70: causal, the diagonal
// aligned to the end of the keys when a request has cached tokens before this step's).  A request
// with q_len new tokens and kv_len tokens in the cache after this step has its query i at position
// kv_len - q_len + i; it reads keys first..position, first = max(0, position - window + 1) with a
// window, else 0.  The step's own keys are in the cache already.
//
// Work split: a workgroup takes 32 query rows of one request and up to 4 query heads of one kv head
// (one head per wave), so that a K/V tile is fetched once for the group.  A CU holds 8 of these waves
// (their registers): two workgroups, which fill each other's waits.  Where a step has no more
// workgroups than the GPU has CUs, a workgroup has two such sets of 4 waves instead: the sets take the
// tiles of 64 keys in turn (set 0 the even ones, set 1 the odd ones), each with tile buffers, running
// maxima, sums and accumulators of its own, and at the end set 0 adds set 1's, passed through LDS;
// this way all 8 waves of a CU work on its one workgroup's rows.  Per tile:
//   S^T[64 keys x 32 queries] = K Q^T                 32x32x16 MFMAs, Q in registers, K from LDS
//   online softmax per query column (in-lane + one exchange between the lane halves)
//   O^T[D x 32 queries] += V^T P^T                    P never leaves registers, V^T from LDS
// The rows of the S tiles are permuted (row 8a+4h+b holds key 16(a/2)+8h+4(a%2)+b) so that the
// sixteen scores a lane holds per tile are keys 8h..8h+7 and 16+8h..16+8h+7: two operands of the
// second product as they are.
//
// The tiles come from the pages into LDS without passing registers (16 bytes per lane and load, a
// wave's 64 lanes to 1 KB in a row), two tiles ahead for K and one for V, each into one of two
// buffers.  Such a load fixes where in LDS a lane's bytes go, not which bytes it fetches, so the
// layout that keeps the products' reads free of bank conflicts is made on that side: of a row of R
// 16-byte pieces, piece p lies in slot (p ^ turn(row)) of its group of 16, 8 or 4 slots.
//
// Requires head_dim % 32 == 0 (32..256), page_size % 8 == 0 and block tables of at most 4096 pages
// (the table row is staged in LDS).  The launcher refuses anything else with an error; the host
// wrapper knows these limits and runs the general kernel instead.
#include "common.h"

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(4))) __bf16 bf16x4;
typedef __attribute__((ext_vector_type(2))) __bf16 bf16x2;
typedef __attribute__((ext_vector_type(16))) float f32x16;

#define PF_BM 32
#define PF_BN 64
#define PF_WAVES 4
#ifndef PF_AHEAD
#define PF_AHEAD 7     // reads of LDS operands in flight before the product that uses the first
#endif

struct Masked { static constexpr bool value = true; };     // a tile that the window's start or the diagonal cuts
struct Whole { static constexpr bool value = false; };     // a tile every row of the workgroup sees whole
typedef Masked Yes;
typedef Whole No;

// Waves per SIMD: two (at most 256 registers each) up to head_dim 128; beyond that the accumulators need
// more.
#define PF_WAVES_PER_SIMD(D) ((D) <= 128 ? 2 : 1)

// Where the 16-byte pieces of a tile's rows lie in LDS.  Rows follow each other without padding, R
// pieces each; sixteen lanes read the same piece of sixteen rows in a row at a time, and LDS serves
// them at once if their slots differ modulo 16.  Rows 16 / GROUP apart share their banks, so the
// piece's place within its group of GROUP slots is turned by the row's number among those.
template <int R>
struct Swizzle {
    static constexpr int GROUP = R % 16 == 0 ? 16 : R % 8 == 0 ? 8 : 4;
    __device__ static __forceinline__ int slot(int row, int piece) {        // its own inverse
        const int turn = (row / (16 / GROUP)) % GROUP;
        return (piece & ~(GROUP - 1)) | ((piece ^ turn) & (GROUP - 1));
    }
};

// 16 bytes per lane from global memory to LDS at lds + 16 * lane (lds the same for the whole wave).
// Written out by hand: of the loads the compiler emits itself it takes every later read of LDS to
// depend, and waits for all of them before it.  These are waited for by count (wait_loads_but) and
// shown to the other waves by a barrier, as the schedule below says.
__device__ __forceinline__ void load_to_lds(const __bf16* src, uint32_t lds) {
    asm volatile("s_mov_b32 m0, %1\n\tglobal_load_lds_dwordx4 %0, off" ::"v"(src), "s"(__builtin_amdgcn_readfirstlane(lds)) : "memory", "m0");
}
// the same from base (the same for the whole wave) + offset (bytes, per lane)
__device__ __forceinline__ void load_to_lds(const __bf16* base, uint32_t offset, uint32_t lds) {
    asm volatile("s_mov_b32 m0, %2\n\tglobal_load_lds_dwordx4 %0, %1" ::"v"(offset), "s"(base), "s"(__builtin_amdgcn_readfirstlane(lds)) : "memory", "m0");
}

template <int N>
__device__ __forceinline__ void wait_loads_but() {          // until at most N loads of this wave are on their way
    asm volatile("s_waitcnt vmcnt(%0)" ::"n"(N) : "memory");
}

// The workgroup's barrier, after this wave's own LDS traffic is done.  (__syncthreads() would also
// wait for every load on its way to LDS.)
__device__ __forceinline__ void barrier() { asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory"); }

template <int D, int SETS>
__global__ void __launch_bounds__(SETS * PF_WAVES * NVA_WAVE, PF_WAVES_PER_SIMD(D))
attn_prefill_kernel(const __bf16* __restrict__ q, int64_t q_stride, __bf16* __restrict__ out, int64_t out_stride,
                    const __bf16* __restrict__ k_cache, const __bf16* __restrict__ v_cache,
                    const int32_t* __restrict__ block_tables, int table_stride,
                    const int32_t* __restrict__ cu_seqlens_q, const int32_t* __restrict__ kv_lens,
                    const int32_t* __restrict__ tiles, int num_tiles, int paired, int num_q_heads, int num_kv_heads,
                    int page_size, float scale, int window, int32_t* error_flag) {
    constexpr int DC = D / 16;            // 16-channel steps of the first product
    constexpr int MT = D / 32;            // 32-channel tiles of the output
    constexpr int KR = D / 8;             // 16-byte pieces of a K row (one key)
    constexpr int VR = PF_BN / 8;         // 16-byte pieces of a V row (one channel, the tile's 64 keys)
    constexpr int TILE = PF_BN * D;       // elements of a K tile, and of a V tile
    constexpr int PIECES = KR / PF_WAVES; // loads per wave and tile: 64 * KR pieces, 64 lanes, 4 waves
    constexpr int SET_THREADS = PF_WAVES * NVA_WAVE;
    typedef Swizzle<KR> SwK;
    typedef Swizzle<VR> SwV;
    // per set: two K tiles, two V tiles
    __shared__ __attribute__((aligned(16))) __bf16 tiles_s[SETS * 4 * TILE];
    static_assert(SETS == 1 || (size_t)PF_WAVES * NVA_WAVE * (D / 2 + 2) * sizeof(float) <= sizeof(tiles_s),
                  "set 1's accumulators, maxima and sums fit the tile buffers");

    // ---- which request, which 32 rows of it, which heads.  `tiles` lists (request, row tile) from the
    // most keys to the fewest; a rank counts (tile, head chunk) pairs in that order.  Workgroups are
    // handed out in the order of their index, to the XCDs in turn and within an XCD to its CUs in turn,
    // as many to a CU as it holds: the heaviest go first and the light ones fill the gaps.  Where all
    // of a step's workgroups are on the GPU at once, two to a CU (`paired`: their number then), the
    // first half of the indices takes the heavy ranks in order and the second half the light ranks from
    // the lightest, so that a CU's two workgroups are a heavy and a light one: the heavy one then works
    // alone (at one wave per SIMD) for the shortest time the pairing allows.  With as many head chunks
    // as XCDs, a kv head's keys and values stay in one XCD's L2.
    const int ny = num_kv_heads * ((num_q_heads / num_kv_heads + PF_WAVES - 1) / PF_WAVES);
    int rank = blockIdx.x;
    if (paired) {
        const int heavy = NVA_XCDS * ((paired + 2 * NVA_XCDS - 1) / (2 * NVA_XCDS));
        if (rank >= heavy) rank = paired - 1 - (rank - heavy);
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
    // Waves go to the SIMDs in turn: waves w and w + 4, one of each set, share one.
    const int set = __builtin_amdgcn_readfirstlane(threadIdx.x / SET_THREADS);     // which tiles of keys: set, set + SETS, ...
    const int tid = threadIdx.x % SET_THREADS, lane = tid % NVA_WAVE;
    const int wave = __builtin_amdgcn_readfirstlane(tid / NVA_WAVE);
    const int col = lane & 31, h = lane >> 5;
    __bf16* const set_s = tiles_s + set * 4 * TILE;   // K tiles at 0 and TILE, V tiles at 2 TILE and 3 TILE
    // where in LDS this wave's loads of a tile begin: buffer b of K at + b * 2 TILE bytes, of V at + (2 + b) * 2 TILE
    const uint32_t lds_wave = (uint32_t)(size_t)(__attribute__((address_space(3))) __bf16*)set_s + wave * NVA_WAVE * 16;
    constexpr uint32_t LOAD_BYTES = PF_WAVES * NVA_WAVE * 16;          // of the four waves' loads of one turn
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
    for (int i = threadIdx.x; i < num_pages; i += SETS * SET_THREADS) {
        const int page = table[page_lo + i];
        // pages before the first visible key may have been given back (a window): no fault
        if (page < 0 && page_lo + i >= first_any / page_size && error_flag) atomicOr(error_flag, 2);
        table_s[i] = max(page, 0);
    }
    // the Q loads are done before the tiles' loads are counted
    wait_loads_but<0>();
    barrier();

    // ---- the tiles' loads.  Load i of a wave fills the 64 slots from (4 i + wave) * 64 of the tile: of
    // K, slot n is row n / KR (a key), place n % KR; of V, row n / 8 (a channel), place n % 8 (eight
    // keys).  Every load is unconditional.  Where pages hold whole tiles (page_size % 64 == 0) a tile's
    // loads are one base address, held in scalar registers, plus an offset per lane that never changes;
    // else every lane looks its key's page up, and a key outside the visible range is replaced by the
    // nearest visible one.  Either way the scores of keys outside the range are masked by the key index
    // and what V holds for them is cleared in LDS, in the tiles at the two ends only.
    //
    // The tiles fall into three runs: those the window's start cuts, those every row sees whole, and
    // those the diagonal cuts.  The middle run, most of a long prompt, runs without any masking, and
    // where pages hold whole tiles (page_size % 64 == 0) its loads are one base address per tile, held
    // in scalar registers, plus an offset per lane that never changes.
    const int last_key = kb_hi - 1;
    // whole tiles: kb in [a_end, b_end)
    const int whole_lo = window > 0 ? (first_any + PF_BM + PF_BN - 1) & ~(PF_BN - 1) : kb_lo;
    const int whole_hi = (start + q0 + 1) & ~(PF_BN - 1);
    const int a_end = min(max(whole_lo, kb_lo), (kb_hi + PF_BN - 1) & ~(PF_BN - 1));
    const int b_end = max(a_end, min(whole_hi, kb_hi));
    const int after_last = last_key & ~(PF_BN - 1);                      // tiles after the last: it again, dropped
    const bool fast_pages = page_size % PF_BN == 0;
    uint32_t k_off[PIECES], v_off[PIECES];     // a lane's offsets from a whole tile's first key, in bytes
#pragma unroll
    for (int i = 0; i < PIECES; ++i) {
        const int n = (PF_WAVES * i + wave) * NVA_WAVE + lane;
        const int key = n / KR, piece = SwK::slot(key, n % KR);
        k_off[i] = (key * D + piece * 8) * 2;
        const int d = n / VR, group = SwV::slot(d, n % VR);              // keys 8 group .. 8 group + 7 of the tile
        v_off[i] = (((group / 4) * D + d) * 32 + (group % 4) * 8) * 2;
    }
    // a whole tile of one page: page * page_stride + head_off + (first key within the page) * D elements
    // from the cache's start, K and V alike (V's blocks of 32 keys are D * 32 elements each)
    const int64_t page_stride = (int64_t)num_kv_heads * page_size * D;
    const int64_t head_off = (int64_t)kvh * page_size * D;
    auto load_fast = [&](const __bf16* cache, int page, int kip, const uint32_t* off, uint32_t lds) __attribute__((always_inline)) {
        const uint64_t address = (uint64_t)(cache + (page * page_stride + head_off + (int64_t)kip * D));
        // (the same in every lane; said so for the scalar registers the loads take it from)
        const uint32_t low = __builtin_amdgcn_readfirstlane((uint32_t)address);
        const uint32_t high = __builtin_amdgcn_readfirstlane((uint32_t)(address >> 32));
        const __bf16* base = (const __bf16*)((uint64_t)high << 32 | low);
#pragma unroll
        for (int i = 0; i < PIECES; ++i) load_to_lds(base, off[i], lds + i * LOAD_BYTES);
    };
    // A tile in pages of whole tiles, wherever it lies: keys of it outside the visible range are
    // fetched as they are (they lie in the tile's own page; the scores of such keys are masked by the
    // key index and what V holds for them is cleared in LDS); a tile past the last is the last again.
    auto load_in_page = [&](const __bf16* cache, int kb, const uint32_t* off, uint32_t lds) __attribute__((always_inline)) {
        kb = min(kb, after_last);
        const int page = __builtin_amdgcn_readfirstlane(table_s[kb / page_size - page_lo]);
        load_fast(cache, page, kb % page_size, off, lds);
    };
    auto load_k_any = [&](int kb, int buf) __attribute__((always_inline)) {
        kb = min(kb, after_last);
        const uint32_t dst = lds_wave + buf * 2 * TILE;
#pragma unroll
        for (int i = 0; i < PIECES; ++i) {
            const int n = (PF_WAVES * i + wave) * NVA_WAVE + lane;
            const int r = n / KR, piece = SwK::slot(r, n % KR);
            const int key = min(max(kb + r, first_any), last_key);
            const int page = table_s[key / page_size - page_lo];
            load_to_lds(k_cache + (((int64_t)page * num_kv_heads + kvh) * page_size + key % page_size) * D + piece * 8,
                        dst + i * LOAD_BYTES);
        }
    };
    auto load_v_any = [&](int kb, int buf) __attribute__((always_inline)) {
        kb = min(kb, after_last);
        const uint32_t dst = lds_wave + (2 + buf) * 2 * TILE;
#pragma unroll
        for (int i = 0; i < PIECES; ++i) {
            const int n = (PF_WAVES * i + wave) * NVA_WAVE + lane;
            const int d = n / VR, group = SwV::slot(d, n % VR);
            const int key0 = min(max(kb + group * 8, first_any & ~7), last_key & ~7);
            const int page = table_s[key0 / page_size - page_lo];
            load_to_lds(v_cache + ((int64_t)page * num_kv_heads + kvh) * D * (int64_t)page_size +
                            nva_v_offset(key0 % page_size, d, D, vt),
                        dst + i * LOAD_BYTES);
        }
    };
    // What this lane's own loads put into the V tile for keys outside the visible range is cleared
    // (after the loads have arrived, before the barrier that shows the tile to the other waves): a
    // probability of zero does not cancel what a cache entry never written may hold.
    auto clear_v_outside = [&](int kb, int buf) __attribute__((always_inline)) {
        __bf16* tile_v = set_s + (2 + buf) * TILE;
#pragma unroll
        for (int i = 0; i < PIECES; ++i) {
            const int n = (PF_WAVES * i + wave) * NVA_WAVE + lane;
            const int key0 = kb + SwV::slot(n / VR, n % VR) * 8;
            if (key0 + 8 > kb_hi || key0 < first_any) {
                bf16x8 v = *reinterpret_cast<bf16x8*>(tile_v + n * 8);
#pragma unroll
                for (int e = 0; e < 8; ++e)
                    if (key0 + e >= kb_hi || key0 + e < first_any) v[e] = (__bf16)0.f;
                *reinterpret_cast<bf16x8*>(tile_v + n * 8) = v;
            }
        }
    };

    // ---- the three steps of a tile
    f32x16 s[2];                 // scores of 2 x 32 keys
    bf16x8 pf[2][2];             // their exponentials, the operands of the second product
    float alpha = 1.f;           // what the accumulators are to be scaled by before the tile's product is added
    bool rescale = false;
    // this lane: query `col`; register e of tile kt is key kb + 32*kt + 16*(e/8) + 8*h + e%8.
    // The maximum is taken of the raw scores (scale > 0) and the scale folded, with log2(e),
    // into the exponent: p = 2^((s - m) * scale * log2 e), one fused multiply-add per score.
    auto softmax = [&](int kb, auto masked_tag) __attribute__((always_inline)) {
        float m_new = m_run;
        if (decltype(masked_tag)::value) {
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
        float of_lower, of_upper;
        nva_lane_halves(m_new, of_lower, of_upper);
        m_new = fmaxf(of_lower, of_upper);
        // a row that has seen no key yet keeps -inf as its maximum; exponents then use a finite
        // stand-in so that -inf - (-inf) never arises
        const float m_use = fmaxf(m_new, -1e30f);
        const float neg_mc = -m_use * c_exp;
        // the sum is taken of the rounded values, the ones the second product weighs V with, two
        // of them per instruction
        float psum = 0.f;
        const bf16x2 ones = {(__bf16)1.f, (__bf16)1.f};
#pragma unroll
        for (int kt = 0; kt < 2; ++kt)
#pragma unroll
            for (int e = 0; e < 16; e += 2) {
                const bf16x2 pair = {(__bf16)__builtin_amdgcn_exp2f(fmaf(s[kt][e], c_exp, neg_mc)),
                                     (__bf16)__builtin_amdgcn_exp2f(fmaf(s[kt][e + 1], c_exp, neg_mc))};
                pf[kt][e >> 3][e & 7] = pair[0];
                pf[kt][e >> 3][(e & 7) + 1] = pair[1];
                psum = __builtin_amdgcn_fdot2_f32_bf16(pair, ones, psum, false);
            }
        nva_lane_halves(psum, of_lower, of_upper);
        psum = of_lower + of_upper;
        // The accumulators are rescaled only when some row of the wave has a new maximum (after the
        // first tiles of a row that is rare): alpha is exactly 1 otherwise.
        alpha = __builtin_amdgcn_exp2f((fmaxf(m_run, -1e30f) - m_use) * c_exp);
        rescale = __any(m_new > m_run);
        l_run = l_run * alpha + psum;
        m_run = m_new;
    };
    // The two products of an interval: O^T += V^T P^T of one tile (buffer v_buf; with_values), then the
    // scores of the next (buffer k_buf).  Their operands from LDS are fetched PF_AHEAD products ahead of
    // the one that uses them, through one ring of registers over both (the compiler by itself leaves
    // each pair of products waiting for its own reads).
    //   second product: step i = 2 kt + ks of a channel tile reads pieces 2i and 2i + 1 (the lane halves) of the channels' rows
    //   first product:  step c reads pieces 2c and 2c + 1 of the keys' rows
    int v_rd[4];                                 // this lane's offsets in a V tile for steps 0 .. 3, channel tile 0
#pragma unroll
    for (int i = 0; i < 4; ++i) v_rd[i] = (col * VR + SwV::slot(col, 2 * i + h)) * 8;
    constexpr int KG = SwK::GROUP / 2;           // steps whose pieces lie in one group of slots
    int k_rd[KG];                                // this lane's offsets in a K tile for steps 0 .. KG - 1, key half 0
#pragma unroll
    for (int c = 0; c < KG; ++c) k_rd[c] = (row_key * KR + SwK::slot(row_key, 2 * c + h)) * 8;
    auto products_of = [&](int v_buf, int k_buf, auto with_values) __attribute__((always_inline)) {
        constexpr int NV = decltype(with_values)::value ? 4 * MT : 0;   // 4 steps of 16 keys for every 32 channels
        constexpr int N = NV + 2 * DC;                                    // 16-channel steps of both key halves
        bf16x8 ring[PF_AHEAD + 1];
        const __bf16* tile_v = set_s + (2 + v_buf) * TILE;
        const __bf16* tile_k = set_s + k_buf * TILE;
        auto fetch = [&](int n) __attribute__((always_inline)) {
            if (n < NV) {
                ring[n % (PF_AHEAD + 1)] = *reinterpret_cast<const bf16x8*>(tile_v + v_rd[n % 4] + (n / 4) * 32 * VR * 8);
            } else {
                const int kt = (n - NV) / DC, c = (n - NV) % DC;
                ring[n % (PF_AHEAD + 1)] = *reinterpret_cast<const bf16x8*>(
                    tile_k + k_rd[c % KG] + kt * 32 * KR * 8 + (c / KG) * SwK::GROUP * 8);
            }
        };
#pragma unroll
        for (int n = 0; n < PF_AHEAD && n < N; ++n) fetch(n);
        if (NV && rescale) {
#pragma unroll
            for (int mt = 0; mt < MT; ++mt)
#pragma unroll
                for (int e = 0; e < 16; ++e) acc[mt][e] *= alpha;
        }
#pragma unroll
        for (int n = 0; n < N; ++n) {
            if (n + PF_AHEAD < N) fetch(n + PF_AHEAD);
            __builtin_amdgcn_sched_barrier(0);
            if (n < NV) {
                const int i = n % 4;
                acc[n / 4] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(ring[n % (PF_AHEAD + 1)], pf[i >> 1][i & 1], acc[n / 4], 0, 0, 0);
            } else {
                const int kt = (n - NV) / DC, c = (n - NV) % DC;
                if (c == 0) {
#pragma unroll
                    for (int e = 0; e < 16; ++e) s[kt][e] = 0.f;
                }
                s[kt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(ring[n % (PF_AHEAD + 1)], qf[c], s[kt], 0, 0, 0);
            }
            __builtin_amdgcn_sched_barrier(0);
        }
    };

    // ---- the schedule.  A set's tile j (keys from kb) takes two intervals between barriers:
    //   exponentials: the loads of K of tile j + 2 and of V of tile j + 1 are sent off, the softmax of
    //                 tile j's scores (vector unit), the wait for K of tile j + 1 and V of tile j;
    //   products:     O += P V of tile j, the scores of tile j + 1 (matrix cores, operands from LDS).
    // Tile j's K lies in buffer j % 2 and so does its V.  With two sets, set 1 runs one interval behind
    // set 0 (it passes one barrier before it starts, set 0 one after it has ended), so that on every
    // SIMD one wave is in its products while the other is in its exponentials.  Both sets run as many
    // rounds as set 0 has tiles; a round past a set's last tile adds nothing (every key is masked).
    constexpr int STEP = SETS * PF_BN;
    int buf = 0;                 // of this round's tile
    auto products = [&]() __attribute__((always_inline)) {
        wait_loads_but<2 * PIECES>();
        barrier();
        if (active) products_of(buf, buf ^ 1, Yes());
        barrier();
        buf ^= 1;
    };
    auto load_k = [&](int kb, int b) __attribute__((always_inline)) {
        if (fast_pages) load_in_page(k_cache, kb, k_off, lds_wave + b * 2 * TILE);
        else load_k_any(kb, b);
    };
    auto load_v = [&](int kb, int b) __attribute__((always_inline)) {
        if (fast_pages) load_in_page(v_cache, kb, v_off, lds_wave + (2 + b) * 2 * TILE);
        else load_v_any(kb, b);
    };
    auto round = [&](int kb, auto masked_tag) __attribute__((always_inline)) {
        if (active) softmax(kb, masked_tag);
        load_k(kb + 2 * STEP, buf);
        load_v(kb + STEP, buf ^ 1);
        wait_loads_but<2 * PIECES>();
        if (decltype(masked_tag)::value && (kb < first_any || kb + PF_BN > kb_hi)) clear_v_outside(kb, buf);
        products();
    };
    // A round of the run of whole tiles in pages of whole tiles.  Which page the tile after the next
    // lies in, and where, follows from where the next lies; its page number is looked up (in LDS)
    // before the softmax and used after it.
    int next_page = 0, next_entry = 0, next_kip = 0;      // of the tile at kb + STEP: page, its entry in table_s, first key within
    auto start_fast = [&](int kb) __attribute__((always_inline)) {
        next_entry = (kb + STEP) / page_size - page_lo;
        next_kip = (kb + STEP) % page_size;
        next_page = __builtin_amdgcn_readfirstlane(table_s[next_entry]);
    };
    auto round_fast = [&](int kb) __attribute__((always_inline)) {
        int entry = next_entry, kip = next_kip + STEP;
        while (kip >= page_size) {
            kip -= page_size;
            ++entry;
        }
        const int looked_up = table_s[entry];
        if (active) softmax(kb, Whole());
        const int page = __builtin_amdgcn_readfirstlane(looked_up);
        load_fast(k_cache, page, kip, k_off, lds_wave + buf * 2 * TILE);
        load_fast(v_cache, next_page, next_kip, v_off, lds_wave + (2 + (buf ^ 1)) * 2 * TILE);
        next_page = page, next_entry = entry, next_kip = kip;
        products();
    };
    const int rounds = ((kb_hi - kb_lo + PF_BN - 1) / PF_BN + SETS - 1) / SETS;
    if (SETS > 1 && set == 1) barrier();
    int kb = kb_lo + set * PF_BN;
    load_k(kb, 0);
    load_k(kb + STEP, 1);
    load_v(kb, 0);
    wait_loads_but<2 * PIECES>();
    barrier();
    if (active) products_of(0, 0, No());
    barrier();
    int r = 0;
    for (; r < rounds && kb < a_end; ++r, kb += STEP) round(kb, Masked());
    if (fast_pages && r < rounds && kb + 2 * STEP < b_end) {
        start_fast(kb);
        for (; r < rounds && kb + 2 * STEP < b_end; ++r, kb += STEP) round_fast(kb);
    }
    for (; r < rounds && kb < b_end; ++r, kb += STEP) round(kb, Whole());
    for (; r < rounds; ++r, kb += STEP) round(kb, Masked());
    if (SETS > 1 && set == 0) barrier();
    // the last rounds' loads, which nothing reads, have to be in before the buffers are used again
    wait_loads_but<0>();
    barrier();

    // ---- set 1's share through LDS (each lane its own registers), added by set 0
    if (SETS > 1) {
        float* const share = reinterpret_cast<float*>(tiles_s) + wave * (MT * 16 + 2) * NVA_WAVE + lane;
        if (set == 1) {
#pragma unroll
            for (int mt = 0; mt < MT; ++mt)
#pragma unroll
                for (int e = 0; e < 16; ++e) share[(mt * 16 + e) * NVA_WAVE] = acc[mt][e];
            share[MT * 16 * NVA_WAVE] = m_run;
            share[(MT * 16 + 1) * NVA_WAVE] = l_run;
        }
        barrier();
        if (set != 0) return;
        const float m_other = share[MT * 16 * NVA_WAVE], l_other = share[(MT * 16 + 1) * NVA_WAVE];
        const float m_use = fmaxf(fmaxf(m_run, m_other), -1e30f);
        const float f_own = __builtin_amdgcn_exp2f((fmaxf(m_run, -1e30f) - m_use) * c_exp);
        const float f_other = __builtin_amdgcn_exp2f((fmaxf(m_other, -1e30f) - m_use) * c_exp);
        l_run = l_run * f_own + l_other * f_other;
#pragma unroll
        for (int mt = 0; mt < MT; ++mt)
#pragma unroll
            for (int e = 0; e < 16; ++e) acc[mt][e] = acc[mt][e] * f_own + share[(mt * 16 + e) * NVA_WAVE] * f_other;
    }

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
// nva_attn_prefill_sets (-1, 1 or 2) fixes the sets of waves per workgroup for tests; -1 leaves the choice
// to the launcher.
// Refuses (non-zero code and a message) shapes this kernel does not take.
static int forced_sets = -1;
NVA_EXPORT void nva_attn_prefill_sets(int sets) { forced_sets = sets; }

NVA_EXPORT int nva_attn_prefill_bf16(const void* q, int64_t q_stride, void* out, int64_t out_stride,
                                     const void* k_cache, const void* v_cache, const int32_t* block_tables,
                                     int table_stride, const int32_t* cu_seqlens_q, const int32_t* kv_lens,
                                     const int32_t* tiles, int64_t num_tiles, int num_q_heads,
                                     int num_kv_heads, int head_dim, int page_size, float scale, int window,
                                     int32_t* error_flag, hipStream_t stream) {
    if (num_tiles == 0) return 0;
    if (num_q_heads <= 0 || num_kv_heads <= 0 || num_q_heads % num_kv_heads)
        return nva_fail("attn_prefill: %d query heads do not divide into %d kv heads", num_q_heads, num_kv_heads);
    if (!(scale > 0.f) || !(scale <= 3.0e38f)) {
        // the running maximum is taken of the raw scores and the scale folded into the exponent
        nva_fail("attn_prefill: needs a positive, finite scale (got %g)", (double)scale);
        return 1;
    }
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
    dim3 grid((unsigned)(num_tiles * grid_y));
    static int cus = 0;
    if (!cus) {
        int dev = 0;
        if (hipGetDevice(&dev) != hipSuccess || hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || cus <= 0) {
            cus = 0;
            return nva_fail("attn_prefill: cannot read the number of CUs");
        }
    }
    // two sets of waves in a workgroup where every CU gets one workgroup at most
    const int64_t total = num_tiles * grid_y;
    const bool two_sets = forced_sets > 0 ? forced_sets == 2 : total <= cus;
#define LAUNCH_SETS(DD, SS)                                                                                        \
    hipLaunchKernelGGL((attn_prefill_kernel<DD, SS>), grid, dim3(SS * PF_WAVES * NVA_WAVE), table_bytes, stream,     \
                       (const __bf16*)q, q_stride, (__bf16*)out, out_stride, (const __bf16*)k_cache,                 \
                       (const __bf16*)v_cache, block_tables, table_stride, cu_seqlens_q, kv_lens, tiles,             \
                       (int)num_tiles, SS == 1 && PF_WAVES_PER_SIMD(DD) == 2 && total <= 2 * cus ? (int)total : 0,   \
                       num_q_heads, num_kv_heads, page_size, scale, window, error_flag)
#define LAUNCH(DD)                                                                                                 \
    do {                                                                                                           \
        if (PF_WAVES_PER_SIMD(DD) == 2 && two_sets) LAUNCH_SETS(DD, PF_WAVES_PER_SIMD(DD));                         \
        else LAUNCH_SETS(DD, 1);                                                                                   \
    } while (0)
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
#undef LAUNCH_SETS
    return nva_check_launch("attn_prefill");
}

NVA_DEFINE_LAST_ERROR(nva_attn_prefill)
