// y[M, N] = x[M, K] W[N, K]^T (bfloat16) for 17 rows of x and more: the linear layers of a step of
// many tokens (nanovllm/layers/linear.py:51,73,153), where a weight is read once and shared by all the
// step's rows.  An LDS-tiled product on the matrix cores: a workgroup of four waves takes BM rows of
// x (all of them, up to 256; a grid dimension beyond) and BN rows of W over a range of k, in chunks
// of 64.  Both tiles go from global memory straight into LDS (16 bytes per lane, a wave's load fills
// eight rows of 128 bytes: whole cache lines), STAGES chunks in a ring, so that STAGES - 1 chunks are
// on their way while one is being multiplied; no registers hold data in flight.  One barrier per chunk.
// The layout that keeps the products' reads of LDS free of bank conflicts is an XOR of a 16-byte
// piece's place in its row with the row's number, made by choosing which bytes each lane fetches.
// Each wave multiplies a (BM / WM) x (BN / WN) part with 32x32x16 MFMAs, x as the A operand (rows of
// the result tile) and W as the B operand (its columns), so that 32 lanes hold 32 neighbouring
// columns of one row of y.  A weight of few rows is shared out over k as well (grid.y ranges), each
// workgroup writing float partial sums [range][M][N] for the consumer to add.
//
// Requires K % 64 == 0 and 16-byte aligned rows; the launcher refuses anything else (code 1) and the
// caller runs another kernel.
#include "common.h"

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(16))) float f32x16;

#ifndef TL_BK
#define TL_BK 64                                  // k of a chunk: 64 or 128
#endif
#define TL_WAVES 4
#define TL_ROW_BYTES (TL_BK * 2)
#define TL_LOAD_ROWS (1024 / TL_ROW_BYTES)        // rows of a tile that one load of a wave fills
#define TL_PIECES (TL_BK / 8)                     // 16-byte pieces of a row
// the turn of a row's pieces: rows whose pieces of one number would meet in the same banks get
// different turns (a row is 128 or 256 bytes, LDS serves 256 bytes at once)
__device__ __forceinline__ int tl_turn(int row) { return TL_BK == 64 ? (row / 2) % 8 : row % 16; }

enum { TL_PLAIN = 0, TL_PLAIN_F32 = 1, TL_GATED = 2, TL_PARTIAL = 3 };

struct TileArgs {
    const __bf16* x; int64_t x_stride;
    const __bf16* w; int64_t w_stride; const __bf16* bias;
    void* y; int64_t y_stride; float* partial; int mode;
    int M, N, K, chunks_per_range;
    int cols_per_wg;        // columns of y a workgroup takes: those of its tile, or fewer (the tile's other rows of W are not fetched)
};

// 16 bytes per lane from base + offset (base the same for the whole wave, offset in bytes per lane)
// to LDS at lds + 16 * lane (lds the same for the whole wave).  Written by hand: the compiler would
// make every later read of LDS wait for all such loads; these are waited for by count.
__device__ __forceinline__ void tl_load_to_lds(const __bf16* base, uint32_t offset, uint32_t lds) {
    asm volatile("s_mov_b32 m0, %2\n\tglobal_load_lds_dwordx4 %0, %1" ::"v"(offset), "s"(base), "s"(lds) : "memory", "m0");
}
// Workgroups walk the chunks of their range in rotated order, each from another start: at one k the
// rows of a tile (a power of two apart, as a rule) lie in few channels of the memory and of the L2,
// and workgroups that all fetch the same k at the same time queue up there.  (Past the range's end:
// its last chunk again.)
__device__ __forceinline__ uint32_t tl_chunk_offset(int c, int chunks, int rot) {
    const int cc = min(c, chunks - 1) + rot;
    return (uint32_t)(cc >= chunks ? cc - chunks : cc) * TL_ROW_BYTES;
}
// (the counter of loads on their way has six bits: the launcher refuses what would need more)
template <int N> __device__ __forceinline__ void tl_wait_loads_but() { asm volatile("s_waitcnt vmcnt(%0)" ::"n"(N < 64 ? N : 63) : "memory"); }
__device__ __forceinline__ void tl_barrier() { asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory"); }

// The products of one chunk of 64 k: x_stage and w_stage are the chunk's tiles in LDS, a_row / b_row
// the byte offsets of this lane's row in the first 32-row block of its wave's part, slot[ks] the byte
// offset of its piece in k step ks.  The fragments of a step are read while the products of the step
// before are running.
template <int TM, int TN>
__device__ __forceinline__ void tile_chunk(const char* x_stage, const char* w_stage, uint32_t a_row, uint32_t b_row,
                                           const uint32_t* slot, f32x16 (&acc)[TM][TN]) {
    bf16x8 fa[2][TM], fb[2][TN];
    auto read = [&](int ks, int buf) {
#pragma unroll
        for (int tm = 0; tm < TM; ++tm)
            fa[buf][tm] = *reinterpret_cast<const bf16x8*>(x_stage + a_row + tm * 32 * TL_ROW_BYTES + slot[ks]);
#pragma unroll
        for (int tn = 0; tn < TN; ++tn)
            fb[buf][tn] = *reinterpret_cast<const bf16x8*>(w_stage + b_row + tn * 32 * TL_ROW_BYTES + slot[ks]);
    };
    read(0, 0);
#pragma unroll
    for (int ks = 0; ks < TL_BK / 16; ++ks) {
        // the next step's reads of LDS go out before this step's products and complete during them
        // (pinned: with one wave per SIMD nothing else covers their latency)
        if (ks + 1 < TL_BK / 16) read(ks + 1, (ks + 1) & 1);
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int tm = 0; tm < TM; ++tm)
#pragma unroll
            for (int tn = 0; tn < TN; ++tn)
                acc[tm][tn] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fa[ks & 1][tm], fb[ks & 1][tn], acc[tm][tn], 0, 0, 0);
        __builtin_amdgcn_sched_barrier(0);
    }
}

// acc[tm][tn][v] = y[m][n], m = m_wave + 32 tm + 8 (v / 4) + 4 (lane / 32) + v % 4; n: column
// lane % 32 of block tn of the wave's part, which starts at column r_wave of the workgroup's tile.
template <int TM, int TN, int PART>
__device__ __forceinline__ void tile_store(const TileArgs& a, const f32x16 (&acc)[TM][TN], int m_wave, int n0, int wn, int lane) {
    const int half = lane / 32, r32 = lane % 32;
    const int inner = a.N / 2;
    if (a.mode == TL_GATED) {
        // the wave's part holds HALF gate columns and then the HALF up columns of the same outputs;
        // both are rounded before the gating, as the projection's output is (activation.py:8-11)
        constexpr int HALF = PART / 2;
        if constexpr (TN % 2 == 0) {
#pragma unroll
            for (int tm = 0; tm < TM; ++tm)
#pragma unroll
                for (int tn = 0; tn < TN / 2; ++tn)
#pragma unroll
                    for (int v = 0; v < 16; ++v) {
                        const int m = m_wave + tm * 32 + 8 * (v / 4) + 4 * half + v % 4;
                        const int j = n0 + wn * HALF + tn * 32 + r32;
                        const float gate = round_through<__bf16>(acc[tm][tn][v]);
                        const float up = round_through<__bf16>(acc[tm][tn + TN / 2][v]);
                        if (m < a.M && j < min(inner, n0 + a.cols_per_wg))
                            ((__bf16*)a.y)[(int64_t)m * a.y_stride + j] = (__bf16)(gate / (1.f + __expf(-gate)) * up);
                    }
        }
        return;
    }
    const int r_wave = wn * PART;
#pragma unroll
    for (int tm = 0; tm < TM; ++tm)
#pragma unroll
        for (int tn = 0; tn < TN; ++tn) {
            const int n = n0 + r_wave + tn * 32 + r32;
            float b = 0.f;
            if (a.bias && a.mode != TL_PARTIAL && n < a.N) b = (float)a.bias[n];
#pragma unroll
            for (int v = 0; v < 16; ++v) {
                const int m = m_wave + tm * 32 + 8 * (v / 4) + 4 * half + v % 4;
                if (m >= a.M || n >= min(a.N, n0 + a.cols_per_wg)) continue;
                const float val = acc[tm][tn][v] + b;
                if (a.mode == TL_PARTIAL) a.partial[((int64_t)blockIdx.y * a.M + m) * a.N + n] = val;
                else if (a.mode == TL_PLAIN_F32) ((float*)a.y)[(int64_t)m * a.y_stride + n] = val;
                else ((__bf16*)a.y)[(int64_t)m * a.y_stride + n] = (__bf16)val;
            }
        }
}

// The row of W that lies in LDS row r of the workgroup's W tile: BN rows in a row from n0, or
// (gated) for every wave's part half as many gate rows followed by the up rows that belong to them,
// so that a lane holds both of an output.  Kept inside the weight.
// A workgroup that takes fewer columns than its tile has fetches the row of its last column again
// in place of the others (the same line, found in the cache).
template <int PART>
__device__ __forceinline__ int tile_w_row(const TileArgs& a, int n0, int r) {
    if (a.mode != TL_GATED) return min(n0 + min(r, a.cols_per_wg - 1), a.N - 1);
    constexpr int HALF = PART / 2;
    const int inner = a.N / 2, part = r / PART, q = r % PART;
    const int col = min(part * HALF + (q < HALF ? q : q - HALF), a.cols_per_wg - 1);
    return min(n0 + col, inner - 1) + (q < HALF ? 0 : inner);
}

// Four waves that fetch and multiply: every wave brings its share of both tiles, STAGES chunks in
// one ring.  For steps of many rows, where the products are the bound.
template <int BM, int BN, int WM, int WN, int STAGES>
__global__ void __launch_bounds__(TL_WAVES * NVA_WAVE)
linear_tile_kernel(const TileArgs a) {
    static_assert(WM * WN == TL_WAVES, "four waves");
    constexpr int TM = BM / WM / 32, TN = BN / WN / 32;          // 32x32 tiles of a wave's part
    constexpr int ROWS = BM + BN;                                 // rows of a stage in LDS: x rows, then W rows
    constexpr int STAGE_BYTES = ROWS * TL_ROW_BYTES;
    constexpr int LOADS = ROWS / TL_LOAD_ROWS / TL_WAVES;         // loads per wave and chunk
    constexpr int X_LOADS = BM / TL_LOAD_ROWS / TL_WAVES;         // the first of them fetch rows of x
    static_assert(BM % 32 == 0 && BN % 32 == 0, "tile sizes");
    extern __shared__ __attribute__((aligned(1024))) char tl_lds[];
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / NVA_WAVE), lane = threadIdx.x % NVA_WAVE;
    const int wm = wave / WN, wn = wave % WN;
    const int m0 = blockIdx.z * BM;
    const int n0 = blockIdx.x * a.cols_per_wg;
    const int chunks_total = a.K / TL_BK;
    const int chunk_begin = blockIdx.y * a.chunks_per_range;
    const int chunks = min(a.chunks_per_range, chunks_total - chunk_begin);
    const int rot = (int)((blockIdx.x * 5u + blockIdx.y * 3u + blockIdx.z) % (unsigned)chunks);

    // ---- what this lane fetches: load i of this wave fills LDS rows 8 * (i * 4 + wave) .. + 7 of a stage;
    // the lane's place there is row lane / 8, slot lane % 8, and it fetches the piece that belongs there
    uint32_t src[LOADS];
#pragma unroll
    for (int i = 0; i < LOADS; ++i) {
        const int row = TL_LOAD_ROWS * (i * TL_WAVES + wave) + lane / TL_PIECES;     // row of the stage
        const int piece = (lane % TL_PIECES) ^ tl_turn(row);
        const int64_t elems = i < X_LOADS ? (int64_t)min(m0 + row, a.M - 1) * a.x_stride
                                          : (int64_t)tile_w_row<BN / WN>(a, n0, row - BM) * a.w_stride;
        src[i] = (uint32_t)((elems + (int64_t)chunk_begin * TL_BK + piece * 8) * 2);
    }
    const uint32_t lds_base = (uint32_t)(size_t)(__attribute__((address_space(3))) char*)tl_lds;
    auto issue = [&](int c) {                                     // chunk c of the range into its ring place
        const uint32_t stage = lds_base + (uint32_t)(c % STAGES) * STAGE_BYTES + wave * 1024;
        const uint32_t k_off = tl_chunk_offset(c, chunks, rot);
#pragma unroll
        for (int i = 0; i < LOADS; ++i)
            tl_load_to_lds(i < X_LOADS ? a.x : a.w, src[i] + k_off, __builtin_amdgcn_readfirstlane(stage + i * TL_WAVES * 1024));
    };

    // ---- what this lane reads: row lane % 32 of each 32-row block of its wave's part, pieces 2 * ks + lane / 32
    const int half = lane / 32, r32 = lane % 32;
    const int turn = tl_turn(r32);                                // the same for every block (blocks start at multiples of 32)
    const uint32_t a_row = (uint32_t)(wm * (BM / WM) + r32) * TL_ROW_BYTES;
    const uint32_t b_row = (uint32_t)(BM + wn * (BN / WN) + r32) * TL_ROW_BYTES;
    uint32_t slot[TL_BK / 16];
#pragma unroll
    for (int ks = 0; ks < TL_BK / 16; ++ks) slot[ks] = (uint32_t)(((2 * ks + half) ^ turn) * 16);

    f32x16 acc[TM][TN];
#pragma unroll
    for (int tm = 0; tm < TM; ++tm)
#pragma unroll
        for (int tn = 0; tn < TN; ++tn)
#pragma unroll
            for (int v = 0; v < 16; ++v) acc[tm][tn][v] = 0.f;

#pragma unroll
    for (int s = 0; s < STAGES - 1; ++s) issue(s);
    for (int c = 0; c < chunks; ++c) {
        tl_wait_loads_but<LOADS * (STAGES - 2)>();                // this wave's part of chunk c has landed
        tl_barrier();                                             // everybody's has, and chunk c - 1 is done with
        issue(c + STAGES - 1);
        const char* stage = tl_lds + (c % STAGES) * STAGE_BYTES;
        tile_chunk<TM, TN>(stage, stage, a_row, b_row, slot, acc);
    }
    tl_wait_loads_but<0>();                                       // the loads past the end, before the workgroup leaves
    tile_store<TM, TN, BN / WN>(a, acc, m0 + wm * (BM / WM), n0, wn, lane);
}

// Four waves that multiply and fetch W, and a fifth that fetches x: the x tiles have SX places in a
// ring of their own, the W tiles SW.  For steps of few rows, where the time is the time to stream W:
// what counts then is how many bytes of W are on their way, and a wave's loads complete in the order
// they were sent, so x (from the L2, back soon) must not queue behind W (from HBM) in one wave, nor
// take LDS that W could be flying into: x gets two or three places, W all the rest.
template <int BM, int BN, int WM, int WN, int SX, int SW>
__global__ void __launch_bounds__((TL_WAVES + 1) * NVA_WAVE)
linear_tile_fed_kernel(const TileArgs a) {
    static_assert(WM * WN == TL_WAVES, "four waves multiply");
    constexpr int TM = BM / WM / 32, TN = BN / WN / 32;
    constexpr int X_STAGE = BM * TL_ROW_BYTES, W_STAGE = BN * TL_ROW_BYTES;
    constexpr int XL = BM / TL_LOAD_ROWS, WL = BN / TL_LOAD_ROWS / TL_WAVES;   // loads per chunk: of the fifth wave, of each of the four
    extern __shared__ __attribute__((aligned(1024))) char tl_lds[];     // [SX] x tiles, then [SW] W tiles
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / NVA_WAVE), lane = threadIdx.x % NVA_WAVE;
    const int m0 = blockIdx.z * BM;
    const int n0 = blockIdx.x * a.cols_per_wg;
    const int chunks_total = a.K / TL_BK;
    const int chunk_begin = blockIdx.y * a.chunks_per_range;
    const int chunks = min(a.chunks_per_range, chunks_total - chunk_begin);
    const int rot = (int)((blockIdx.x * 5u + blockIdx.y * 3u + blockIdx.z) % (unsigned)chunks);
    const uint32_t lds_base = (uint32_t)(size_t)(__attribute__((address_space(3))) char*)tl_lds;

    if (wave == TL_WAVES) {                                       // ---- the wave that fetches x
        uint32_t src[XL];
#pragma unroll
        for (int i = 0; i < XL; ++i) {
            const int row = TL_LOAD_ROWS * i + lane / TL_PIECES;
            const int piece = (lane % TL_PIECES) ^ tl_turn(row);
            src[i] = (uint32_t)(((int64_t)min(m0 + row, a.M - 1) * a.x_stride + (int64_t)chunk_begin * TL_BK + piece * 8) * 2);
        }
        auto issue = [&](int c) {
            const uint32_t stage = lds_base + (uint32_t)(c % SX) * X_STAGE;
            const uint32_t k_off = tl_chunk_offset(c, chunks, rot);
#pragma unroll
            for (int i = 0; i < XL; ++i) tl_load_to_lds(a.x, src[i] + k_off, __builtin_amdgcn_readfirstlane(stage + i * 1024));
        };
#pragma unroll
        for (int s = 0; s < SX - 1; ++s) issue(s);
        for (int c = 0; c < chunks; ++c) {
            tl_wait_loads_but<XL * (SX - 2)>();
            tl_barrier();
            issue(c + SX - 1);
        }
        tl_wait_loads_but<0>();
        return;
    }
    // ---- the waves that multiply; load i of wave w fills rows 8 * (4 i + w) .. + 7 of a W tile
    uint32_t src[WL];
#pragma unroll
    for (int i = 0; i < WL; ++i) {
        const int row = TL_LOAD_ROWS * (i * TL_WAVES + wave) + lane / TL_PIECES;
        const int piece = (lane % TL_PIECES) ^ tl_turn(row);
        src[i] = (uint32_t)(((int64_t)tile_w_row<BN / WN>(a, n0, row) * a.w_stride + (int64_t)chunk_begin * TL_BK + piece * 8) * 2);
    }
    auto issue = [&](int c) {
        const uint32_t stage = lds_base + SX * X_STAGE + (uint32_t)(c % SW) * W_STAGE + wave * 1024;
        const uint32_t k_off = tl_chunk_offset(c, chunks, rot);
#pragma unroll
        for (int i = 0; i < WL; ++i) tl_load_to_lds(a.w, src[i] + k_off, __builtin_amdgcn_readfirstlane(stage + i * TL_WAVES * 1024));
    };
    const int wm = wave / WN, wn = wave % WN;
    const int half = lane / 32, r32 = lane % 32;
    const int turn = tl_turn(r32);
    const uint32_t a_row = (uint32_t)(wm * (BM / WM) + r32) * TL_ROW_BYTES;
    const uint32_t b_row = (uint32_t)(wn * (BN / WN) + r32) * TL_ROW_BYTES;
    uint32_t slot[TL_BK / 16];
#pragma unroll
    for (int ks = 0; ks < TL_BK / 16; ++ks) slot[ks] = (uint32_t)(((2 * ks + half) ^ turn) * 16);
    f32x16 acc[TM][TN];
#pragma unroll
    for (int tm = 0; tm < TM; ++tm)
#pragma unroll
        for (int tn = 0; tn < TN; ++tn)
#pragma unroll
            for (int v = 0; v < 16; ++v) acc[tm][tn][v] = 0.f;
#pragma unroll
    for (int s = 0; s < SW - 1; ++s) issue(s);
    for (int c = 0; c < chunks; ++c) {
        tl_wait_loads_but<WL * (SW - 2)>();                       // this wave's part of W chunk c has landed
        tl_barrier();                                             // all of chunk c has, and chunk c - 1 is done with
        issue(c + SW - 1);
        tile_chunk<TM, TN>(tl_lds + (c % SX) * X_STAGE, tl_lds + SX * X_STAGE + (c % SW) * W_STAGE, a_row, b_row, slot, acc);
    }
    tl_wait_loads_but<0>();
    tile_store<TM, TN, BN / WN>(a, acc, m0 + wm * (BM / WM), n0, wn, lane);
}

// y = x W^T.  mode: 0 elements (+ bias), 1 float (+ bias), 2 SwiGLU gating of W = [gate rows; up rows]
// (y [M, N / 2], no bias), 3 float partial sums [ranges][M][N] into `partial` (no bias: the consumer
// adds it).  shape: which tile the workgroups take and which kernel runs (see tile_shapes below; the
// gated form needs a tile of two column blocks per wave).  stages: chunks of W in LDS at once; ranges:
// parts the k range is cut into (> 1 only with mode 3); ranges_used receives how many there really
// are.  Returns 1 for shapes this kernel does not take (K not a multiple of 64, offsets beyond 32 bits).
struct TileShapeInfo { int bm, bn, wm, wn, fed, x_stages; };
static const TileShapeInfo tile_shapes[] = {
    {64, 128, 1, 4, 1, 3},     // 0: up to 64 rows, one column block per wave (no gating)
    {64, 128, 2, 2, 1, 3},     // 1: up to 64 rows
    {128, 128, 2, 2, 1, 3},    // 2: up to 128 rows
    {256, 128, 2, 2, 1, TL_BK == 64 ? 3 : 2},    // 3: up to 256 rows
    {64, 256, 1, 4, 1, 3},     // 4: up to 64 rows, wide
    {128, 128, 2, 2, 0, 0},    // 5: the waves fetch for themselves
    {256, 128, 2, 2, 0, 0},    // 6
    {256, 256, 2, 2, 0, 0},    // 7: many rows
};
NVA_EXPORT int nva_linear_tile_shapes() { return (int)(sizeof(tile_shapes) / sizeof(tile_shapes[0])); }

NVA_EXPORT int nva_linear_tile_bf16(const void* x, int64_t x_stride, const void* w, int64_t w_stride, const void* bias,
                                    void* y, int64_t y_stride, float* partial, int mode, int64_t M, int64_t N, int64_t K,
                                    int shape, int stages, int ranges, int cols_per_wg, int* ranges_used, hipStream_t stream) {
    // cols_per_wg: 0, or the columns of y one workgroup takes where that is to be fewer than its tile
    // has (64 of the gated form's 128 rows of W, else 128 or 256): more, lighter workgroups, so that
    // a weight's rows can be shared out evenly over the CUs.
    if (M == 0 || N == 0) return 0;
    if (M < 0 || N < 0 || K <= 0 || K % TL_BK || M > 0x7fffffff || N > 0x7fffffff ||
        (M * x_stride + K) * 2 > 0xffffffffLL || (N * w_stride + K) * 2 > 0xffffffffLL) {
        nva_fail("linear_tile: needs K %% 64 == 0 and operands below 4 GiB (M=%lld N=%lld K=%lld)", (long long)M,
                 (long long)N, (long long)K);
        return 1;
    }
    if (!x || !w || x_stride % 8 || w_stride % 8 || !nva_aligned(x, 16) || !nva_aligned(w, 16))
        return nva_fail("linear_tile: x and W need 16-byte aligned rows");
    if (mode < 0 || mode > 3) return nva_fail("linear_tile: unknown mode %d", mode);
    if (shape < 0 || shape >= nva_linear_tile_shapes()) return nva_fail("linear_tile: unknown tile shape %d", shape);
    const TileShapeInfo sh = tile_shapes[shape];
    if (mode == TL_GATED && (N % 2 || bias)) return nva_fail("linear_tile: the gated form needs an even number of weight rows and no bias");
    if (mode == TL_GATED && (sh.bn / sh.wn / 32) % 2) return nva_fail("linear_tile: the gated form needs a tile of two column blocks per wave");
    if (mode == TL_PARTIAL ? !partial : !y) return nva_fail("linear_tile: no output");
    if (ranges < 1 || ranges > 65535 || (ranges > 1 && mode != TL_PARTIAL))
        return nva_fail("linear_tile: %d ranges of k need the partial-sum mode", ranges);
    const size_t lds = sh.fed ? (size_t)(sh.x_stages * sh.bm + stages * sh.bn) * TL_ROW_BYTES
                              : (size_t)stages * (sh.bm + sh.bn) * TL_ROW_BYTES;
    if (stages < 2 || lds > 160 * 1024) return nva_fail("linear_tile: %d stages of tile shape %d do not fit LDS", stages, shape);
    const int x_loads = sh.bm / TL_LOAD_ROWS, w_loads = sh.bn / TL_LOAD_ROWS;
    if (sh.fed ? (x_loads * (sh.x_stages - 2) > 63 || w_loads / TL_WAVES * (stages - 2) > 63)
               : (x_loads + w_loads) / TL_WAVES * (stages - 2) > 63)
        return nva_fail("linear_tile: %d stages of tile shape %d are more loads on their way than a wave can count", stages, shape);
    TileArgs a;
    a.x = (const __bf16*)x; a.x_stride = x_stride;
    a.w = (const __bf16*)w; a.w_stride = w_stride; a.bias = (const __bf16*)bias;
    a.y = y; a.y_stride = y_stride; a.partial = partial; a.mode = mode;
    a.M = (int)M; a.N = (int)N; a.K = (int)K;
    const int chunks = (int)(K / TL_BK);
    a.chunks_per_range = (chunks + ranges - 1) / ranges;
    const int real_ranges = (chunks + a.chunks_per_range - 1) / a.chunks_per_range;
    const int64_t cols = mode == TL_GATED ? N / 2 : N;
    const int tile_cols = mode == TL_GATED ? sh.bn / 2 : sh.bn;
    if (cols_per_wg < 0 || cols_per_wg > tile_cols) return nva_fail("linear_tile: %d columns per workgroup of a tile of %d", cols_per_wg, tile_cols);
    const int per_wg = cols_per_wg ? cols_per_wg : tile_cols;
    a.cols_per_wg = per_wg;
    if ((cols + per_wg - 1) / per_wg > 0x7fffffff) return nva_fail("linear_tile: too many workgroups");
    const dim3 grid((unsigned)((cols + per_wg - 1) / per_wg), (unsigned)real_ranges, (unsigned)((M + sh.bm - 1) / sh.bm));
#define LAUNCH_KERNEL(KERNEL, THREADS)                                                                                 \
    do {                                                                                                               \
        static bool set = false;                                                                                       \
        if (!set) {                                                                                                    \
            if (hipFuncSetAttribute((const void*)KERNEL, hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024) != hipSuccess) \
                return nva_fail("linear_tile: cannot raise the kernel's LDS limit");                                   \
            set = true;                                                                                                \
        }                                                                                                              \
        hipLaunchKernelGGL(KERNEL, grid, dim3(THREADS), lds, stream, a);                                               \
    } while (0)
#define FED(BM, BN, WM, WN, SX)                                                                                        \
    do {                                                                                                               \
        switch (stages) {                                                                                              \
            case 2: LAUNCH_KERNEL((linear_tile_fed_kernel<BM, BN, WM, WN, SX, 2>), 320); break;                        \
            case 3: LAUNCH_KERNEL((linear_tile_fed_kernel<BM, BN, WM, WN, SX, 3>), 320); break;                        \
            case 4: LAUNCH_KERNEL((linear_tile_fed_kernel<BM, BN, WM, WN, SX, 4>), 320); break;                        \
            case 8: LAUNCH_KERNEL((linear_tile_fed_kernel<BM, BN, WM, WN, SX, 8>), 320); break;                        \
            default: return nva_fail("linear_tile: 2, 3, 4 or 8 stages are built for this tile, not %d", stages);                                    \
        }                                                                                                              \
    } while (0)
#define SELF(BM, BN, WM, WN)                                                                                           \
    do {                                                                                                               \
        switch (stages) {                                                                                              \
            case 2: LAUNCH_KERNEL((linear_tile_kernel<BM, BN, WM, WN, 2>), 256); break;                                \
            case 3: LAUNCH_KERNEL((linear_tile_kernel<BM, BN, WM, WN, 3>), 256); break;                                \
            default: return nva_fail("linear_tile: 2 or 3 stages are built for this tile, not %d", stages);                                    \
        }                                                                                                              \
    } while (0)
    switch (shape) {
        case 0: FED(64, 128, 1, 4, 3); break;
        case 1: FED(64, 128, 2, 2, 3); break;
        case 2: FED(128, 128, 2, 2, 3); break;
        case 3: FED(256, 128, 2, 2, (TL_BK == 64 ? 3 : 2)); break;
        case 4: FED(64, 256, 1, 4, 3); break;
        case 5: SELF(128, 128, 2, 2); break;
        case 6: SELF(256, 128, 2, 2); break;
        default: SELF(256, 256, 2, 2); break;
    }
#undef SELF
#undef FED
#undef LAUNCH_KERNEL
    if (ranges_used) *ranges_used = real_ranges;
    return nva_check_launch("linear_tile");
}

NVA_DEFINE_LAST_ERROR(nva_gemm_tile)
