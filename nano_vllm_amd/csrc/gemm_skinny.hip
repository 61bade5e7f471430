// y[M, N] = x[M, K] W[N, K]^T for few rows (bfloat16): the linear layers of a decode step
// (nanovllm/layers/linear.py:51,73,153; embed_head.py:61), where every weight is read once and the
// time is the time to stream W from HBM.  Two kernels: linear_skinny_kernel for up to 64 rows of x
// (described first), linear_medium_kernel for up to 256.
//
// One wave owns 16 output columns (16 rows of W) over a range of k.  W rows are the A operand of
// a 16x16x32 MFMA, 16 rows of x its 16 columns (rows >= M idle); with more than 16 rows of x the
// same W fragment feeds one MFMA per block of 16 rows.  A lane reads four 16-byte pieces of its W
// row per step of 128 k (the k index is permuted alike in both operands), straight from global into
// registers; the workgroup's slice of x is staged in LDS.  For small N the k range is split over
// workgroups, each writing float partial sums; a second kernel adds the partials in a fixed order,
// applies the optional bias and the optional SwiGLU gating (W = [gate rows; up rows]) and rounds once.
//
// Requires K % 8 == 0 and 16-byte aligned rows; the launcher refuses anything else and the caller
// uses the library product or the tiled kernel.
#include "common.h"
#include "no_alloc.h"
#include <mutex>
#include <type_traits>

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(4))) __bf16 bf16x4;
typedef __attribute__((ext_vector_type(4))) float f32x4;

#define SK_KSTEP 128
#define SK_UNROLL 2
#define SK_MAX_ROWS 64

// Row blocks of x (MB) and waves per workgroup: more rows of x take more waves, so that a staged
// slice of x serves more rows of W.
template <int MB> struct SkShape;
template <> struct SkShape<1> { static constexpr int waves = 4; };
template <> struct SkShape<2> { static constexpr int waves = 8; };
template <> struct SkShape<4> { static constexpr int waves = 8; };
// KW waves of a workgroup may share 16 rows of W and take every KW-th step of k each; their sums
// meet in LDS.  That makes more and shorter waves without more partial sums in memory.

__device__ __forceinline__ bf16x8 zero8() {
    bf16x8 z;
#pragma unroll
    for (int e = 0; e < 8; ++e) z[e] = (__bf16)0.f;
    return z;
}

// direct: 0 = float partials [split][M][N]; 1 = the only split writes y itself (as bfloat16 or
// float); 2 = the same for W = [gate rows; up rows]: a wave then takes 8 gate rows and the 8 up rows
// that belong to them, and writes silu(gate) * up, [M][N / 2].
//
// The workgroup's waves share one range of k, so its slice of x is staged in LDS, `chunk` columns
// at a time (a multiple of 256; row stride padded by 16 bytes against bank conflicts): the M rows
// and one row of zeros, which the MFMA columns beyond M read.  Lane (row, g) takes the 16-byte piece
// g + 4c of its row's 256 bytes in load c, so that one load instruction covers 64 contiguous bytes
// of each of the wave's 16 rows; x is read from LDS at the same k.  The loads of a step of 256 k
// are issued at its top and the products wait for them one by one: the other waves of the CU cover
// the latency, so many short waves (a finer split of k) run faster than few long ones.  A chunk's
// first loads are issued before its slice of x is staged.  Only a ragged last step (K % 256) moves
// its offsets back into the row: what it reads beyond K meets zeros of x_s.
template <int MB, int WAVES, int KW>
__global__ void __launch_bounds__(WAVES * NVA_WAVE)
linear_skinny_kernel(const __bf16* __restrict__ x, int64_t x_stride, const __bf16* __restrict__ w, int64_t w_stride,
                     float* __restrict__ partial, void* __restrict__ y, int64_t y_stride, int y_is_f32, int direct,
                     int M, int N, int K, int k_per_split, int chunk) {
    constexpr int STEP = SK_KSTEP * SK_UNROLL;
    extern __shared__ __attribute__((aligned(16))) __bf16 x_s[];     // [M + 1][chunk + 8]
    const int wave = threadIdx.x / NVA_WAVE, lane = threadIdx.x % NVA_WAVE;
    const int col = lane & 15, g = lane >> 4;
    const int split = blockIdx.y;
    const int k_begin = split * k_per_split;
    const int k_end = min(K, k_begin + k_per_split);
    const int xs_stride = chunk + 8;

    const bool gated = direct == 2;
    const int inner = N / 2;
    const int tile = blockIdx.x * (WAVES / KW) + wave / KW;
    const int ksub = wave % KW;
    const int n0 = gated ? tile * 8 : tile * 16;
    const bool active = n0 < (gated ? inner : N);     // idle waves still help to stage x
    const int w_row = gated ? min(n0 + (col & 7), inner - 1) + (col >= 8 ? inner : 0) : min(n0 + col, N - 1);
    const __bf16* wrow = w + (int64_t)w_row * w_stride;
    f32x4 acc[MB];
    const __bf16* xrow[MB];
#pragma unroll
    for (int b = 0; b < MB; ++b) {
        acc[b] = f32x4{0.f, 0.f, 0.f, 0.f};
        xrow[b] = x_s + min(col + 16 * b, M) * xs_stride + 8 * g;
    }
    const int k_last = K - 8;
    bf16x8 a[SK_UNROLL][4];

#define SK_LOAD_CLAMPED(kk)                                                                                            \
    _Pragma("unroll") for (int u = 0; u < SK_UNROLL; ++u) _Pragma("unroll") for (int c = 0; c < 4; ++c)                \
        a[u][c] = *reinterpret_cast<const bf16x8*>(wrow + min((kk) + u * SK_KSTEP + 8 * g + 32 * c, k_last))
#define SK_PRODUCTS(off)                                                                                               \
    _Pragma("unroll") for (int u = 0; u < SK_UNROLL; ++u) _Pragma("unroll") for (int c = 0; c < 4; ++c)                \
        _Pragma("unroll") for (int b = 0; b < MB; ++b)                                                                 \
            acc[b] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(                                                          \
                a[u][c], *reinterpret_cast<const bf16x8*>(xrow[b] + (off) + u * SK_KSTEP + 32 * c), acc[b], 0, 0, 0)

    for (int c_begin = k_begin; c_begin < k_end; c_begin += chunk) {
        const int c_end = min(k_end, c_begin + chunk);
        const int len = c_end - c_begin;
        SK_LOAD_CLAMPED(c_begin + ksub * STEP);
        // ---- stage x[0:M][c_begin:c_begin + chunk] and the zero row (zeros beyond c_end as well)
        __syncthreads();
        for (int idx = threadIdx.x; idx < (M + 1) * (chunk / 8); idx += WAVES * NVA_WAVE) {
            const int m = idx / (chunk / 8), piece = idx % (chunk / 8);
            const int k = c_begin + piece * 8;
            bf16x8 v = zero8();
            if (m < M && k < c_end) v = *reinterpret_cast<const bf16x8*>(x + (int64_t)m * x_stride + k);
            *reinterpret_cast<bf16x8*>(&x_s[m * xs_stride + piece * 8]) = v;
        }
        __syncthreads();
        if (!active || ksub * STEP >= len) continue;
        SK_PRODUCTS(ksub * STEP);
        const int full = len / STEP;
        const bf16x8* wp = reinterpret_cast<const bf16x8*>(wrow + c_begin + 8 * g);
        int s = ksub + KW;
        for (; s < full; s += KW) {
#pragma unroll
            for (int u = 0; u < SK_UNROLL; ++u)
#pragma unroll
                for (int c = 0; c < 4; ++c) a[u][c] = wp[(s * STEP + u * SK_KSTEP + 32 * c) / 8];
            SK_PRODUCTS(s * STEP);
        }
        if (s == full && s * STEP < len) {
            SK_LOAD_CLAMPED(c_begin + s * STEP);
            SK_PRODUCTS(s * STEP);
        }
    }
#undef SK_LOAD_CLAMPED
#undef SK_PRODUCTS
    if (KW > 1) {
        // the sums of the waves that share rows of W meet in LDS (x_s is done with), in a fixed order
        f32x4* sums = reinterpret_cast<f32x4*>(x_s);                 // [WAVES][MB][lanes]
        __syncthreads();
        if (ksub != 0)
#pragma unroll
            for (int b = 0; b < MB; ++b) sums[(wave * MB + b) * NVA_WAVE + lane] = acc[b];
        __syncthreads();
        if (ksub != 0) return;
#pragma unroll
        for (int o = 1; o < KW; ++o)
#pragma unroll
            for (int b = 0; b < MB; ++b) {
                const f32x4 v = sums[((wave + o) * MB + b) * NVA_WAVE + lane];
                acc[b][0] += v[0]; acc[b][1] += v[1]; acc[b][2] += v[2]; acc[b][3] += v[3];
            }
    }
    if (!active) return;
    if (gated) {
        // acc[b][i] of lanes g < 2 is the gate of y[m = 16 * b + col][j = n0 + 4*g + i], the same register
        // of lane + 32 its up; both are rounded to bfloat16 before the gating as the reference's
        // projection is (activation.py:8-11)
#pragma unroll
        for (int b = 0; b < MB; ++b) {
            const int m = 16 * b + col;
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const float up = (float)(__bf16)__shfl(acc[b][i], (lane + 32) % NVA_WAVE, NVA_WAVE);
                const float gate = (float)(__bf16)acc[b][i];
                const int j = n0 + 4 * g + i;
                if (g < 2 && m < M && j < inner) {
                    const float v = gate / (1.f + __expf(-gate)) * up;
                    if (y_is_f32) ((float*)y)[(int64_t)m * y_stride + j] = v;
                    else ((__bf16*)y)[(int64_t)m * y_stride + j] = (__bf16)v;
                }
            }
        }
        return;
    }
    // acc[b][i] = y[m = 16 * b + col][n = n0 + 4*g + i]
    const int n = n0 + 4 * g;
#pragma unroll
    for (int b = 0; b < MB; ++b) {
        const int m = 16 * b + col;
        if (m >= M) continue;
        if (!direct) {
            float* p = partial + ((int64_t)split * M + m) * N + n;
            if (n + 3 < N && (N % 4) == 0) {
                *reinterpret_cast<f32x4*>(p) = acc[b];
            } else {
#pragma unroll
                for (int i = 0; i < 4; ++i)
                    if (n + i < N) p[i] = acc[b][i];
            }
        } else if (y_is_f32) {
            float* p = (float*)y + (int64_t)m * y_stride + n;
#pragma unroll
            for (int i = 0; i < 4; ++i)
                if (n + i < N) p[i] = acc[b][i];
        } else {
            __bf16* p = (__bf16*)y + (int64_t)m * y_stride + n;
#pragma unroll
            for (int i = 0; i < 4; ++i)
                if (n + i < N) p[i] = (__bf16)acc[b][i];
        }
    }
}

// The same product for more rows of x (up to 256), where the slice of x no longer fits LDS for a
// long range of k and the reads of x from LDS weigh as much as the products.  A workgroup of four
// waves takes 16 * RT rows of W per wave and walks its k range in chunks of 128: the chunk of x
// lies in LDS twice (the next one is fetched into registers during the products and written to
// the other half, one barrier per chunk), every fragment of x read from LDS feeds RT products, and
// each 16-byte piece of W is asked for again, one chunk ahead, as soon as its products are issued.
// direct and the layout of the results: as above.
#define MD_KC 128
#define MD_XS (MD_KC + 8)
#define MD_MAX_ROWS 256
// WAVES (3 or 4) and RT (1 to 3) set how many blocks of 16 weight rows a workgroup takes: a CU draws
// only about its share of the memory's bandwidth, so the product is as fast as its most loaded CU,
// and the launcher's caller picks the pair that spreads the weight's blocks evenly over the CUs.
template <int MB, int RT, int WAVES>
__global__ void __launch_bounds__(WAVES * NVA_WAVE) __attribute__((amdgpu_waves_per_eu(MB > 8 ? 1 : 2)))
linear_medium_kernel(const __bf16* __restrict__ x, int64_t x_stride, const __bf16* __restrict__ w, int64_t w_stride,
                     float* __restrict__ partial, void* __restrict__ y, int64_t y_stride, int y_is_f32, int direct,
                     int M, int N, int K, int k_per_split) {
    constexpr int ROWS = 16 * MB + 1;                                 // the last row stays zero when M = 16 * MB
    extern __shared__ __attribute__((aligned(16))) __bf16 x_s[];      // [2][ROWS][MD_XS]
    const int wave = threadIdx.x / NVA_WAVE, lane = threadIdx.x % NVA_WAVE;
    const int col = lane & 15, g = lane >> 4;
    const int split = blockIdx.y;
    const int k_begin = split * k_per_split;
    const int k_end = min(K, k_begin + k_per_split);
    const int chunks = (k_end - k_begin + MD_KC - 1) / MD_KC;
    const bool gated = direct == 2;
    const int inner = N / 2;
    const int per_tile = gated ? 8 : 16;
    const int tile0 = (blockIdx.x * WAVES + wave) * RT;
    const int k_last = K - 8;

    const __bf16* wrow[RT];
#pragma unroll
    for (int rt = 0; rt < RT; ++rt) {
        const int n0 = (tile0 + rt) * per_tile;
        const int w_row = gated ? min(n0 + (col & 7), inner - 1) + (col >= 8 ? inner : 0) : min(n0 + col, N - 1);
        wrow[rt] = w + (int64_t)w_row * w_stride + 8 * g;
    }
    int xoff[MB];
    f32x4 acc[RT][MB];
#pragma unroll
    for (int b = 0; b < MB; ++b) {
        xoff[b] = min(col + 16 * b, M) * MD_XS + 8 * g;
#pragma unroll
        for (int rt = 0; rt < RT; ++rt) acc[rt][b] = f32x4{0.f, 0.f, 0.f, 0.f};
    }
    // staging: thread t moves the 16-byte piece t % 16 of rows t / 16 + SR * j (below 16 * MB)
    constexpr int SR = WAVES * NVA_WAVE / 16, SJ = (16 * MB + SR - 1) / SR;
    const int s_row = threadIdx.x / 16, s_piece = threadIdx.x % 16;
    constexpr int XD = MB > 8 ? 1 : 2;                                // chunks that x is asked for ahead (registers allowing)
    bf16x8 xr[XD][SJ];                                                // x of the next chunks, on its way
    // (every load of the loop is unconditional, from an address moved into the operand where it
    // would lie outside, and what must be zero is made zero when it is written to LDS: a branch
    // around a load makes the compiler wait for all loads in flight at every turn)
    auto fetch_x = [&](int k0, bf16x8* xr) {
#pragma unroll
        for (int j = 0; j < SJ; ++j)
            xr[j] = *reinterpret_cast<const bf16x8*>(x + (int64_t)min(s_row + SR * j, M - 1) * x_stride +
                                                     min(k0 + 8 * s_piece, k_last));
    };
    auto store_x = [&](int buf, int k0, const bf16x8* xr) {
        const bool k_ok = k0 + 8 * s_piece < k_end;
#pragma unroll
        for (int j = 0; j < SJ; ++j)
            if (16 * MB % SR == 0 || s_row + SR * j < 16 * MB)
                *reinterpret_cast<bf16x8*>(&x_s[(buf * ROWS + s_row + SR * j) * MD_XS + 8 * s_piece]) =
                    k_ok && s_row + SR * j < M ? xr[j] : zero8();
    };
    // Workgroups walk their chunks in rotated order, each from another start: at one k the rows of
    // x (a power of two apart, as a rule) lie in few channels of the L2, and workgroups that all
    // fetch the same chunk at the same time queue up there.
    const int rot = (blockIdx.x * 5 + blockIdx.y) % chunks;
    // (past the last chunk: K, from where every load is moved back to the rows' last pieces)
    auto k_of = [&](int c) { return c < chunks ? k_begin + (c + rot) % chunks * MD_KC : K; };
    // x is asked for two chunks ahead (a chunk's products take less time than a load from the L2),
    // every piece of W one chunk ahead, as soon as its products are issued
    bf16x8 a[RT][4];
    fetch_x(k_of(0), xr[0]);
#pragma unroll
    for (int rt = 0; rt < RT; ++rt)
#pragma unroll
        for (int c = 0; c < 4; ++c)
            a[rt][c] = *reinterpret_cast<const bf16x8*>(wrow[rt] + min(k_of(0) + 32 * c, k_last - 8 * g));
    if (threadIdx.x < 2 * (MD_XS / 8)) {                              // the row beyond the staged ones, in both halves
        const int buf = threadIdx.x / (MD_XS / 8), piece = threadIdx.x % (MD_XS / 8);
        *reinterpret_cast<bf16x8*>(&x_s[(buf * ROWS + ROWS - 1) * MD_XS + 8 * piece]) = zero8();
    }
    store_x(0, k_of(0), xr[0]);
    if (XD == 2) fetch_x(k_of(1), xr[XD - 1]);
    __syncthreads();
    auto chunk = [&](int c, auto half) {
        constexpr int H = decltype(half)::value;                      // the half of x_s this chunk reads
        const int k_next = k_of(c + 1), k_ahead = k_of(c + 2);
        if (XD == 2) fetch_x(k_ahead, xr[H % XD]);                    // xr[H ^ 1] holds the next chunk's
        else fetch_x(k_next, xr[0]);
        const __bf16* xb = x_s + H * ROWS * MD_XS;
        // The fragments of x come from LDS in groups of GS, one group ahead of the products that use
        // them: with one or two waves per SIMD nothing else covers the latency of LDS.
        constexpr int GS = MB % 4 == 0 ? 4 : 2, GROUPS = 4 * MB / GS;          // groups of a chunk: (piece p, blocks b)
        bf16x8 frag[2][GS];
#pragma unroll
        for (int i = 0; i < GS; ++i) frag[0][i] = *reinterpret_cast<const bf16x8*>(xb + xoff[i]);
#pragma unroll
        for (int gi = 0; gi < GROUPS; ++gi) {
            constexpr int PER_P = MB / GS;
            const int p = gi / PER_P, b0 = gi % PER_P * GS;
            if (gi + 1 < GROUPS) {
                const int pn = (gi + 1) / PER_P, bn = (gi + 1) % PER_P * GS;
#pragma unroll
                for (int i = 0; i < GS; ++i)
                    frag[(gi + 1) & 1][i] = *reinterpret_cast<const bf16x8*>(xb + xoff[bn + i] + 32 * pn);
            }
            __builtin_amdgcn_sched_barrier(0);                        // keep the reads ahead of the products
#pragma unroll
            for (int i = 0; i < GS; ++i)
#pragma unroll
                for (int rt = 0; rt < RT; ++rt)
                    acc[rt][b0 + i] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a[rt][p], frag[gi & 1][i], acc[rt][b0 + i], 0, 0, 0);
            __builtin_amdgcn_sched_barrier(0);
            if (gi % PER_P == PER_P - 1)
#pragma unroll
                for (int rt = 0; rt < RT; ++rt)  // past the last chunk all lanes read one piece of the first row
                    a[rt][p] = *reinterpret_cast<const bf16x8*>((c + 1 < chunks ? wrow[rt] : w + 8 * g) + min(k_next + 32 * p, k_last - 8 * g));
        }
        store_x(H ^ 1, k_next, xr[(H ^ 1) % XD]);                                    // after the last chunk: written, never read
        __syncthreads();
    };
    for (int c = 0; c < chunks; c += 2) {
        chunk(c, std::integral_constant<int, 0>());
        if (c + 1 < chunks) chunk(c + 1, std::integral_constant<int, 1>());
    }
#pragma unroll
    for (int rt = 0; rt < RT; ++rt) {
        const int n0 = (tile0 + rt) * per_tile;
        if (n0 >= (gated ? inner : N)) continue;
        if (gated) {
#pragma unroll
            for (int b = 0; b < MB; ++b) {
                const int m = 16 * b + col;
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    const float up = (float)(__bf16)__shfl(acc[rt][b][i], (lane + 32) % NVA_WAVE, NVA_WAVE);
                    const float gate = (float)(__bf16)acc[rt][b][i];
                    const int j = n0 + 4 * g + i;
                    if (g < 2 && m < M && j < inner) {
                        const float v = gate / (1.f + __expf(-gate)) * up;
                        if (y_is_f32) ((float*)y)[(int64_t)m * y_stride + j] = v;
                        else ((__bf16*)y)[(int64_t)m * y_stride + j] = (__bf16)v;
                    }
                }
            }
            continue;
        }
        const int n = n0 + 4 * g;
#pragma unroll
        for (int b = 0; b < MB; ++b) {
            const int m = 16 * b + col;
            if (m >= M) continue;
            if (!direct) {
                float* p = partial + ((int64_t)split * M + m) * N + n;
                if (n + 3 < N && (N % 4) == 0) {
                    *reinterpret_cast<f32x4*>(p) = acc[rt][b];
                } else {
#pragma unroll
                    for (int i = 0; i < 4; ++i)
                        if (n + i < N) p[i] = acc[rt][b][i];
                }
            } else if (y_is_f32) {
                float* p = (float*)y + (int64_t)m * y_stride + n;
#pragma unroll
                for (int i = 0; i < 4; ++i)
                    if (n + i < N) p[i] = acc[rt][b][i];
            } else {
                __bf16* p = (__bf16*)y + (int64_t)m * y_stride + n;
#pragma unroll
                for (int i = 0; i < 4; ++i)
                    if (n + i < N) p[i] = (__bf16)acc[rt][b][i];
            }
        }
    }
}

// y[m][n] = sum over splits of partial[s][m][n] (+ bias[n]); with swiglu, N is the width of the
// partials (2 * inner) and y[m][j] = silu(sum_gate[j]) * sum_up[j], j < inner.
__global__ void __launch_bounds__(256)
linear_skinny_finish_kernel(const float* __restrict__ partial, int splits, const __bf16* __restrict__ bias,
                            void* __restrict__ y, int64_t y_stride, int y_is_f32, int swiglu, int M, int N) {
    const int out_n = swiglu ? N / 2 : N;
    const int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (idx >= (int64_t)M * out_n) return;
    const int m = (int)(idx / out_n), j = (int)(idx % out_n);
    float v = 0.f, u = 0.f;
    for (int s = 0; s < splits; ++s) {
        const float* p = partial + ((int64_t)s * M + m) * N;
        v += p[j];
        if (swiglu) u += p[out_n + j];
    }
    if (bias) {
        v += (float)bias[j];
        if (swiglu) u += (float)bias[out_n + j];
    }
    if (swiglu) {
        // the reference rounds the projection to bfloat16 before the gating (activation.py:8-11)
        v = (float)(__bf16)v;
        u = (float)(__bf16)u;
        v = v / (1.f + __expf(-v)) * u;
    }
    if (y_is_f32) ((float*)y)[(int64_t)m * y_stride + j] = v;
    else ((__bf16*)y)[(int64_t)m * y_stride + j] = (__bf16)v;
}

// waves_per_tile: 1, 2 or 4 waves of a workgroup share 16 rows of W and split the k range between
// them (pays for very few rows of x).  splits: how many ranges k is cut into (>= 1); scratch must hold splits * M * N floats when
// splits > 1 or a bias, swiglu or defer_finish is asked for.  splits_used receives the number of
// ranges really used (k per range is rounded up to a multiple of 256).  Refuses (non-zero code and a message) shapes this kernel does not take.
NVA_EXPORT int nva_linear_skinny_bf16(const void* x, int64_t x_stride, const void* w, int64_t w_stride,
                                      const void* bias, void* y, int64_t y_stride, int y_is_f32, int swiglu,
                                      float* scratch, int splits, int waves_per_tile, int defer_finish, int64_t M,
                                      int64_t N, int64_t K, int* splits_used, hipStream_t stream) {
    if (M == 0 || N == 0) return 0;
    if (M < 0 || M > SK_MAX_ROWS || K % 8 || K <= 0 || x_stride % 8 || w_stride % 8 || !nva_aligned(x, 16) || !nva_aligned(w, 16)) {
        nva_fail("linear_skinny: needs 1..%d rows, K %% 8 == 0 and 16-byte aligned rows (M=%lld K=%lld)", SK_MAX_ROWS,
                 (long long)M, (long long)K);
        return 1;
    }
    if (N > 0x7fffffff || K > 0x7fffffff || splits < 1 || splits > 65535) return nva_fail("linear_skinny: bad sizes");
    if (waves_per_tile != 1 && waves_per_tile != 2 && waves_per_tile != 4)
        return nva_fail("linear_skinny: 1, 2 or 4 waves share rows of W, not %d", waves_per_tile);
    if (swiglu && (N % 2)) return nva_fail("linear_skinny: the gated form needs an even number of weight rows");
    const int direct = splits == 1 && !bias && !defer_finish ? (swiglu ? 2 : 1) : 0;
    if (!direct && !scratch) return nva_fail("linear_skinny: this call needs scratch memory");
    int kps = (int)((K + splits - 1) / splits);
    kps = (kps + SK_KSTEP * SK_UNROLL - 1) / (SK_KSTEP * SK_UNROLL) * (SK_KSTEP * SK_UNROLL);
    const int real_splits = (int)((K + kps - 1) / kps);
    const int64_t tiles = direct == 2 ? (N / 2 + 7) / 8 : (N + 15) / 16;
    // columns of x staged at a time: about 36 KB of LDS for the M + 1 rows, so that several workgroups fit a CU
    int chunk = (36864 / (2 * ((int)M + 1)) - 8) / 256 * 256;
    chunk = chunk < 256 ? 256 : chunk > 2048 ? 2048 : chunk;
    if (chunk > kps) chunk = kps;
    size_t lds = (size_t)(M + 1) * (chunk + 8) * sizeof(__bf16);
#define LAUNCH(MB, KW)                                                                                                 \
    do {                                                                                                               \
        constexpr int waves = SkShape<MB>::waves, per_wg = waves / KW;                                                 \
        if (KW > 1 && lds < (size_t)waves * MB * NVA_WAVE * sizeof(f32x4)) lds = (size_t)waves * MB * NVA_WAVE * sizeof(f32x4); \
        dim3 grid((unsigned)((tiles + per_wg - 1) / per_wg), (unsigned)real_splits);                                   \
        hipLaunchKernelGGL((linear_skinny_kernel<MB, waves, KW>), grid, dim3(waves * NVA_WAVE), lds, stream,                  \
                           (const __bf16*)x, x_stride, (const __bf16*)w, w_stride, scratch, y, y_stride, y_is_f32,     \
                           direct, (int)M, (int)N, (int)K, kps, chunk);                                                \
    } while (0)
#define LAUNCH_KW(MB)                                                                                                  \
    do {                                                                                                               \
        if (waves_per_tile == 1) LAUNCH(MB, 1);                                                                        \
        else if (waves_per_tile == 2) LAUNCH(MB, 2);                                                                   \
        else LAUNCH(MB, 4);                                                                                            \
    } while (0)
    if (M <= 16) LAUNCH_KW(1);
    else if (M <= 32) LAUNCH_KW(2);
    else LAUNCH_KW(4);
#undef LAUNCH_KW
#undef LAUNCH
    if (splits_used) *splits_used = real_splits;
    int rc = nva_check_launch("linear_skinny");
    // deferred: the partial sums [real_splits][M][N] stay in scratch for a kernel that consumes them
    if (rc || direct || defer_finish) return rc;
    const int64_t outs = M * (swiglu ? N / 2 : N);
    hipLaunchKernelGGL(linear_skinny_finish_kernel, dim3((unsigned)((outs + 255) / 256)), dim3(256), 0, stream, scratch,
                       real_splits, (const __bf16*)bias, y, y_stride, y_is_f32, swiglu, (int)M, (int)N);
    return nva_check_launch("linear_skinny_finish");
}

// The kernel for up to 256 rows of x.  waves (3 or 4; 3 up to 96 rows of x) and row_tiles (1 to 3; 3 up
// to 96 rows, 1 beyond 224): a workgroup takes waves * row_tiles blocks of 16 rows of W.  The other arguments as for
// nva_linear_skinny; k per range is rounded up to a multiple of 128.
NVA_EXPORT int nva_linear_medium_bf16(const void* x, int64_t x_stride, const void* w, int64_t w_stride,
                                      const void* bias, void* y, int64_t y_stride, int y_is_f32, int swiglu,
                                      float* scratch, int splits, int row_tiles, int waves, int defer_finish, int64_t M,
                                      int64_t N, int64_t K, int* splits_used, hipStream_t stream) {
    if (M == 0 || N == 0) return 0;
    if (M < 0 || M > MD_MAX_ROWS || K % 8 || K <= 0 || x_stride % 8 || w_stride % 8 || !nva_aligned(x, 16) || !nva_aligned(w, 16)) {
        nva_fail("linear_medium: needs 1..%d rows, K %% 8 == 0 and 16-byte aligned rows (M=%lld K=%lld)", MD_MAX_ROWS,
                 (long long)M, (long long)K);
        return 1;
    }
    if (N > 0x7fffffff || K > 0x7fffffff || splits < 1 || splits > 65535) return nva_fail("linear_medium: bad sizes");
    const int mb = (int)((M + 15) / 16 + 1) / 2 * 2;                   // instances for 2, 4, 6, ... 16 blocks of 16 rows
    if (waves != 3 && waves != 4) return nva_fail("linear_medium: 3 or 4 waves per workgroup, not %d", waves);
    if (row_tiles < 1 || row_tiles > 3 || (row_tiles == 3 && mb > 6) || (row_tiles == 2 && mb > 14) || (waves == 3 && mb > 6))
        return nva_fail("linear_medium: %d row tiles per wave and %d waves are not built for %lld rows", row_tiles, waves, (long long)M);
    if (swiglu && (N % 2)) return nva_fail("linear_medium: the gated form needs an even number of weight rows");
    const int direct = splits == 1 && !bias && !defer_finish ? (swiglu ? 2 : 1) : 0;
    if (!direct && !scratch) return nva_fail("linear_medium: this call needs scratch memory");
    int kps = (int)((K + splits - 1) / splits);
    kps = (kps + MD_KC - 1) / MD_KC * MD_KC;
    const int real_splits = (int)((K + kps - 1) / kps);
    const int64_t tiles = direct == 2 ? (N / 2 + 7) / 8 : (N + 15) / 16;
    const size_t lds = (size_t)2 * (16 * mb + 1) * MD_XS * sizeof(__bf16);
#define LAUNCH(MB, RT, WV)                                                                                             \
    do {                                                                                                               \
        dim3 grid((unsigned)((tiles + WV * RT - 1) / (WV * RT)), (unsigned)real_splits);                               \
        hipLaunchKernelGGL((linear_medium_kernel<MB, RT, WV>), grid, dim3(WV * NVA_WAVE), lds, stream,                 \
                           (const __bf16*)x, x_stride, (const __bf16*)w, w_stride, scratch, y, y_stride, y_is_f32,     \
                           direct, (int)M, (int)N, (int)K, kps);                                                       \
    } while (0)
#define LAUNCH_SMALL(MB)                                                                                               \
    do {                                                                                                               \
        if (waves == 4) { if (row_tiles == 1) LAUNCH(MB, 1, 4); else if (row_tiles == 2) LAUNCH(MB, 2, 4); else LAUNCH(MB, 3, 4); } \
        else { if (row_tiles == 1) LAUNCH(MB, 1, 3); else if (row_tiles == 2) LAUNCH(MB, 2, 3); else LAUNCH(MB, 3, 3); } \
    } while (0)
#define LAUNCH_LARGE(MB)                                                                                               \
    do {                                                                                                               \
        if (row_tiles == 1) LAUNCH(MB, 1, 4);                                                                          \
        else LAUNCH(MB, 2, 4);                                                                                         \
    } while (0)
    switch (mb) {
        case 2: LAUNCH_SMALL(2); break;
        case 4: LAUNCH_SMALL(4); break;
        case 6: LAUNCH_SMALL(6); break;
        case 8: LAUNCH_LARGE(8); break;
        case 10: LAUNCH_LARGE(10); break;
        case 12: LAUNCH_LARGE(12); break;
        case 14: LAUNCH_LARGE(14); break;
        default: LAUNCH(16, 1, 4); break;      // more than 224 rows: one block of weight rows per wave (registers)
    }
#undef LAUNCH_SMALL
#undef LAUNCH_LARGE
#undef LAUNCH
    if (splits_used) *splits_used = real_splits;
    int rc = nva_check_launch("linear_medium");
    if (rc || direct || defer_finish) return rc;
    const int64_t outs = M * (swiglu ? N / 2 : N);
    hipLaunchKernelGGL(linear_skinny_finish_kernel, dim3((unsigned)((outs + 255) / 256)), dim3(256), 0, stream, scratch,
                       real_splits, (const __bf16*)bias, y, y_stride, y_is_f32, swiglu, (int)M, (int)N);
    return nva_check_launch("linear_skinny_finish");
}

// The finishing pass alone, for partial sums that were left by a call with defer_finish.
NVA_EXPORT int nva_linear_skinny_finish_bf16(const float* partial, int splits, const void* bias, void* y,
                                             int64_t y_stride, int y_is_f32, int swiglu, int64_t M, int64_t N,
                                             hipStream_t stream) {
    if (M == 0 || N == 0) return 0;
    if (!partial || splits <= 0 || M < 0 || N < 0 || N > 0x7fffffff || M > 0x7fffffff)
        return nva_fail("linear_skinny_finish: bad arguments");
    const int64_t outs = M * (swiglu ? N / 2 : N);
    hipLaunchKernelGGL(linear_skinny_finish_kernel, dim3((unsigned)((outs + 255) / 256)), dim3(256), 0, stream, partial,
                       splits, (const __bf16*)bias, y, y_stride, y_is_f32, swiglu, (int)M, (int)N);
    return nva_check_launch("linear_skinny_finish");
}

// ---------------------------------------------------------------------------- without allocation
// The partial sums of nva_linear_skinny_static live here (no_alloc.h).  In host code the array's
// name is a stand-in, not a device address: the address on each device is asked for once, with that
// device current, and only that pointer is handed to kernels.
static __device__ __align__(256) float scratch[NVA_STATIC_SCRATCH_FLOATS];

#define NVA_MAX_DEVICES 64
static float* static_scratch_ptr[NVA_MAX_DEVICES];
static std::mutex static_scratch_lock;

// The current device's copy of the array, or null after leaving a message.
static float* static_scratch() {
    int dev = -1;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess || dev < 0 || dev >= NVA_MAX_DEVICES) {
        nva_fail("linear_skinny_static: no current device (%s)", hipGetErrorString(e));
        return nullptr;
    }
    std::lock_guard<std::mutex> hold(static_scratch_lock);
    if (!static_scratch_ptr[dev]) {
        float* ptr = nullptr;
        e = hipGetSymbolAddress((void**)&ptr, HIP_SYMBOL(scratch));
        if (e != hipSuccess || !ptr) {
            nva_fail("linear_skinny_static: the address of the static scratch array on device %d is not to be had (%s)",
                     dev, hipGetErrorString(e));
            return nullptr;
        }
        static_scratch_ptr[dev] = ptr;
    }
    return static_scratch_ptr[dev];
}

static int skinny_real_splits(int splits, int64_t K) {
    int kps = (int)((K + splits - 1) / splits);
    kps = (kps + SK_KSTEP * SK_UNROLL - 1) / (SK_KSTEP * SK_UNROLL) * (SK_KSTEP * SK_UNROLL);
    return (int)((K + kps - 1) / kps);
}

NVA_EXPORT int64_t nva_linear_skinny_static_need_bf16(const void* bias, int swiglu, int splits, int64_t M, int64_t N,
                                                      int64_t K) {
    if (splits < 1 || M <= 0 || N <= 0 || K <= 0) return 0;
    if (splits == 1 && !bias) return 0;                    // the product kernel writes y itself (gated or not)
    return (int64_t)skinny_real_splits(splits, K) * M * N;
}

NVA_EXPORT int nva_linear_skinny_static_bf16(const void* x, int64_t x_stride, const void* w, int64_t w_stride,
                                             const void* bias, void* y, int64_t y_stride, int y_is_f32, int swiglu,
                                             int splits, int waves_per_tile, int64_t M, int64_t N, int64_t K,
                                             int* splits_used, hipStream_t stream) {
    if (M == 0 || N == 0) return 0;
    if (M < 0 || N < 0 || K <= 0 || splits < 1 || splits > 65535) return nva_fail("linear_skinny_static: bad sizes");
    const int64_t need = nva_linear_skinny_static_need_bf16(bias, swiglu, splits, M, N, K);
    if (need > NVA_STATIC_SCRATCH_FLOATS)
        return nva_fail("linear_skinny_static: %lld ranges of k x %lld rows x %lld columns need %lld floats of partial "
                        "sums; the static array holds %lld (16 MiB): fewer ranges, or the entry point with a workspace",
                        (long long)skinny_real_splits(splits, K), (long long)M, (long long)N, (long long)need,
                        (long long)NVA_STATIC_SCRATCH_FLOATS);
    float* ptr = static_scratch();
    if (!ptr) return -1;
    return nva_linear_skinny_bf16(x, x_stride, w, w_stride, bias, y, y_stride, y_is_f32, swiglu, ptr, splits,
                                  waves_per_tile, 0, M, N, K, splits_used, stream);
}

NVA_DEFINE_LAST_ERROR(nva_gemm_skinny)
