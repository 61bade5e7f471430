// y[M, N] = x[M, K] * W[N, K]^T (+ bias[N]): the linear layer of
// nanovllm/layers/linear.py:51,73,153 and the output head of embed_head.py:61, with the weight
// in its stored [out, in] layout.
//
// This is the tiled kernel on the vector units: inputs are read as they are stored, every
// product and sum is a float operation (no matrix-core instruction, no reduced-precision
// input format), and each output is one chain of multiply-adds over k in ascending order,
// whatever M is and whichever tile shape runs: the result does not depend on the batch.  It is the
// matrix product of the 32-bit path and accepts any M, N, K.  The result is written as elements
// or, for logits, as float.
//
// A workgroup of 256 threads takes BM rows of x and BN rows of W; a thread TM x TN outputs, in
// groups of up to four consecutive rows and columns BM / GM and BN / GN apart (the reads of LDS are
// then 16 bytes per lane, neighbours side by side).  The tiles of x and W go through LDS k-major,
// BK columns at a time, in two buffers: the next tile's global loads are on their way while this
// one is multiplied, one barrier per tile.  Four shapes: 128 x 128 where that gives every CU a
// workgroup, else 64 x 64; for the few rows of a decode step, where W is streamed once, 16 x 64 with
// tiles of 64 columns (four rows a thread: its reads of x are one broadcast), or 16 x 16 where W has too
// few rows to give every CU a workgroup of 64 of them.
#include "common.h"

template <typename T>
__device__ __forceinline__ void load4(const T* __restrict__ p, bool whole, int k_left, float v[4]) {
    if (whole) {
        if (sizeof(T) == 4) {
            const float4 f = *reinterpret_cast<const float4*>(p);
            v[0] = f.x; v[1] = f.y; v[2] = f.z; v[3] = f.w;
        } else {
            typedef __attribute__((ext_vector_type(4))) __bf16 b4;
            const b4 f = *reinterpret_cast<const b4*>(p);
#pragma unroll
            for (int e = 0; e < 4; ++e) v[e] = static_cast<float>(f[e]);
        }
    } else {
#pragma unroll
        for (int e = 0; e < 4; ++e) v[e] = e < k_left ? to_float(p[e]) : 0.f;
    }
}

// R rows x BK columns of a matrix, from its row `row0` and column k0, as 4-column pieces: piece p of
// a thread is number tid + 256 p; its row is number / (BK / 4).  Rows and columns past the end are zeros.
template <typename T, int R, int BK>
struct TileLoad {
    static constexpr int PIECES = R * BK / 4 / 256;
    static_assert(R * BK / 4 % 256 == 0 && PIECES >= 1, "a tile is a whole number of pieces per thread");
    float v[PIECES][4];
    __device__ __forceinline__ void fetch(const T* __restrict__ src, int64_t stride, int rows_left, int k_left, bool vec, int tid) {
#pragma unroll
        for (int p = 0; p < PIECES; ++p) {
            const int n = tid + 256 * p, r = n / (BK / 4), kq = (n % (BK / 4)) * 4;
            if (r < rows_left && kq < k_left) {
                load4<T>(src + (int64_t)r * stride + kq, vec && kq + 4 <= k_left, k_left - kq, v[p]);
            } else {
#pragma unroll
                for (int e = 0; e < 4; ++e) v[p][e] = 0.f;
            }
        }
    }
    __device__ __forceinline__ void store(float (*dst)[R + 4], int tid) const {
#pragma unroll
        for (int p = 0; p < PIECES; ++p) {
            const int n = tid + 256 * p, r = n / (BK / 4), kq = (n % (BK / 4)) * 4;
#pragma unroll
            for (int e = 0; e < 4; ++e) dst[kq + e][r] = v[p][e];
        }
    }
};

template <typename T, typename OutT, int BM, int BN, int BK, int TM, int TN>
__global__ void __launch_bounds__(256, 2)
linear_tiled_kernel(const T* __restrict__ x, int64_t x_stride, const T* __restrict__ w, int64_t w_stride,
                    const T* __restrict__ bias, OutT* __restrict__ y, int64_t y_stride, int M, int N, int K,
                    int vec) {
    constexpr int VM = TM >= 4 ? 4 : TM, GM = TM / VM;       // a thread's rows: GM groups of VM consecutive ones
    constexpr int VN = TN >= 4 ? 4 : TN, GN = TN / VN;
    constexpr int TX = BN / TN;                               // threads side by side along n
    static_assert((BM / TM) * TX == 256, "256 threads cover the tile");
    __shared__ float xs[2][BK][BM + 4];
    __shared__ float ws[2][BK][BN + 4];
    const int tid = threadIdx.x;
    const int m0 = blockIdx.y * BM, n0 = blockIdx.x * BN;
    const int ty = tid / TX, tx = tid % TX;
    float acc[TM][TN];
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j) acc[i][j] = 0.f;

    TileLoad<T, BM, BK> lx;
    TileLoad<T, BN, BK> lw;
    const T* xp = x + (int64_t)m0 * x_stride;
    const T* wp = w + (int64_t)n0 * w_stride;
    lx.fetch(xp, x_stride, M - m0, K, vec, tid);
    lw.fetch(wp, w_stride, N - n0, K, vec, tid);
    lx.store(xs[0], tid);
    lw.store(ws[0], tid);
    __syncthreads();
    int buf = 0;
    for (int k0 = 0; k0 < K; k0 += BK) {
        const bool more = k0 + BK < K;
        if (more) {
            lx.fetch(xp + k0 + BK, x_stride, M - m0, K - k0 - BK, vec, tid);
            lw.fetch(wp + k0 + BK, w_stride, N - n0, K - k0 - BK, vec, tid);
        }
#pragma unroll 4
        for (int k = 0; k < BK; ++k) {
            float av[TM], bv[TN];
#pragma unroll
            for (int g = 0; g < GM; ++g)
#pragma unroll
                for (int i = 0; i < VM; ++i) av[g * VM + i] = xs[buf][k][g * (BM / GM) + ty * VM + i];
#pragma unroll
            for (int g = 0; g < GN; ++g)
#pragma unroll
                for (int j = 0; j < VN; ++j) bv[g * VN + j] = ws[buf][k][g * (BN / GN) + tx * VN + j];
#pragma unroll
            for (int i = 0; i < TM; ++i)
#pragma unroll
                for (int j = 0; j < TN; ++j) acc[i][j] += av[i] * bv[j];
        }
        if (more) {
            // the other buffer was last read before the barrier that ended the previous tile
            lx.store(xs[buf ^ 1], tid);
            lw.store(ws[buf ^ 1], tid);
        }
        __syncthreads();
        buf ^= 1;
    }
#pragma unroll
    for (int i = 0; i < TM; ++i) {
        const int m = m0 + (i / VM) * (BM / GM) + ty * VM + i % VM;
        if (m >= M) continue;
#pragma unroll
        for (int j = 0; j < TN; ++j) {
            const int n = n0 + (j / VN) * (BN / GN) + tx * VN + j % VN;
            if (n >= N) continue;
            float v = acc[i][j];
            if (bias) v += to_float(bias[n]);
            y[(int64_t)m * y_stride + n] = from_float<OutT>(v);
        }
    }
}

NVA_EXPORT int NVA_NAME(nva_linear_tiled)(const void* x, int64_t x_stride, const void* w, int64_t w_stride,
                                          const void* bias, void* y, int64_t y_stride, int out_is_f32, int64_t M,
                                          int64_t N, int64_t K, hipStream_t stream) {
    if (M == 0 || N == 0) return 0;
    if (M < 0 || N < 0 || K <= 0 || M > 0x7fffffff || N > 0x7fffffff || K > 0x7fffffff)
        return nva_fail("linear: bad shape M=%lld N=%lld K=%lld", (long long)M, (long long)N, (long long)K);
    const size_t vb = 4 * sizeof(elem_t);
    const int vec = x_stride % 4 == 0 && w_stride % 4 == 0 && nva_aligned(x, vb) && nva_aligned(w, vb);
#define LAUNCH_AS(OUT, BM, BN, BK, TM, TN)                                                                            \
    hipLaunchKernelGGL((linear_tiled_kernel<elem_t, OUT, BM, BN, BK, TM, TN>), grid, dim3(256), 0, stream,            \
                       (const elem_t*)x, x_stride, (const elem_t*)w, w_stride, (const elem_t*)bias, (OUT*)y, y_stride, \
                       (int)M, (int)N, (int)K, vec)
#define LAUNCH(BM, BN, BK, TM, TN)                                                                                    \
    do {                                                                                                              \
        const int64_t grid_m = (M + BM - 1) / BM, grid_n = (N + BN - 1) / BN;                                         \
        if (grid_m > 65535) return nva_fail("linear: M=%lld exceeds %d rows per call", (long long)M, 65535 * BM);     \
        dim3 grid((unsigned)grid_n, (unsigned)grid_m);                                                                \
        if (out_is_f32) LAUNCH_AS(float, BM, BN, BK, TM, TN);                                                         \
        else LAUNCH_AS(elem_t, BM, BN, BK, TM, TN);                                                                   \
    } while (0)
    static int cus = 0;
    if (!cus) {
        int dev = 0;
        if (hipGetDevice(&dev) != hipSuccess || hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || cus <= 0) {
            cus = 0;
            return nva_fail("linear: cannot read the number of CUs");
        }
    }
    if (M <= 16) {
        if (N >= 64 * (int64_t)cus) LAUNCH(16, 64, 64, 4, 1);
        else LAUNCH(16, 16, 64, 1, 1);
    } else if (((M + 127) / 128) * ((N + 127) / 128) >= cus) LAUNCH(128, 128, 16, 8, 8);
    else LAUNCH(64, 64, 16, 4, 4);
#undef LAUNCH
#undef LAUNCH_AS
    return nva_check_launch("linear_tiled");
}

NVA_DEFINE_LAST_ERROR(nva_gemm)
