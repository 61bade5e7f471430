// y[M, N] = x[M, K] W[N, K]^T for at most 16 rows of x (bfloat16) and a W of many rows: the gate/up
// product of a decode step of few requests with its SwiGLU gating (nanovllm/layers/linear.py:87-93,
// activation.py:8-11) and the output head (embed_head.py:61).  k is never split over workgroups, so
// no partial sums travel through memory and the gating happens in the product's own epilogue.
//
// One workgroup of eight waves ("a team") takes a run of blocks of 16 rows of W; its waves split k
// between them, each wave owning the same eighth of k in every block.  W goes from HBM straight
// into registers as the A operand of a 16x16x32 MFMA (64 contiguous bytes of each of 16 rows per
// load); a ring of NFW fragments is always in flight: a fragment's register is asked for again,
// for the next block, as soon as its product is issued.  x is the B operand and goes through no
// LDS at all, because a wave's slice of k is its own: either it is kept in registers for all the
// team's blocks (HELD: the slice has at most NFW fragments, K <= 256 * NFW), or it is loaded again
// beside W (any K).  The eight partial tiles of a block meet in LDS; one wave adds them in a fixed
// order and does the epilogue.
#include "common.h"

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(4))) __bf16 bf16x4;
typedef __attribute__((ext_vector_type(4))) float f32x4;

#define TM_WAVES 8
#define TM_ROUND 19          // blocks of W rows whose partial tiles lie in LDS at once (8 KB each; 152 KB of the 160)
#define TM_MAX_ROWS 16

enum { TM_PLAIN = 0, TM_PLAIN_F32 = 1, TM_GATED = 2 };

struct TeamArgs {
    const __bf16* x; int64_t x_stride;
    const __bf16* w; int64_t w_stride; const __bf16* bias;
    void* y; int64_t y_stride; int mode;
    int M, N, K, blocks, blocks_per_team, frags_per_wave;
};

__device__ __forceinline__ bf16x8 tm_zero8() {
    bf16x8 z;
#pragma unroll
    for (int e = 0; e < 8; ++e) z[e] = (__bf16)0.f;
    return z;
}

template <int NFW, bool HELD>
__global__ void __launch_bounds__(TM_WAVES * NVA_WAVE)
linear_team_kernel(const TeamArgs a) {
    __shared__ f32x4 tiles_s[TM_ROUND * TM_WAVES * NVA_WAVE];
    const int wave = threadIdx.x / NVA_WAVE, lane = threadIdx.x % NVA_WAVE;
    const int col = lane & 15, g = lane >> 4;
    const bool gated = a.mode == TM_GATED;
    const int inner = a.N / 2;
    const int block0 = blockIdx.x * a.blocks_per_team;
    const int nblocks = min(a.blocks_per_team, a.blocks - block0);
    // The wave's slice of k, in fragments of 32: [own_begin, own_end).  It is walked in passes of NFW
    // fragments (one pass when HELD); a pass that would run past the slice's end, or a slice shorter
    // than a pass, is moved back so that every load lies inside the row, and the fragments it meets
    // a second time (or that belong to the wave before) get a zero B operand.
    const int frags_total = a.K / 32;
    const int own_begin = min(wave * a.frags_per_wave, frags_total);
    const int own_end = min(frags_total, own_begin + a.frags_per_wave);
    const int passes = HELD ? 1 : (a.frags_per_wave + NFW - 1) / NFW;       // the same for every wave of the team
    const int items = nblocks * passes;
    auto pass_start = [&](int p) { return max(0, min(own_begin + p * NFW, own_end - NFW)); };
    auto frag_valid = [&](int p, int f) {
        const int frag = pass_start(p) + f;
        return frag >= own_begin + p * NFW && frag < own_end;
    };

    // the row of W that this lane reads in block b (of the whole product)
    auto w_row = [&](int b) -> const __bf16* {
        const int row = gated ? min(b * 8 + (col & 7), inner - 1) + (col >= 8 ? inner : 0) : min(b * 16 + col, a.N - 1);
        return a.w + (int64_t)row * a.w_stride + 8 * g;
    };
    const int x_row = min(col, a.M - 1);             // MFMA columns beyond M compute what nobody reads
    const __bf16* xrow = a.x + (int64_t)x_row * a.x_stride + 8 * g;

    bf16x8 wa[NFW], xb[NFW];
    // ---- the ring's first filling: W of the first item
    {
        const __bf16* wr = w_row(block0) + 32 * pass_start(0);
#pragma unroll
        for (int f = 0; f < NFW; ++f) wa[f] = *reinterpret_cast<const bf16x8*>(wr + 32 * f);
    }
    // ---- the B operand
    {
        const __bf16* xr = xrow + 32 * pass_start(0);
#pragma unroll
        for (int f = 0; f < NFW; ++f) {
            const bf16x8 v = *reinterpret_cast<const bf16x8*>(xr + 32 * f);
            xb[f] = frag_valid(0, f) ? v : tm_zero8();
        }
    }

    f32x4 acc[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) acc[i] = f32x4{0.f, 0.f, 0.f, 0.f};

    // what the ring asks for after item `item`: the following pass of this block, or the first of the
    // next block; past the last item every lane reads the first pieces of W again (cached lines, no traffic)
    auto next_w = [&](int item, int& npass, bool& more) -> const __bf16* {
        more = item + 1 < items;
        const int nb = HELD ? item + 1 : (item + 1) / passes;
        npass = HELD ? 0 : (item + 1) % passes;
        return more ? w_row(block0 + nb) + 32 * pass_start(npass) : a.w + 8 * g;
    };
    for (int item = 0; item < items; ++item) {
        const int b = HELD ? item : item / passes, pass = HELD ? 0 : item % passes;
        {
            int npass; bool more;
            const __bf16* wr = next_w(item, npass, more);
            const __bf16* xr = HELD ? nullptr : xrow + (more ? 32 * pass_start(npass) : 0);
#pragma unroll
            for (int f = 0; f < NFW; ++f) {
                acc[f & 3] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wa[f], xb[f], acc[f & 3], 0, 0, 0);
                wa[f] = *reinterpret_cast<const bf16x8*>(wr + 32 * f);
                if (!HELD) {
                    const bf16x8 v = *reinterpret_cast<const bf16x8*>(xr + 32 * f);
                    xb[f] = frag_valid(npass, f) ? v : tm_zero8();
                }
            }
        }
        if (pass != passes - 1) continue;
        // ---- the block is done: this wave's partial tile goes to LDS
        const int slot = b % TM_ROUND;
        f32x4 sum;
#pragma unroll
        for (int i = 0; i < 4; ++i) sum[i] = (acc[0][i] + acc[1][i]) + (acc[2][i] + acc[3][i]);
#pragma unroll
        for (int i = 0; i < 4; ++i) acc[i] = f32x4{0.f, 0.f, 0.f, 0.f};
        tiles_s[(slot * TM_WAVES + wave) * NVA_WAVE + lane] = sum;
        if (slot != TM_ROUND - 1 && b != nblocks - 1) continue;
        // ---- a round of blocks is done: every wave finishes some of them
        __syncthreads();
        const int first = b - slot;
        for (int tl = wave; tl <= slot; tl += TM_WAVES) {
            f32x4 v = tiles_s[(tl * TM_WAVES) * NVA_WAVE + lane];
#pragma unroll
            for (int wv = 1; wv < TM_WAVES; ++wv) {
                const f32x4 u = tiles_s[(tl * TM_WAVES + wv) * NVA_WAVE + lane];
                v[0] += u[0]; v[1] += u[1]; v[2] += u[2]; v[3] += u[3];
            }
            const int blk = block0 + first + tl;
            const int m = col;
            if (gated) {
                // v[i] of lanes g < 2 is the gate of column 8 * blk + 4 * g + i, the same register of
                // lane + 32 its up; both are rounded before the gating, as the projection's output is
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    const float up = round_through<__bf16>(__shfl(v[i], (lane + 32) % NVA_WAVE, NVA_WAVE));
                    const float gate = round_through<__bf16>(v[i]);
                    const int j = blk * 8 + 4 * g + i;
                    if (g < 2 && m < a.M && j < inner)
                        ((__bf16*)a.y)[(int64_t)m * a.y_stride + j] = (__bf16)(gate / (1.f + __expf(-gate)) * up);
                }
                continue;
            }
            const int n = blk * 16 + 4 * g;
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                if (m >= a.M || n + i >= a.N) continue;
                float val = v[i];
                if (a.bias) val += (float)a.bias[n + i];
                if (a.mode == TM_PLAIN_F32) ((float*)a.y)[(int64_t)m * a.y_stride + n + i] = val;
                else ((__bf16*)a.y)[(int64_t)m * a.y_stride + n + i] = (__bf16)val;
            }
        }
        __syncthreads();
    }
}

// y = x W^T (+ bias) for 1..16 rows of x.  mode: 0 elements, 1 float, 2 SwiGLU gating of W = [gate
// rows; up rows] (y [M, N / 2], no bias).  teams: the number of workgroups to aim for (the CUs of the
// GPU); every team takes ceil(blocks / teams) blocks of 16 rows of W.  Returns 1 for shapes this
// kernel does not take: more than 16 rows, K not a multiple of 32.
NVA_EXPORT int nva_linear_team_bf16(const void* x, int64_t x_stride, const void* w, int64_t w_stride, const void* bias,
                                    void* y, int64_t y_stride, int mode, int64_t M, int64_t N, int64_t K, int teams,
                                    hipStream_t stream) {
    if (M == 0 || N == 0) return 0;
    if (M < 0 || M > TM_MAX_ROWS || K <= 0 || K % 32 || N > 0x7fffffff || K > 0x7fffffff) {
        nva_fail("linear_team: needs 1..%d rows and K %% 32 == 0 (M=%lld K=%lld)", TM_MAX_ROWS, (long long)M, (long long)K);
        return 1;
    }
    if (teams <= 0 || !x || !w || !y || x_stride % 8 || w_stride % 8 || !nva_aligned(x, 16) || !nva_aligned(w, 16))
        return nva_fail("linear_team: x and W need 16-byte aligned rows, and an output");
    if (mode < 0 || mode > 2) return nva_fail("linear_team: unknown mode %d", mode);
    if (mode == TM_GATED && (N % 2 || bias)) return nva_fail("linear_team: the gated form needs an even number of weight rows and no bias");
    TeamArgs a;
    a.x = (const __bf16*)x; a.x_stride = x_stride;
    a.w = (const __bf16*)w; a.w_stride = w_stride; a.bias = (const __bf16*)bias;
    a.y = y; a.y_stride = y_stride; a.mode = mode;
    a.M = (int)M; a.N = (int)N; a.K = (int)K;
    a.blocks = mode == TM_GATED ? (int)((N / 2 + 7) / 8) : (int)((N + 15) / 16);
    a.blocks_per_team = (a.blocks + teams - 1) / teams;
    const int frags = (int)(K / 32);
    a.frags_per_wave = (frags + TM_WAVES - 1) / TM_WAVES;
    const unsigned grid = (unsigned)((a.blocks + a.blocks_per_team - 1) / a.blocks_per_team);
#define LAUNCH(NFW, HELD) hipLaunchKernelGGL((linear_team_kernel<NFW, HELD>), dim3(grid), dim3(TM_WAVES * NVA_WAVE), 0, stream, a)
    const int fpw = a.frags_per_wave;
    if (a.blocks_per_team > 1 && fpw <= 24) {
        // x stays in registers for all the team's blocks
        if (fpw <= 1) LAUNCH(1, true);
        else if (fpw <= 2) LAUNCH(2, true);
        else if (fpw <= 4) LAUNCH(4, true);
        else if (fpw <= 8) LAUNCH(8, true);
        else if (fpw <= 12) LAUNCH(12, true);
        else if (fpw <= 16) LAUNCH(16, true);
        else if (fpw <= 20) LAUNCH(20, true);
        else LAUNCH(24, true);
    } else if (fpw <= 1) LAUNCH(1, false);           // x is loaded beside W, again for every block
    else if (fpw <= 2) LAUNCH(2, false);
    else if (fpw <= 4) LAUNCH(4, false);
    else if (fpw <= 8) LAUNCH(8, false);
    else if (fpw <= 12) LAUNCH(12, false);
    else if (fpw <= 16) LAUNCH(16, false);
    else {
        // several passes over the wave's slice: the pass length that walks the fewest fragments twice
        const int w12 = (fpw + 11) / 12 * 12, w16 = (fpw + 15) / 16 * 16, w20 = (fpw + 19) / 20 * 20;
        if (w20 <= w16 && w20 <= w12) LAUNCH(20, false);
        else if (w16 <= w12) LAUNCH(16, false);
        else LAUNCH(12, false);
    }
#undef LAUNCH
    return nva_check_launch("linear_team");
}

NVA_DEFINE_LAST_ERROR(nva_gemm_team)
