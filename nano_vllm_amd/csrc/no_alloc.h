// An entry point that allocates nothing.
//
// It has no counterpart in the reference (nanovllm/ holds Python only and lets torch allocate
// wherever it likes).  It is for callers that cannot allocate device memory: code under HIP graph
// capture, tight serving loops, harnesses that forbid hipMalloc.
//
// nva_linear_skinny_static_bf16 is nva_linear_skinny_bf16 (the weight-streaming product
// y[M, N] = x[M, K] W[N, K]^T for up to 64 rows of x, gemm_skinny.hip) without the workspace
// argument: the float partial sums of a product whose k range is split, or that adds a bias or
// gates, go to an array that the library holds in device memory from load to exit instead of to
// memory the caller brings:
//
//     NVA_STATIC_SCRATCH_FLOATS floats = 16 MiB on every GPU the library runs on.
//
// The caller still passes inputs and outputs.  A call that needs more than that
// (splits_used * M * N floats) is refused with a message that names the limit; so is anything
// nva_linear_skinny_bf16 refuses.  No hipMalloc, hipFree or allocating library routine is called.
// Every call on a GPU shares that GPU's array: the kernels overwrite every partial sum they
// later read, so nothing has to be cleared between calls, but two calls that overlap on one GPU
// (two streams, two threads) race on it and must be ordered by the caller.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#define NVA_STATIC_SCRATCH_FLOATS (4 << 20)

extern "C" int nva_linear_skinny_static_bf16(const void* x, int64_t x_stride, const void* w, int64_t w_stride,
                                             const void* bias, void* y, int64_t y_stride, int y_is_f32, int swiglu,
                                             int splits, int waves_per_tile, int64_t M, int64_t N, int64_t K,
                                             int* splits_used, hipStream_t stream);

// Floats of the static array that a call with these arguments would use (0: it writes y directly).
extern "C" int64_t nva_linear_skinny_static_need_bf16(const void* bias, int swiglu, int splits, int64_t M, int64_t N,
                                                      int64_t K);
