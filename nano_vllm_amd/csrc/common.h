// Shared by every kernel source of the engine (gfx950, wave64).
//
// Each source is compiled once per element type: -DNVA_BF16 gives entry points that end in
// _bf16 and work on bfloat16 storage, -DNVA_F32 gives _f32 entry points on float storage.
// Arithmetic is float in both; only loads and stores differ.  Entry points are extern "C",
// take raw device pointers, sizes and a hipStream_t, launch asynchronously on that stream and
// return 0, or a negative code after leaving a message for nva_last_error().
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdio.h>
#include <stdarg.h>

#if defined(NVA_BF16)
typedef __bf16 elem_t;
#define NVA_NAME(base) base##_bf16
#define NVA_ELEM_NAME "bfloat16"
#elif defined(NVA_F32)
typedef float elem_t;
#define NVA_NAME(base) base##_f32
#define NVA_ELEM_NAME "float32"
#else
#define NVA_NAME(base) base
#define NVA_ELEM_NAME "none"
#endif

#define NVA_WAVE 64
// gfx950: the compute units are spread over this many dies (XCDs), each with an L2 of its own;
// workgroups are handed to the dies in turn, in the order of their index.
#define NVA_XCDS 8

// ---------------------------------------------------------------------------- errors
static thread_local char nva_error_text[512];

static inline int nva_fail(const char* fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(nva_error_text, sizeof(nva_error_text), fmt, ap);
    va_end(ap);
    return -1;
}

static inline int nva_check_launch(const char* what) {
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return nva_fail("%s: launch failed: %s", what, hipGetErrorString(e));
    return 0;
}

#define NVA_EXPORT extern "C" __attribute__((visibility("default")))

// Every library exports its own copy under a name of its own; the loader asks the library
// whose call failed.
#define NVA_DEFINE_LAST_ERROR(lib) \
    NVA_EXPORT const char* lib##_last_error() { return nva_error_text; }

// ---------------------------------------------------------------------------- element access
__device__ __forceinline__ float to_float(float x) { return x; }
__device__ __forceinline__ float to_float(__bf16 x) { return static_cast<float>(x); }

template <typename T> __device__ __forceinline__ T from_float(float x);
template <> __device__ __forceinline__ float from_float<float>(float x) { return x; }
template <> __device__ __forceinline__ __bf16 from_float<__bf16>(float x) { return static_cast<__bf16>(x); }

// Round a float through the element type: what storing and loading it again would give.
template <typename T> __device__ __forceinline__ float round_through(float x) {
    return to_float(from_float<T>(x));
}

// ---------------------------------------------------------------------------- reductions
__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
    for (int off = NVA_WAVE / 2; off > 0; off >>= 1) v += __shfl_xor(v, off, NVA_WAVE);
    return v;
}

__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
    for (int off = NVA_WAVE / 2; off > 0; off >>= 1) v = fmaxf(v, __shfl_xor(v, off, NVA_WAVE));
    return v;
}

// Sum over a whole block of up to 1024 threads; every thread gets the result.
// `scratch` must hold at least 16 floats of shared memory and may be reused after the call.
__device__ __forceinline__ float block_sum(float v, float* scratch) {
    v = wave_sum(v);
    const int wave = threadIdx.x / NVA_WAVE, lane = threadIdx.x % NVA_WAVE;
    const int nwaves = (blockDim.x + NVA_WAVE - 1) / NVA_WAVE;
    __syncthreads();
    if (lane == 0) scratch[wave] = v;
    __syncthreads();
    float total = 0.f;
    for (int i = 0; i < nwaves; ++i) total += scratch[i];
    return total;
}

// ---------------------------------------------------------------------------- vector access
// Eight consecutive elements at a 16-byte aligned address (32-byte for float).
__device__ __forceinline__ void load8(const __bf16* p, float* out) {
    typedef __attribute__((ext_vector_type(8))) __bf16 v8;
    v8 v = *reinterpret_cast<const v8*>(p);
#pragma unroll
    for (int i = 0; i < 8; ++i) out[i] = static_cast<float>(v[i]);
}
__device__ __forceinline__ void load8(const float* p, float* out) {
    float4 a = reinterpret_cast<const float4*>(p)[0], b = reinterpret_cast<const float4*>(p)[1];
    out[0] = a.x; out[1] = a.y; out[2] = a.z; out[3] = a.w;
    out[4] = b.x; out[5] = b.y; out[6] = b.z; out[7] = b.w;
}
__device__ __forceinline__ void store8(__bf16* p, const float* in) {
    typedef __attribute__((ext_vector_type(8))) __bf16 v8;
    v8 v;
#pragma unroll
    for (int i = 0; i < 8; ++i) v[i] = static_cast<__bf16>(in[i]);
    *reinterpret_cast<v8*>(p) = v;
}
__device__ __forceinline__ void store8(float* p, const float* in) {
    reinterpret_cast<float4*>(p)[0] = make_float4(in[0], in[1], in[2], in[3]);
    reinterpret_cast<float4*>(p)[1] = make_float4(in[4], in[5], in[6], in[7]);
}

static inline bool nva_aligned(const void* p, size_t bytes) {
    return (reinterpret_cast<uintptr_t>(p) % bytes) == 0;
}

// exp for softmax and SiLU: the accurate routine in the float build, the fast one otherwise.
__device__ __forceinline__ float nva_exp(float x) {
#if defined(NVA_F32)
    return expf(x);
#else
    return __expf(x);
#endif
}

// ---------------------------------------------------------------------------- split products
// A product whose k range was split over workgroups leaves float partial sums
// [splits][rows][width] (gemm_skinny.hip).  Kernels that consume such a product add the partials
// in the order of the splits, add the optional bias and round to the element type: what the
// product's own finishing pass would have stored.
struct PartialInput {
    const float* sums;        // null: x is read as elements
    int splits;
    int64_t split_stride;     // rows * width
    const void* bias;         // elements, or null
};

template <typename T>
__device__ __forceinline__ float partial_value(const PartialInput& p, int64_t row, int width, int i) {
    float v = 0.f;
    const float* q = p.sums + row * width + i;
#pragma unroll 8
    for (int s = 0; s < p.splits; ++s) v += q[s * p.split_stride];      // independent loads, one sum in split order
    if (p.bias) v += to_float(static_cast<const T*>(p.bias)[i]);
    return round_through<T>(v);
}

template <typename T>
__device__ __forceinline__ void partial_value8(const PartialInput& p, int64_t row, int width, int i, float* out) {
    const float* q = p.sums + row * width + i;
#pragma unroll
    for (int e = 0; e < 8; ++e) out[e] = 0.f;
#pragma unroll 8
    for (int s = 0; s < p.splits; ++s) {
        float v[8];
        load8(q + s * p.split_stride, v);
#pragma unroll
        for (int e = 0; e < 8; ++e) out[e] += v[e];
    }
    if (p.bias) {
        float b[8];
        load8(static_cast<const T*>(p.bias) + i, b);
#pragma unroll
        for (int e = 0; e < 8; ++e) out[e] += b[e];
    }
#pragma unroll
    for (int e = 0; e < 8; ++e) out[e] = round_through<T>(out[e]);
}


// Exchanges between the rows of 16 lanes of a wave by one vector instruction each (a shuffle goes
// through LDS and waits for it).  nva_lane_halves: what the lanes 0..31 and the lanes 32..63 hold of
// x, each in all lanes of its own lane number modulo 32.  nva_lane_rows: of each pair of rows (0 and
// 1, 2 and 3) what the even and what the odd row holds, in both rows of the pair.
__device__ __forceinline__ void nva_lane_halves(float x, float& lower, float& upper) {
    unsigned a = __builtin_bit_cast(unsigned, x), b = a;
    asm volatile("s_nop 1\n\tv_permlane32_swap_b32 %0, %1\n\ts_nop 1" : "+v"(a), "+v"(b));
    lower = __builtin_bit_cast(float, a);
    upper = __builtin_bit_cast(float, b);
}
__device__ __forceinline__ void nva_lane_rows(float x, float& even, float& odd) {
    unsigned a = __builtin_bit_cast(unsigned, x), b = a;
    asm volatile("s_nop 1\n\tv_permlane16_swap_b32 %0, %1\n\ts_nop 1" : "+v"(a), "+v"(b));
    even = __builtin_bit_cast(float, a);
    odd = __builtin_bit_cast(float, b);
}
// the maximum and the sum over the four lanes l, l + 16, l + 32, l + 48, in all four
__device__ __forceinline__ float nva_max_over_rows(float x) {
    float a, b;
    nva_lane_rows(x, a, b);
    nva_lane_halves(fmaxf(a, b), a, b);
    return fmaxf(a, b);
}
__device__ __forceinline__ float nva_sum_over_rows(float x) {
    float a, b;
    nva_lane_rows(x, a, b);
    nva_lane_halves(a + b, a, b);
    return a + b;
}

// ---------------------------------------------------------------------------- cache layout
// K [pages, kv_heads, page_size, head_dim].
// V [pages, kv_heads, page_size / vt, head_dim, vt]: transposed (the keys of one channel are
// contiguous) in tiles of vt keys, vt = 32 when the page size is a multiple of 32, else the page
// size.  A tile of 32 keys is what the decode attention reads per step: 8 KiB contiguous at
// head_dim 128, instead of half of every 128-byte line of a whole page.
__host__ __device__ __forceinline__ int nva_v_tile(int page_size) { return page_size % 32 == 0 ? 32 : page_size; }

// Offset of (key `kip` of the page, channel d) within the [head_dim * page_size] block of one (page, kv head).
__device__ __forceinline__ int64_t nva_v_offset(int kip, int d, int head_dim, int vt) {
    return ((int64_t)(kip / vt) * head_dim + d) * vt + kip % vt;
}
