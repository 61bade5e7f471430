// Row gather: out[t, :] = table[ids[t], :].  Serves the token embedding
// (nanovllm/layers/embed_head.py:38) and the selection of the rows whose logits are wanted
// (embed_head.py:59-60).  An id outside [0, rows) yields a row of zeros and raises the error
// flag, which the host reads after the step; ids that come from the host are checked there.
#include "common.h"

template <typename T>
__global__ void __launch_bounds__(256)
gather_rows_kernel(const T* __restrict__ table, int64_t table_stride, int64_t table_rows,
                   const int32_t* __restrict__ ids, T* __restrict__ out, int64_t out_stride, int width,
                   int vec, int32_t* error_flag) {
    const int64_t t = blockIdx.x;
    const int64_t id = ids[t];
    const bool ok = id >= 0 && id < table_rows;
    if (!ok && threadIdx.x == 0 && error_flag) atomicOr(error_flag, 1);
    const T* src = table + (ok ? id : 0) * table_stride;
    T* dst = out + t * out_stride;
    if (vec) {
        typedef __attribute__((ext_vector_type(4))) uint32_t u32x4;
        const int per = 16 / sizeof(T);
        const u32x4 zero = {0, 0, 0, 0};
        for (int i = threadIdx.x * per; i < width; i += blockDim.x * per)
            *reinterpret_cast<u32x4*>(dst + i) = ok ? *reinterpret_cast<const u32x4*>(src + i) : zero;
    } else {
        for (int i = threadIdx.x; i < width; i += blockDim.x) dst[i] = ok ? src[i] : from_float<T>(0.f);
    }
}

NVA_EXPORT int NVA_NAME(nva_gather_rows)(const void* table, int64_t table_stride, int64_t table_rows,
                                         const int32_t* ids, void* out, int64_t out_stride,
                                         int64_t count, int width, int32_t* error_flag, hipStream_t stream) {
    if (count == 0) return 0;
    if (count < 0 || count > 0x7fffffff || width <= 0 || table_rows <= 0)
        return nva_fail("gather_rows: bad shape count=%lld width=%d rows=%lld", (long long)count, width,
                        (long long)table_rows);
    const int per = 16 / sizeof(elem_t);
    const int vec = width % per == 0 && table_stride % per == 0 && out_stride % per == 0 &&
                    nva_aligned(table, 16) && nva_aligned(out, 16);
    const int threads = width >= 2048 ? 256 : (width >= 512 ? 128 : 64);
    hipLaunchKernelGGL(gather_rows_kernel<elem_t>, dim3((unsigned)count), dim3(threads), 0, stream,
                       (const elem_t*)table, table_stride, table_rows, ids, (elem_t*)out, out_stride, width,
                       vec, error_flag);
    return nva_check_launch("gather_rows");
}

NVA_DEFINE_LAST_ERROR(nva_embed)
