/*
 * The reference's C++ launcher names over the C ABI of sgemm.h, for harness mains that call them
 * directly (projects/skinny_gemm/test.cu:82, bench.cu:54-59; test.cu:69-70 of the async_gemm projects;
 * tiled_sum_reduce/test.cu:48-49): include this instead of the reference's
 * "./skinny_gemm_caller.cu" / "./src.cu" and link libsgemm.so.  Same parameter lists; fp8 is a byte
 * (__hip_fp8_storage_t, core.cu:10); D is bf16 (uint16_t bits) and is overwritten, see sgemm.h.
 */
#ifndef SGEMM_COMPAT_HPP
#define SGEMM_COMPAT_HPP

#include <hip/hip_runtime.h>

#include "sgemm.h"

typedef unsigned char fp8;

/* skinny_gemm/skinny_gemm_caller.cu:343-346 */
inline int skinny_gemm_fastpath(const fp8* A, const fp8* B, void* D_bf16, const float* scale_tensor, int m, int n, int k) {
    return sg_skinny_gemm_fastpath(A, B, D_bf16, scale_tensor, m, n, k);
}

/* skinny_gemm/skinny_gemm_caller.cu:20-43 */
inline int skinny_gemm(const fp8* A, const fp8* B, void* D_bf16, const float* scale_tensor, int m, int n, int k,
                       int b_stride, int split_k, int A_producers, int B_producers, int consumers, int b_lanes,
                       int qsize, int op_m, int ops, hipStream_t stream) {
    return sg_skinny_gemm(A, B, D_bf16, scale_tensor, m, n, k, b_stride, split_k, A_producers, B_producers, consumers,
                          b_lanes, qsize, op_m, ops, static_cast<void*>(stream));
}

/* async_gemm_sparse/sparse_k.cu:45-53 and its siblings: D = A * B^T, no scale, default stream.  The reference
 * prints and exits on a bad shape; these return the library's code instead (0 = success). */
template <class out_dtype>
int async_gemm(const fp8* A, const fp8* B, out_dtype* D, int m, int n, int k);
template <>
inline int async_gemm<float>(const fp8* A, const fp8* B, float* D, int m, int n, int k) {
    return sg_async_gemm_f32(A, B, D, m, n, k);
}
template <>
inline int async_gemm<unsigned short>(const fp8* A, const fp8* B, unsigned short* D_bf16, int m, int n, int k) {
    return sg_async_gemm_bf16(A, B, D_bf16, m, n, k);
}

/* tiled_sum_reduce/src.cu:52-59; define SGEMM_COMPAT_TSR_ASYNC before including this header to get the launcher of
 * tiled_sum_reduce_async/src.cu:179-200 (same name, same arguments, batches staged through a queue in LDS) instead */
inline int tiled_sum_reduce(const float* A, const float* B, float* D, int b, int m, int n) {
#ifdef SGEMM_COMPAT_TSR_ASYNC
    return sg_tiled_sum_reduce_async(A, B, D, b, m, n, nullptr);
#else
    return sg_tiled_sum_reduce(A, B, D, b, m, n, nullptr);
#endif
}

#endif /* SGEMM_COMPAT_HPP */
