/*
 * C ABI of the dense floating-point GEMM beside the quantized-linear path (libgpu_blas.so, over hipBLASLt).
 * Entry points keep the reference's names, argument order and return codes (src/ffi.rs, csrc/gemm.cu:46-110).
 * All pointers are device pointers; `stream` is a hipStream_t (0 = the null stream).
 *
 * Return codes: 0 success; -1 / -2 gpu_blas_init could not create the hipBLASLt handle / allocate the workspace;
 * -100 gpu_gemm before gpu_blas_init; -101 no algorithm for the problem (or a bad dtype / K); -1000 - s for a
 * hipblasStatus_t s returned by the launch.
 */
#ifndef GPU_BLAS_API_H
#define GPU_BLAS_API_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* Creates the handle and a workspace of `workspace_bytes` once per process; later calls return 0.
 * Replaces gpu_blas_init, csrc/gemm.cu:46-53. */
int gpu_blas_init(size_t workspace_bytes);

/* Row-major D[M,N] = alpha * A[M,K] . op(B) (+ bias[N]) (+ beta * D).
 *   transb = 1: B is [N,K] (a Linear weight); transb = 0: B is [K,N].  lda, ldb, ldd: elements between rows.
 *   A and B in in_dt, D and bias in out_dt (DT_F32 = 0, DT_F16 = 1, DT_BF16 = 2); fp32 accumulation, fp32 inputs are
 *   multiplied as fp32 (no reduced-precision matrix path).
 * Replaces gpu_gemm, csrc/gemm.cu:55-110. */
int gpu_gemm(const void* A, int64_t lda, const void* B, int64_t ldb, void* D, int64_t ldd, const void* bias, int64_t M,
             int64_t N, int64_t K, int transb, int in_dt, int out_dt, float alpha, float beta, void* stream);

#ifdef __cplusplus
}
#endif
#endif
