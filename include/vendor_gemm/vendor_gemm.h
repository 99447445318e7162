/*
 * libvendor_gemm.so -- the vendor libraries behind one GEMM call, for context numbers.
 *
 * Counterpart of the reference's rocblas_wrapper library (reference
 * rocblas_wrapper/include/rocblas_wrapper/gemm.hpp:33-107, rocblas_wrapper/src/gemm.cpp:29-123:
 * init_rocblas / cleanup_rocblas / gemm<TRANSPOSE_A, TRANSPOSE_B>, fp16 only, C always
 * column-major), widened to what the GEMM library itself covers so that every number it
 * reports can have the vendor's beside it: rocBLAS (rocblas_gemm_ex and
 * rocblas_gemm_strided_batched_ex) and hipBLASLt (hipblasLtMatmul with the first algorithm
 * its heuristic returns), the four type pairs, all eight row/column-major layouts of A, B
 * and C, strided batches.  Same argument conventions as rocm_wmma_gemm_c.h: C = A * B, dense
 * packed operands, layout 0 = row-major, 1 = column-major, `stream` is the ADDRESS of a
 * hipStream_t, fp32 accumulation (compute type f32).  Not part of the GEMM library: nothing
 * in librocm_wmma_gemm_gfx950.so links or loads it.
 */
#ifndef VENDOR_GEMM_H
#define VENDOR_GEMM_H

#include <stddef.h>

#ifdef __cplusplus
extern "C" {
#endif

#define VENDOR_GEMM_ROCBLAS 0
#define VENDOR_GEMM_HIPBLASLT 1

/* Creates the rocBLAS and hipBLASLt handles (reference init_rocblas, src/gemm.cpp:29-38).
 * Returns 0, or -1 if a handle could not be created.  Calling it again is harmless. */
int vendor_gemm_init(void);

/* Destroys the handles and frees the hipBLASLt workspace (reference cleanup_rocblas,
 * src/gemm.cpp:40-47). */
void vendor_gemm_cleanup(void);

/* C = A * B through the named backend.  type_idx as in rocm_wmma_gemm_c.h
 * (0 f16->f16, 1 f16->f32, 2 bf16->bf16, 3 bf16->f32).  Returns 0 on success, -1 before
 * vendor_gemm_init, -2 for a bad argument, -3 if the library rejected the problem (its
 * status code is printed to stderr), -4 if hipBLASLt has no algorithm for it. */
int vendor_gemm(int backend, int type_idx, void* C, void* A, void* B, size_t M, size_t N, size_t K,
                size_t batch_count, int layout_c, int layout_a, int layout_b, void* stream);

#ifdef __cplusplus
}
#endif

#endif /* VENDOR_GEMM_H */
