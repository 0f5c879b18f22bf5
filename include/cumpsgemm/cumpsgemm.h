/* C ABI of the MI355X (gfx950) mutable-precision SGEMM/CGEMM library.
 *
 * Every entry point below replaces the reference entry point of the same name
 * with CUDA/cuBLAS types swapped for their HIP/hipBLAS counterparts
 * (cublasStatus_t -> hipblasStatus_t, cublasOperation_t -> hipblasOperation_t,
 * cudaStream_t -> hipStream_t, cuComplex -> hipComplex == float2).
 * Matrices are column-major device pointers that are only borrowed for the
 * duration of the (asynchronous) call; alpha/beta are HOST pointers and are
 * read before the call returns; work is enqueued on the handle's stream and
 * never synchronised.  The handle is not thread-safe (as in the reference);
 * its scratch is shared by all its calls, so changing its stream orders the
 * new stream behind the work queued on the old one.
 */
#ifndef CUMPSGEMM_AMD_H
#define CUMPSGEMM_AMD_H
#include "detail/common.h"
#include <hip/hip_complex.h>
#include <hip/hip_runtime_api.h>
#include <hipblas/hipblas.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* reference include/cumpsgemm/cumpsgemm.h:7 (src/handle.cu:7-38).  Binds to the
 * CURRENT HIP device.  HIPBLAS_STATUS_ALLOC_FAILED / INTERNAL_ERROR on failure. */
hipblasStatus_t cuMpSGEMM_create(cuMpSGEMM_handle_t *handle);

/* reference cumpsgemm.h:9 (src/handle.cu:40-46); also frees the scratch the
 * reference leaks. */
hipblasStatus_t cuMpSGEMM_destroy(cuMpSGEMM_handle_t handle);

/* reference cumpsgemm.h:11-12 (src/handle.cu:48-52) */
hipblasStatus_t cuMpSGEMM_set_stream(cuMpSGEMM_handle_t handle,
                                     hipStream_t stream);

/* reference cumpsgemm.h:14-15 (src/cumpsgemm_cublas.cu:163-196) */
const char *cuMpSGEMM_get_compute_mode_string(cuMpSGEMM_compute_mode_t mode);

/* The user-replaceable rule (reference cumpsgemm.h:17-21, default body
 * src/default_cumpsgemm_rule.cu:6-49).  A default implementation ships in
 * libcumpsgemm_rule.so and is also built into libcumpsgemm.so; a user library
 * named libcumpsgemm_rule.so on the loader path that defines this symbol takes
 * precedence.  func_name is the intercepted hipBLAS symbol. */
cuMpSGEMM_compute_mode_t
cuMpSGEMM_get_compute_mode(const char *func_name, hipblasHandle_t hipblas_handle,
                           hipblasOperation_t op_A, hipblasOperation_t op_B,
                           unsigned m, unsigned n, unsigned k);

/* reference cumpsgemm.h:23-30 (src/cumpsgemm.cu:549-563).
 * compute_mode in {FP16TCEC, TF32TCEC, FP16TC, TF32TC, AUTO}; any other value
 * returns HIPBLAS_STATUS_INVALID_VALUE (the reference has undefined behaviour),
 * and so do a null handle, scalar or operand pointer, a leading dimension
 * smaller than the stored rows, and sizes beyond 2^31 - 1 (the reference
 * returns success for everything, src/cumpsgemm.cu:418).  m, n or batch 0 is a
 * successful no-op; k = 0 computes C = beta * C and reads neither A nor B.
 * op C is accepted for real data and means T (reference asserts). */
hipblasStatus_t cuMpSGEMM_sgemm(cuMpSGEMM_handle_t handle,
                                hipblasOperation_t op_A, hipblasOperation_t op_B,
                                uint64_t m, uint64_t n, uint64_t k,
                                const float *alpha, const float *a_dmem_ptr,
                                uint64_t lda, const float *b_dmem_ptr,
                                uint64_t ldb, const float *beta,
                                float *c_dmem_ptr, uint64_t ldc,
                                cuMpSGEMM_compute_mode_t compute_mode);

/* reference cumpsgemm.h:32-39 (src/cumpsgemm.cu:565-576) */
hipblasStatus_t cuMpSGEMM_cgemm(cuMpSGEMM_handle_t handle,
                                hipblasOperation_t op_A, hipblasOperation_t op_B,
                                uint64_t m, uint64_t n, uint64_t k,
                                const hipComplex *alpha,
                                const hipComplex *a_dmem_ptr, uint64_t lda,
                                const hipComplex *b_dmem_ptr, uint64_t ldb,
                                const hipComplex *beta, hipComplex *c_dmem_ptr,
                                uint64_t ldc,
                                cuMpSGEMM_compute_mode_t compute_mode);

/* reference cumpsgemm.h:41-48 (src/cumpsgemm.cu:578-591); strides in elements */
hipblasStatus_t cuMpSGEMM_sgemm_strided_batch(
    cuMpSGEMM_handle_t handle, hipblasOperation_t op_A, hipblasOperation_t op_B,
    uint64_t m, uint64_t n, uint64_t k, const float *alpha,
    const float *a_dmem_ptr, uint64_t lda, uint64_t stridea,
    const float *b_dmem_ptr, uint64_t ldb, uint64_t strideb, const float *beta,
    float *c_dmem_ptr, uint64_t ldc, uint64_t stridec, uint64_t batch_count,
    cuMpSGEMM_compute_mode_t compute_mode);

/* reference cumpsgemm.h:50-57 (src/cumpsgemm.cu:593-604) */
hipblasStatus_t cuMpSGEMM_cgemm_strided_batch(
    cuMpSGEMM_handle_t handle, hipblasOperation_t op_A, hipblasOperation_t op_B,
    uint64_t m, uint64_t n, uint64_t k, const hipComplex *alpha,
    const hipComplex *a_dmem_ptr, uint64_t lda, uint64_t stridea,
    const hipComplex *b_dmem_ptr, uint64_t ldb, uint64_t strideb,
    const hipComplex *beta, hipComplex *c_dmem_ptr, uint64_t ldc,
    uint64_t stridec, uint64_t batch_count,
    cuMpSGEMM_compute_mode_t compute_mode);

#ifdef __cplusplus
}
#endif
#endif
