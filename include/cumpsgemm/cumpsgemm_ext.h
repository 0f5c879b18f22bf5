/* Plain-C forms of the library's C++ API, for callers that bind through an FFI
 * (ctypes, cgo, JNI ...) and therefore cannot use the C++ templates of
 * cumpsgemm.hpp.  Each function forwards to the C++ function named in its
 * comment; the reference exposes those only as C++ symbols
 * (include/cumpsgemm/cumpsgemm.hpp:37-129, include/cumpsgemm/hijack_control.hpp).
 * Suffix _s = float, _c = hipComplex. */
#ifndef CUMPSGEMM_AMD_EXT_H
#define CUMPSGEMM_AMD_EXT_H
#include "cumpsgemm.h"
#include <stddef.h>

#ifdef __cplusplus
extern "C" {
#endif

/* cumpsgemm::gemm<T> with the used_kernel_module_id out-parameter
 * (reference cumpsgemm.hpp:16-24): index into the tile-config table, +100 when
 * the split-K path ran, ~0u for AUTO. */
hipblasStatus_t cuMpSGEMM_sgemm_ex(cuMpSGEMM_handle_t handle, hipblasOperation_t op_A,
                                   hipblasOperation_t op_B, uint64_t m, uint64_t n, uint64_t k,
                                   const float *alpha, const float *a, uint64_t lda,
                                   const float *b, uint64_t ldb, const float *beta, float *c,
                                   uint64_t ldc, cuMpSGEMM_compute_mode_t mode,
                                   unsigned *used_kernel_module_id);
hipblasStatus_t cuMpSGEMM_cgemm_ex(cuMpSGEMM_handle_t handle, hipblasOperation_t op_A,
                                   hipblasOperation_t op_B, uint64_t m, uint64_t n, uint64_t k,
                                   const hipComplex *alpha, const hipComplex *a, uint64_t lda,
                                   const hipComplex *b, uint64_t ldb, const hipComplex *beta,
                                   hipComplex *c, uint64_t ldc, cuMpSGEMM_compute_mode_t mode,
                                   unsigned *used_kernel_module_id);

/* cuMpSGEMM_sgemm for callers that cannot allocate device memory (code under
 * HIP graph capture, tight serving loops, harnesses that forbid hipMalloc).
 * No counterpart in the reference.  Same arguments and result as
 * cuMpSGEMM_sgemm for compute_mode FP16TCEC or TF32TCEC, but the call always
 * takes the pre-split path and keeps the fp16 / bf16 planes of A and B in a
 * static device array inside the library instead of the handle's grow-on-demand
 * workspace: it calls no hipMalloc / hipFree and does not synchronise.
 * (The variables that steer cuMpSGEMM_sgemm away from that path --
 * CUMPSGEMM_PACKED=0, CUMPSGEMM_FORCE_TILE_CLASS, CUMPSGEMM_FORCE_KSPLIT -- do
 * not apply to this call.)
 * Limits: k >= 128 and
 *   (roundup(m, 256) + roundup(n, 256)) * roundup(k, 32) * 4 bytes (6 for
 *   TF32TCEC) <= cuMpSGEMM_get_static_scratch_size() (64 MiB);
 * anything else returns HIPBLAS_STATUS_INVALID_VALUE with an error line.
 * Every call on a GPU shares that GPU's array: calls that may overlap on one
 * GPU (two streams, two handles, two threads) race and must be ordered by the
 * caller.  Nothing in the array needs clearing between calls: the pre-pass
 * writes every byte the GEMM kernel reads, padding included. */
hipblasStatus_t cuMpSGEMM_sgemm_no_alloc(cuMpSGEMM_handle_t handle, hipblasOperation_t op_A,
                                         hipblasOperation_t op_B, uint64_t m, uint64_t n, uint64_t k,
                                         const float *alpha, const float *a, uint64_t lda,
                                         const float *b, uint64_t ldb, const float *beta, float *c,
                                         uint64_t ldc, cuMpSGEMM_compute_mode_t compute_mode);
size_t cuMpSGEMM_get_static_scratch_size(void);

/* Diagnostic: a library built with -DCUMPSGEMM_WALK_STAMPS=1 makes the
 * tile-walking pre-split kernel record the shader clock around every K-step's
 * barrier and after every write-out into `device_buffer` (2 x 512 64-bit words,
 * zeroed by the caller: per traced workgroup a count, then the stamps with a tag
 * in bits 60-63: 1 = before the barrier, 0 = behind it, 2 = write-out issued);
 * NULL stops it.  The library that is shipped returns
 * HIPBLAS_STATUS_NOT_SUPPORTED.  No counterpart in the reference. */
hipblasStatus_t cuMpSGEMM_set_walk_stamp_buffer(void *device_buffer);

/* Human-readable description of one tile-config table entry; 0 on success. */
int cuMpSGEMM_describe_tile_config(int compute_mode, int is_complex, int op_A, int op_B,
                                   int tile_class, char *buf, size_t buf_len);

/* Bytes of device memory the handle currently holds as workspace for
 * pre-split operands (0 until a call takes that path; grows on demand; freed
 * by cuMpSGEMM_destroy).  No counterpart in the reference, whose kernels need
 * no workspace beyond the fixed scratch of its handle. */
size_t cuMpSGEMM_get_workspace_size(cuMpSGEMM_handle_t handle);
/* Address of that workspace (NULL until it exists).  A buffer that was in use
 * while the handle's stream was being captured into a HIP graph is never
 * freed before cuMpSGEMM_destroy, so replays of the graph stay valid when a
 * later, larger call makes the handle take a new buffer.  The pre-split path
 * is skipped when its planes would exceed CUMPSGEMM_MAX_WORKSPACE_BYTES
 * (environment, decimal bytes, default 16 GiB; 0 = never allocate). */
const void *cuMpSGEMM_get_workspace_pointer(cuMpSGEMM_handle_t handle);

/* The tuning variables of the GEMM path (CUMPSGEMM_PACKED, _PACKED_WALK,
 * _RASTER_GROUP, _FORCE_TILE_CLASS, _FORCE_KSPLIT, _NO_PERSISTENT,
 * _NO_COLUMN_SPLIT, _CUT_PERCENT, _NO_KSLICE_GROUPS, _NO_EDGE16_TWIN, _NO_FUSED_SCALING,
 * _PERSISTENT_MAX_STEPS, _MAX_WORKSPACE_BYTES) are read from the environment
 * once per process; this reads them again and publishes the new set as one
 * immutable snapshot.  Safe to call while other threads run GEMMs: a call in
 * flight goes on with the values it has already looked up and may take later
 * ones from the new set.  For tests and experiments.  The reference has no
 * such variables. */
void cuMpSGEMM_reload_tuning_env(void);

/* The whole mode pipeline of an intercepted call, callable directly:
 *   FP16TCEC_SCALING: exp_max(A), exp_max(B) -> scale A, B in place -> FP16TCEC
 *                     GEMM -> scale C -> (optionally) undo the scaling of A, B
 *   AUTO:             exp_stats(A), exp_stats(B) -> device-side decision ->
 *                     scale -> FP16TCEC or bf16x3 GEMM -> scale C -> undo
 *   other TCEC modes: plain GEMM.
 * No host synchronisation.  A and B are written (scaled, then restored when
 * restore_AB != 0) exactly as the reference's interposer does
 * (src/cumpsgemm_cublas.cu:446-577 and :836-960).  batch_count == 1 with zero
 * strides is the non-batched form. */
hipblasStatus_t cuMpSGEMM_sgemm_pipeline(cuMpSGEMM_handle_t handle, hipblasOperation_t op_A,
                                         hipblasOperation_t op_B, uint64_t m, uint64_t n,
                                         uint64_t k, const float *alpha, float *a, uint64_t lda,
                                         uint64_t stridea, float *b, uint64_t ldb,
                                         uint64_t strideb, const float *beta, float *c,
                                         uint64_t ldc, uint64_t stridec, uint64_t batch_count,
                                         cuMpSGEMM_compute_mode_t mode, int restore_AB,
                                         unsigned *ids_out /* [3]: A slot, B slot, flag slot */);
hipblasStatus_t cuMpSGEMM_cgemm_pipeline(cuMpSGEMM_handle_t handle, hipblasOperation_t op_A,
                                         hipblasOperation_t op_B, uint64_t m, uint64_t n,
                                         uint64_t k, const hipComplex *alpha, hipComplex *a,
                                         uint64_t lda, uint64_t stridea, hipComplex *b,
                                         uint64_t ldb, uint64_t strideb, const hipComplex *beta,
                                         hipComplex *c, uint64_t ldc, uint64_t stridec,
                                         uint64_t batch_count, cuMpSGEMM_compute_mode_t mode,
                                         int restore_AB, unsigned *ids_out);

/* HBM-streaming (M,2,2) and (2,N,2) GEMMs, the gate-application shapes the
 * reference hands to the external cuGEMM-Mx2x2 kernels
 * (src/cumpsgemm_cublas.cu:269-338, :647-722).  Plain FP32 arithmetic. */
hipblasStatus_t cuMpSGEMM_sgemm_Mx2x2(cuMpSGEMM_handle_t handle, hipblasOperation_t op_A,
                                      hipblasOperation_t op_B, uint64_t m, const float *alpha,
                                      const float *a, uint64_t lda, uint64_t stridea,
                                      const float *b, uint64_t ldb, uint64_t strideb,
                                      const float *beta, float *c, uint64_t ldc, uint64_t stridec,
                                      uint64_t batch_count);
hipblasStatus_t cuMpSGEMM_cgemm_Mx2x2(cuMpSGEMM_handle_t handle, hipblasOperation_t op_A,
                                      hipblasOperation_t op_B, uint64_t m, const hipComplex *alpha,
                                      const hipComplex *a, uint64_t lda, uint64_t stridea,
                                      const hipComplex *b, uint64_t ldb, uint64_t strideb,
                                      const hipComplex *beta, hipComplex *c, uint64_t ldc,
                                      uint64_t stridec, uint64_t batch_count);
hipblasStatus_t cuMpSGEMM_sgemm_2xNx2(cuMpSGEMM_handle_t handle, hipblasOperation_t op_A,
                                      hipblasOperation_t op_B, uint64_t n, const float *alpha,
                                      const float *a, uint64_t lda, uint64_t stridea,
                                      const float *b, uint64_t ldb, uint64_t strideb,
                                      const float *beta, float *c, uint64_t ldc, uint64_t stridec,
                                      uint64_t batch_count);
hipblasStatus_t cuMpSGEMM_cgemm_2xNx2(cuMpSGEMM_handle_t handle, hipblasOperation_t op_A,
                                      hipblasOperation_t op_B, uint64_t n, const hipComplex *alpha,
                                      const hipComplex *a, uint64_t lda, uint64_t stridea,
                                      const hipComplex *b, uint64_t ldb, uint64_t strideb,
                                      const hipComplex *beta, hipComplex *c, uint64_t ldc,
                                      uint64_t stridec, uint64_t batch_count);

/* cumpsgemm::exp_stats_ext<T> / exp_max_ext<T> (reference cumpsgemm.hpp:37-46) */
unsigned cuMpSGEMM_exp_stats_ext_s(cuMpSGEMM_handle_t h, unsigned m, unsigned n, const float *ptr,
                                   unsigned ld, unsigned batch, unsigned stride);
unsigned cuMpSGEMM_exp_stats_ext_c(cuMpSGEMM_handle_t h, unsigned m, unsigned n,
                                   const hipComplex *ptr, unsigned ld, unsigned batch,
                                   unsigned stride);
unsigned cuMpSGEMM_exp_max_ext_s(cuMpSGEMM_handle_t h, unsigned m, unsigned n, const float *ptr,
                                 unsigned ld, unsigned batch, unsigned stride);
unsigned cuMpSGEMM_exp_max_ext_c(cuMpSGEMM_handle_t h, unsigned m, unsigned n,
                                 const hipComplex *ptr, unsigned ld, unsigned batch,
                                 unsigned stride);
/* The statistics of the two operands of one GEMM with ONE launch per pass
 * (the workgroups are shared out between A and B in proportion to their
 * sizes) -- what the FP16TCEC_SCALING and AUTO pipelines use, a kernel
 * boundary being worth several microseconds.  Same results and slot numbering
 * as the _ext call for A followed by the one for B; ids_out[0 / 1] receive the
 * slots of A / B.  exp_stats: flag_id >= 0 also writes that launch flag from
 * the two decisions (cumpsgemm::set_dynamic_launch_buffer_by_exp_stats,
 * reference src/dynamic_scaling.cu:364-397), -1 leaves the flags alone.  No
 * counterpart in the reference, which scans A and B with separate launches
 * (src/cumpsgemm_cublas.cu:455-462, :527-536). */
void cuMpSGEMM_exp_stats_pair_s(cuMpSGEMM_handle_t h, unsigned m_a, unsigned n_a, const float *a,
                                unsigned lda, unsigned m_b, unsigned n_b, const float *b,
                                unsigned ldb, int flag_id, unsigned *ids_out /* [2] */);
void cuMpSGEMM_exp_max_pair_s(cuMpSGEMM_handle_t h, unsigned m_a, unsigned n_a, const float *a,
                              unsigned lda, unsigned m_b, unsigned n_b, const float *b,
                              unsigned ldb, unsigned *ids_out /* [2] */);
/* cumpsgemm::get_exp_stats (cumpsgemm.hpp:48-49): synchronises the stream */
void cuMpSGEMM_get_exp_stats(cuMpSGEMM_handle_t h, unsigned id, uint64_t *underflow,
                             uint64_t *total);
/* cumpsgemm::get_max_exp (cumpsgemm.hpp:64) */
float cuMpSGEMM_get_max_exp(cuMpSGEMM_handle_t h, unsigned id);
/* cumpsgemm::get_exp_stats_compute_mode_level (cumpsgemm.hpp:66-68) */
int cuMpSGEMM_get_exp_stats_compute_mode_level(cuMpSGEMM_handle_t h, unsigned id);
/* cumpsgemm::set_exp_stats_params (cumpsgemm.hpp:55-58) */
void cuMpSGEMM_set_exp_stats_params(cuMpSGEMM_handle_t h, float ignore_threshold,
                                    float underflow_threshold, float tolerance);
unsigned cuMpSGEMM_get_current_exp_stats_buffer_id(cuMpSGEMM_handle_t h);
void cuMpSGEMM_reset_exp_stats_buffer_id(cuMpSGEMM_handle_t h);
void cuMpSGEMM_enable_exp_stats(cuMpSGEMM_handle_t h);
void cuMpSGEMM_disable_exp_stats(cuMpSGEMM_handle_t h);
/* wall-clock profiling of the stats / scaling / GEMM launches (cumpsgemm.hpp:116-129).
 * get_..._entry is debug::get_exp_stats_profiling_result for one label
 * ("exp_stats_1", "exp_stats_2", "exp_max", "scaling_AB", "scaling_C",
 * "reset_scaling_AB", a GEMM label): returns 1 and fills seconds / count when
 * the label has been recorded, else 0. */
void cuMpSGEMM_enable_exp_stats_profiling(cuMpSGEMM_handle_t h);
void cuMpSGEMM_disable_exp_stats_profiling(cuMpSGEMM_handle_t h);
void cuMpSGEMM_reset_exp_stats_profiling(cuMpSGEMM_handle_t h);
void cuMpSGEMM_print_exp_stats_profiling(cuMpSGEMM_handle_t h, unsigned csv);
int cuMpSGEMM_get_exp_stats_profiling_entry(cuMpSGEMM_handle_t h, const char *name,
                                            double *time_sum, uint64_t *n);

/* cumpsgemm::scale_A/B/C, reset_scale_A/B (cumpsgemm.hpp:71-100) */
void cuMpSGEMM_scale_A_s(cuMpSGEMM_handle_t h, unsigned stats_id, unsigned flag_id, unsigned m,
                         unsigned n, float *ptr, unsigned ld, unsigned batch, unsigned stride);
void cuMpSGEMM_scale_A_c(cuMpSGEMM_handle_t h, unsigned stats_id, unsigned flag_id, unsigned m,
                         unsigned n, hipComplex *ptr, unsigned ld, unsigned batch, unsigned stride);
void cuMpSGEMM_scale_B_s(cuMpSGEMM_handle_t h, unsigned stats_id, unsigned flag_id, unsigned m,
                         unsigned n, float *ptr, unsigned ld, unsigned batch, unsigned stride);
void cuMpSGEMM_scale_B_c(cuMpSGEMM_handle_t h, unsigned stats_id, unsigned flag_id, unsigned m,
                         unsigned n, hipComplex *ptr, unsigned ld, unsigned batch, unsigned stride);
void cuMpSGEMM_scale_C_s(cuMpSGEMM_handle_t h, unsigned stats_a, unsigned stats_b, unsigned flag_id,
                         unsigned m, unsigned n, float *ptr, unsigned ld, unsigned batch,
                         unsigned stride);
void cuMpSGEMM_scale_C_c(cuMpSGEMM_handle_t h, unsigned stats_a, unsigned stats_b, unsigned flag_id,
                         unsigned m, unsigned n, hipComplex *ptr, unsigned ld, unsigned batch,
                         unsigned stride);
void cuMpSGEMM_reset_scale_A_s(cuMpSGEMM_handle_t h, unsigned stats_id, unsigned flag_id,
                               unsigned m, unsigned n, float *ptr, unsigned ld, unsigned batch,
                               unsigned stride);
void cuMpSGEMM_reset_scale_A_c(cuMpSGEMM_handle_t h, unsigned stats_id, unsigned flag_id,
                               unsigned m, unsigned n, hipComplex *ptr, unsigned ld,
                               unsigned batch, unsigned stride);
void cuMpSGEMM_reset_scale_B_s(cuMpSGEMM_handle_t h, unsigned stats_id, unsigned flag_id,
                               unsigned m, unsigned n, float *ptr, unsigned ld, unsigned batch,
                               unsigned stride);
void cuMpSGEMM_reset_scale_B_c(cuMpSGEMM_handle_t h, unsigned stats_id, unsigned flag_id,
                               unsigned m, unsigned n, hipComplex *ptr, unsigned ld,
                               unsigned batch, unsigned stride);

/* launch-flag ring (cumpsgemm.hpp:104-114).  The raw flag packs the GEMM mode
 * in bits 0-4, scale-B in bit 5, scale-A in bit 6. */
unsigned cuMpSGEMM_get_current_dynamic_launch_buffer_id(cuMpSGEMM_handle_t h);
unsigned cuMpSGEMM_get_next_dynamic_launch_buffer_id(cuMpSGEMM_handle_t h);
int cuMpSGEMM_get_dynamic_launch_flag(cuMpSGEMM_handle_t h, unsigned id);
void cuMpSGEMM_set_dynamic_launch_buffer_by_exp_stats(cuMpSGEMM_handle_t h, unsigned flag_id,
                                                      unsigned a_id, unsigned b_id);
void cuMpSGEMM_set_dynamic_launch_flag_buffer_id(cuMpSGEMM_handle_t h, unsigned id);
void cuMpSGEMM_unset_dynamic_launch_flag_buffer_id(cuMpSGEMM_handle_t h);

/* cumpsgemm::hijack_control::* (reference hijack_control.hpp:9-32) */
cuMpSGEMM_handle_t cuMpSGEMM_hijack_get_internal_global_handle(void);
int cuMpSGEMM_hijack_set_compute_mode(int mode); /* -1 for FP32_SIMT */
void cuMpSGEMM_hijack_unset_compute_mode(void);
void cuMpSGEMM_hijack_enable_custom_gemm_Mx2x2(void);
void cuMpSGEMM_hijack_disable_custom_gemm_Mx2x2(void);
void cuMpSGEMM_hijack_set_restore_AB(int enable);
size_t cuMpSGEMM_hijack_get_last_called_function_str(char *buf, size_t buf_len);
void cuMpSGEMM_hijack_clear_last_called_function_str(void);
int cuMpSGEMM_hijack_is_library_loaded(void);
void cuMpSGEMM_hijack_set_last_called_function_str(const char *str);
void cuMpSGEMM_hijack_reset_exp_stats_buffer_id(void);
/* thresholds of the AUTO decision on the interposer's handle (creates it) */
void cuMpSGEMM_hijack_set_exp_stats_params(float ignore_threshold, float underflow_threshold,
                                           float underflow_tolerance_rate);
/* hijack_control::set_control_function with a plain function pointer:
 * (op_A, op_B, m, n, k) -> cuMpSGEMM_compute_mode_t value; NULL removes it
 * (reference hijack_control.hpp:28-31, python/src/main.cpp:81-88). */
typedef int (*cuMpSGEMM_control_function_t)(int op_A, int op_B, unsigned m, unsigned n, unsigned k);
void cuMpSGEMM_hijack_set_control_function(cuMpSGEMM_control_function_t fn);
/* The mode the interposer would choose for a call (static mode, control
 * function, rule library, built-in rule -- in that order). */
int cuMpSGEMM_hijack_query_compute_mode(const char *func_name, int op_A, int op_B, unsigned m,
                                        unsigned n, unsigned k);

#ifdef __cplusplus
}
#endif
#endif
