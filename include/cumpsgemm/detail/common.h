/* Opaque handle and compute-mode codes of the cuMpSGEMM API.
 * Replaces: reference include/cumpsgemm/detail/common.h:3-20 (same names, same
 * numeric values, so code compiled against either agrees on the ABI). */
#ifndef CUMPSGEMM_AMD_DETAIL_COMMON_H
#define CUMPSGEMM_AMD_DETAIL_COMMON_H

struct cuMpSGEMM_handle;
typedef struct cuMpSGEMM_handle *cuMpSGEMM_handle_t;

/* On CDNA4 there is no TF32 matrix instruction: the two TF32 modes are served
 * by bf16 splits (TF32TCEC -> bf16x3, 6 products; TF32TC -> bf16x2, 3
 * products), both with the full FP32 exponent range like TF32.
 * The CUBLAS* modes forward to the real hipBLAS. */
enum cuMpSGEMM_compute_mode_t {
  CUMPSGEMM_CUBLAS = 0,            /* forward to hipBLAS, untouched          */
  CUMPSGEMM_FP16TCEC = 1,          /* fp16 MFMA, hi/lo split, 3 products     */
  CUMPSGEMM_TF32TCEC = 2,          /* bf16x3 MFMA, 6 products                */
  CUMPSGEMM_FP16TC = 3,            /* fp16 MFMA, no correction               */
  CUMPSGEMM_TF32TC = 4,            /* bf16x2 MFMA, 3 products                */
  CUMPSGEMM_CUBLAS_SIMT = 5,       /* forward to hipBLAS, FP32 compute       */
  CUMPSGEMM_CUBLAS_FP16TC = 6,     /* forward to hipBLAS                     */
  CUMPSGEMM_CUBLAS_TF32TC = 7,     /* forward to hipBLAS                     */
  CUMPSGEMM_DRY_RUN = 8,           /* log only, touch nothing                */
  CUMPSGEMM_AUTO = 9,              /* exp-stats decide FP16TCEC[+scale]/bf16x3 */
  CUMPSGEMM_UNDEFINED = 10,        /* internal: stage-1 statistics undecided */
  CUMPSGEMM_FP16TCEC_SCALING = 11, /* FP16TCEC after power-of-two scaling    */
  CUMPSGEMM_FP32_SIMT = 12         /* not supported (as in the reference)    */
};
#ifndef __cplusplus
typedef enum cuMpSGEMM_compute_mode_t cuMpSGEMM_compute_mode_t;
#endif

#endif
