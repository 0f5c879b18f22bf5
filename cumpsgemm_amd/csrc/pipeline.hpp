// The per-call mode pipeline shared by the interposer and the direct
// cuMpSGEMM_*gemm_pipeline entry points.
#pragma once
#include <cumpsgemm/cumpsgemm.hpp>

namespace cumpsgemm_amd {
struct PipelineIds {
  unsigned a_slot = 0, b_slot = 0, flag_slot = 0;
};
template <class T>
hipblasStatus_t gemm_pipeline(cuMpSGEMM_handle_t h, hipblasOperation_t op_A,
                              hipblasOperation_t op_B, uint64_t m, uint64_t n, uint64_t k,
                              const T *alpha, T *a, uint64_t lda, uint64_t stridea, T *b,
                              uint64_t ldb, uint64_t strideb, const T *beta, T *c, uint64_t ldc,
                              uint64_t stridec, uint64_t batch, bool batched,
                              cuMpSGEMM_compute_mode_t mode, bool restore_AB, PipelineIds *ids);
// C *= 1 / (the coefficient scale_C applies), see dynamic_scaling.hip
template <class T>
void unscale_C(cuMpSGEMM_handle *h, unsigned slot_a, unsigned slot_b, unsigned flag_id, unsigned m, unsigned n,
               T *ptr, unsigned ld, unsigned batch, unsigned stride);
} // namespace cumpsgemm_amd
