// Mode pipeline of one GEMM call: statistics -> decision -> scaling -> GEMM ->
// inverse scaling -> restore.  Everything is enqueued on the handle's stream;
// the decision lives in device memory (launch flag), so there is no host
// synchronisation.  Follows the orchestration of the reference's interposer,
// src/cumpsgemm_cublas.cu:446-577 (single) and :836-960 (strided batch).
#include "pipeline.hpp"
#include <cstdlib>
#include <type_traits>
#include "handle.hpp"
#include "utils.hpp"
#include <cumpsgemm/cumpsgemm_ext.h>

namespace cumpsgemm_amd {
template <class T>
hipblasStatus_t gemm_pipeline(cuMpSGEMM_handle_t h, hipblasOperation_t op_A,
                              hipblasOperation_t op_B, uint64_t m, uint64_t n, uint64_t k,
                              const T *alpha, T *a, uint64_t lda, uint64_t stridea, T *b,
                              uint64_t ldb, uint64_t strideb, const T *beta, T *c, uint64_t ldc,
                              uint64_t stridec, uint64_t batch, bool batched,
                              cuMpSGEMM_compute_mode_t mode, bool restore_AB, PipelineIds *ids) {
  // the statistics and scaling entry points take 32-bit sizes, leading
  // dimensions and strides (reference include/cumpsgemm/cumpsgemm.hpp:37-46)
  const bool needs_stats = (mode == CUMPSGEMM_AUTO || mode == CUMPSGEMM_FP16TCEC_SCALING);
  const uint64_t lim = 0xffffffffull;
  if (needs_stats && (m > lim || n > lim || k > lim || lda > lim || ldb > lim || ldc > lim ||
                      (batched && (stridea > lim || strideb > lim || stridec > lim || batch > lim)))) {
    log_error("FP16TCEC_SCALING / AUTO: a size, leading dimension or stride does not fit 32 bits");
    return HIPBLAS_STATUS_INVALID_VALUE;
  }
  // A null matrix would make the statistics pass skip its launch (nothing to
  // scan) and leave the slots and the launch flag that everything after it
  // reads with whatever the ring held before: refuse the call before any launch.
  if (needs_stats && m != 0 && n != 0 && batch != 0 && (c == nullptr || (k != 0 && (a == nullptr || b == nullptr)))) {
    log_error("FP16TCEC_SCALING / AUTO: null matrix pointer");
    return HIPBLAS_STATUS_INVALID_VALUE;
  }
  // stored shapes of A and B (rows x cols as laid out in memory)
  const unsigned a_rows = (unsigned)(op_A == HIPBLAS_OP_N ? m : k);
  const unsigned a_cols = (unsigned)(op_A == HIPBLAS_OP_N ? k : m);
  const unsigned b_rows = (unsigned)(op_B == HIPBLAS_OP_N ? k : n);
  const unsigned b_cols = (unsigned)(op_B == HIPBLAS_OP_N ? n : k);
  // the non-batched form scans one matrix: batch 1, stride 0
  const unsigned sb = batched ? (unsigned)batch : 1u;
  const unsigned sa_stride = batched ? (unsigned)stridea : 0u;
  const unsigned sb_stride = batched ? (unsigned)strideb : 0u;
  const unsigned sc_stride = batched ? (unsigned)stridec : 0u;

  // (the statistics of A and B share one launch per pass)
  const MatrixView<T> va{a, a_rows, a_cols, (unsigned)lda, sb, sa_stride};
  const MatrixView<T> vb{b, b_rows, b_cols, (unsigned)ldb, sb, sb_stride};
  unsigned a_id = 0, b_id = 0, flag_id = 0;
  const bool scaled = (mode == CUMPSGEMM_AUTO || mode == CUMPSGEMM_FP16TCEC_SCALING);
  // When A and B are to come out unchanged (restore_AB, the default) the
  // scaling is fused into the GEMM kernel: A and B are multiplied while they
  // are split and C on the way out, so A and B are never written and five
  // read-modify-write passes over A, B and C disappear.  The reference scales
  // A and B in place through a const_cast and undoes it afterwards
  // (src/cumpsgemm_cublas.cu:511-518, :562-573); that form is kept for callers
  // that ask for the scaled operands to be left behind (restore_AB == false).
  // Both forms compute alpha*op(A)*op(B) + beta*C.  (The reference's sequence
  // GEMM-with-beta, then scale_C over all of C also rescales beta*C_old,
  // src/cumpsgemm_cublas.cu:549-559; the stand-alone form here divides C_old
  // by that power of two first, which the final scale_C undoes exactly.)
  bool beta_nonzero;
  if constexpr (std::is_same<T, hipComplex>::value) beta_nonzero = beta != nullptr && (beta->x != 0.0f || beta->y != 0.0f);
  else beta_nonzero = beta != nullptr && *beta != 0.0f;
  // restore_AB == false with beta != 0: the stand-alone sequence would have to
  // divide C_old by the product of the two scaling factors before the GEMM
  // (so that the final pass over C, which multiplies everything by it, leaves
  // beta * C_old alone), and that quotient can leave the FP32 range (factors
  // down to 2^-88 for operands near 2^-30).  The fused GEMM has no such
  // intermediate; A and B are scaled in place afterwards, as the caller asked.
  const bool scale_ab_after = scaled && !restore_AB && beta_nonzero && !tuning().no_fused_scaling;
  const bool fused = scaled && (restore_AB || scale_ab_after) && !tuning().no_fused_scaling;
  if (mode == CUMPSGEMM_AUTO) {
    // (the second statistics pass also writes the launch flag: the reference's
    // set_dynamic_launch_buffer_by_exp_stats, src/cumpsgemm_cublas.cu:463-466,
    // without a launch of its own)
    flag_id = cumpsgemm::get_next_dynamic_launch_buffer_id(h);
    exp_stats_pair<T>(h, va, vb, a_id, b_id, (int)flag_id);
    if (!fused) {
      cumpsgemm::scale_A<T>(h, a_id, flag_id, a_rows, a_cols, a, (unsigned)lda, sb, sa_stride);
      cumpsgemm::scale_B<T>(h, b_id, flag_id, b_rows, b_cols, b, (unsigned)ldb, sb, sb_stride);
    }
    cumpsgemm::set_dynamic_launch_flag_buffer_id(h, flag_id);
  } else if (mode == CUMPSGEMM_FP16TCEC_SCALING) {
    flag_id = 1; // preset: FP16TCEC with both scale bits
    exp_max_pair<T>(h, va, vb, a_id, b_id);
    if (!fused) {
      cumpsgemm::scale_A<T>(h, a_id, flag_id, a_rows, a_cols, a, (unsigned)lda, sb, sa_stride);
      cumpsgemm::scale_B<T>(h, b_id, flag_id, b_rows, b_cols, b, (unsigned)ldb, sb, sb_stride);
    }
  }
  if (scaled && !fused) {
    // (only with CUMPSGEMM_NO_FUSED_SCALING: C_old / factor must stay inside the FP32 range)
    if (beta_nonzero)
      unscale_C<T>(h, a_id, b_id, flag_id, (unsigned)m, (unsigned)n, c, (unsigned)ldc, sb, sc_stride);
  }
  if (fused) {
    h->fused_scaling = true;
    h->fused_slot_a = a_id;
    h->fused_slot_b = b_id;
    h->fused_flag = flag_id;
  }
  const cuMpSGEMM_compute_mode_t gemm_mode =
      (mode == CUMPSGEMM_FP16TCEC_SCALING) ? CUMPSGEMM_FP16TCEC : mode;
  hipblasStatus_t st;
  if (batched) {
    st = cumpsgemm::gemm_stridedBatch<T>(h, op_A, op_B, m, n, k, alpha, a, lda, stridea, b, ldb,
                                         strideb, beta, c, ldc, stridec, batch, gemm_mode);
  } else {
    st = cumpsgemm::gemm<T>(h, op_A, op_B, m, n, k, alpha, a, lda, b, ldb, beta, c, ldc,
                            gemm_mode);
  }
  h->fused_scaling = false;
  if (scale_ab_after) {
    cumpsgemm::scale_A<T>(h, a_id, flag_id, a_rows, a_cols, a, (unsigned)lda, sb, sa_stride);
    cumpsgemm::scale_B<T>(h, b_id, flag_id, b_rows, b_cols, b, (unsigned)ldb, sb, sb_stride);
  }
  if (scaled && !fused) {
    cumpsgemm::scale_C<T>(h, a_id, b_id, flag_id, (unsigned)m, (unsigned)n, c, (unsigned)ldc, sb,
                          sc_stride);
    if (restore_AB) {
      cumpsgemm::reset_scale_A<T>(h, a_id, flag_id, a_rows, a_cols, a, (unsigned)lda, sb,
                                  sa_stride);
      cumpsgemm::reset_scale_B<T>(h, b_id, flag_id, b_rows, b_cols, b, (unsigned)ldb, sb,
                                  sb_stride);
    }
  }
  if (mode == CUMPSGEMM_AUTO) cumpsgemm::unset_dynamic_launch_flag_buffer_id(h);
  if (ids != nullptr) {
    ids->a_slot = a_id;
    ids->b_slot = b_id;
    ids->flag_slot = flag_id;
  }
  return st;
}

template hipblasStatus_t gemm_pipeline<float>(cuMpSGEMM_handle_t, hipblasOperation_t,
                                              hipblasOperation_t, uint64_t, uint64_t, uint64_t,
                                              const float *, float *, uint64_t, uint64_t, float *,
                                              uint64_t, uint64_t, const float *, float *, uint64_t,
                                              uint64_t, uint64_t, bool, cuMpSGEMM_compute_mode_t,
                                              bool, PipelineIds *);
template hipblasStatus_t gemm_pipeline<hipComplex>(
    cuMpSGEMM_handle_t, hipblasOperation_t, hipblasOperation_t, uint64_t, uint64_t, uint64_t,
    const hipComplex *, hipComplex *, uint64_t, uint64_t, hipComplex *, uint64_t, uint64_t,
    const hipComplex *, hipComplex *, uint64_t, uint64_t, uint64_t, bool,
    cuMpSGEMM_compute_mode_t, bool, PipelineIds *);
} // namespace cumpsgemm_amd

using cumpsgemm_amd::PipelineIds;

extern "C" {
hipblasStatus_t cuMpSGEMM_sgemm_pipeline(cuMpSGEMM_handle_t handle, hipblasOperation_t op_A,
                                         hipblasOperation_t op_B, uint64_t m, uint64_t n,
                                         uint64_t k, const float *alpha, float *a, uint64_t lda,
                                         uint64_t stridea, float *b, uint64_t ldb,
                                         uint64_t strideb, const float *beta, float *c,
                                         uint64_t ldc, uint64_t stridec, uint64_t batch_count,
                                         cuMpSGEMM_compute_mode_t mode, int restore_AB,
                                         unsigned *ids_out) {
  PipelineIds ids;
  const bool batched = !(batch_count == 1 && stridea == 0 && strideb == 0 && stridec == 0);
  const auto st = cumpsgemm_amd::gemm_pipeline<float>(handle, op_A, op_B, m, n, k, alpha, a, lda,
                                                      stridea, b, ldb, strideb, beta, c, ldc,
                                                      stridec, batch_count, batched, mode,
                                                      restore_AB != 0, &ids);
  if (ids_out) {
    ids_out[0] = ids.a_slot;
    ids_out[1] = ids.b_slot;
    ids_out[2] = ids.flag_slot;
  }
  return st;
}
hipblasStatus_t cuMpSGEMM_cgemm_pipeline(cuMpSGEMM_handle_t handle, hipblasOperation_t op_A,
                                         hipblasOperation_t op_B, uint64_t m, uint64_t n,
                                         uint64_t k, const hipComplex *alpha, hipComplex *a,
                                         uint64_t lda, uint64_t stridea, hipComplex *b,
                                         uint64_t ldb, uint64_t strideb, const hipComplex *beta,
                                         hipComplex *c, uint64_t ldc, uint64_t stridec,
                                         uint64_t batch_count, cuMpSGEMM_compute_mode_t mode,
                                         int restore_AB, unsigned *ids_out) {
  PipelineIds ids;
  const bool batched = !(batch_count == 1 && stridea == 0 && strideb == 0 && stridec == 0);
  const auto st = cumpsgemm_amd::gemm_pipeline<hipComplex>(
      handle, op_A, op_B, m, n, k, alpha, a, lda, stridea, b, ldb, strideb, beta, c, ldc, stridec,
      batch_count, batched, mode, restore_AB != 0, &ids);
  if (ids_out) {
    ids_out[0] = ids.a_slot;
    ids_out[1] = ids.b_slot;
    ids_out[2] = ids.flag_slot;
  }
  return st;
}
}
