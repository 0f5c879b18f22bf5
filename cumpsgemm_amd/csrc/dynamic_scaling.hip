// Power-of-two scaling of A, B (to max exponent 2^14) and inverse scaling of C,
// plus the device-resident launch-flag ring that AUTO mode uses to pick a
// kernel without a host synchronisation.  HBM-bound streaming kernels: 16-byte
// read-modify-write, the coefficient is derived on the device from the
// statistics slot so nothing is read back to the host.
//
// Follows reference src/dynamic_scaling.cu:15 (2^14 target), :75-97 (A/B),
// :99-126 (C), :128-150 (undo), :364-385 (flag from two stats decisions) and
// src/dynamic_launch.cu / dynamic_launch_utils.hpp (flag ring and bit layout:
// mode in bits 0-4, scale-B bit 5, scale-A bit 6).
#include "handle.hpp"
#include "utils.hpp"
#include <cumpsgemm/cumpsgemm.hpp>
#include <cumpsgemm/cumpsgemm_ext.h>
#include <type_traits>

namespace cumpsgemm_amd {
namespace {
constexpr int kBlock = 256;
constexpr float kHalfExpMax = 16384.0f; // 2^14

// UNSCALE_C: the inverse of SCALE_C's coefficient (see unscale_C below)
enum ScaleKind : int { SCALE_A = 0, SCALE_B = 1, SCALE_C = 2, RESET_A = 3, RESET_B = 4, UNSCALE_C = 5 };

// Coefficient for one scaling launch, or 0 to skip (flag bit clear / max == 0).
__device__ inline float scaling_coef(int kind, const int *flag_ptr, const StatsSlot *slot_a,
                                     const StatsSlot *slot_b) {
  const int flag = *flag_ptr;
  const float ma = __uint_as_float(slot_a->max_exp_bits);
  if (kind == SCALE_C || kind == UNSCALE_C) {
    const float mb = __uint_as_float(slot_b->max_exp_bits);
    if (ma == 0.0f || mb == 0.0f) return 0.0f;
    const bool sa = flag & kScaleABit, sb = flag & kScaleBBit;
    if (!sa && !sb) return 0.0f;
    float coef = 1.0f;
    if (kind == SCALE_C) {
      if (sa) coef *= ma / kHalfExpMax;
      if (sb) coef *= mb / kHalfExpMax;
    } else {
      if (sa) coef *= kHalfExpMax / ma;
      if (sb) coef *= kHalfExpMax / mb;
    }
    return coef;
  }
  const bool is_a = (kind == SCALE_A || kind == RESET_A);
  if (!(flag & (is_a ? kScaleABit : kScaleBBit))) return 0.0f;
  if (ma == 0.0f) return 0.0f;
  return (kind == SCALE_A || kind == SCALE_B) ? kHalfExpMax / ma : ma / kHalfExpMax;
}

__global__ __launch_bounds__(kBlock) void scaling_kernel(
    int kind, const int *flag_ptr, const StatsSlot *slot_a, const StatsSlot *slot_b, float *ptr,
    unsigned long long count_f, unsigned m_f, unsigned n, unsigned long long ld_f,
    unsigned nbatch, unsigned long long stride_f) {
  const float coef = scaling_coef(kind, flag_ptr, slot_a, slot_b);
  if (coef == 0.0f) return;
  const unsigned tid = threadIdx.x;
  if (count_f != 0) {
    const unsigned long long mis = ((16 - ((uintptr_t)ptr & 15)) & 15) / 4;
    const unsigned long long head = mis < count_f ? mis : count_f;
    float4 *body = reinterpret_cast<float4 *>(ptr + head);
    const unsigned long long nvec = (count_f - head) / 4;
    const unsigned long long gsz = (unsigned long long)gridDim.x * kBlock;
    unsigned long long i = (unsigned long long)blockIdx.x * kBlock + tid;
    // contiguous chunks of 4 * kBlock vectors per workgroup: the grid streams
    // one compact window at a time
    constexpr unsigned long long kChunk = 4ull * kBlock;
    const unsigned long long nfull = nvec / kChunk;
    for (unsigned long long c = blockIdx.x; c < nfull; c += gridDim.x) {
      float4 *cp = body + c * kChunk + tid;
      float4 v0 = cp[0], v1 = cp[kBlock], v2 = cp[2 * kBlock], v3 = cp[3 * kBlock];
      v0.x *= coef; v0.y *= coef; v0.z *= coef; v0.w *= coef;
      v1.x *= coef; v1.y *= coef; v1.z *= coef; v1.w *= coef;
      v2.x *= coef; v2.y *= coef; v2.z *= coef; v2.w *= coef;
      v3.x *= coef; v3.y *= coef; v3.z *= coef; v3.w *= coef;
      cp[0] = v0; cp[kBlock] = v1; cp[2 * kBlock] = v2; cp[3 * kBlock] = v3;
    }
    i += nfull * kChunk;
    for (; i < nvec; i += gsz) {
      float4 v = body[i];
      v.x *= coef; v.y *= coef; v.z *= coef; v.w *= coef;
      body[i] = v;
    }
    if (blockIdx.x == 0) {
      if (tid < head) ptr[tid] *= coef;
      const unsigned long long tail0 = head + nvec * 4;
      if (tail0 + tid < count_f) ptr[tail0 + tid] *= coef;
    }
  } else {
    const unsigned long long ncols = (unsigned long long)n * nbatch;
    for (unsigned long long col = blockIdx.x; col < ncols; col += gridDim.x) {
      float *cp = ptr + (col / n) * stride_f + (col % n) * ld_f;
      for (unsigned i = tid; i < m_f; i += kBlock) cp[i] *= coef;
    }
  }
}

template <class T>
void launch_scaling(cuMpSGEMM_handle *h, int kind, unsigned slot_a, unsigned slot_b,
                    unsigned flag_id, unsigned m, unsigned n, T *ptr, unsigned ld, unsigned batch,
                    unsigned stride, const char *label) {
  constexpr unsigned ES = std::is_same<T, hipComplex>::value ? 2 : 1;
  if (ptr == nullptr || m == 0 || n == 0) {
    if (ptr == nullptr && m != 0 && n != 0) log_error(std::string(label) + ": null matrix pointer, nothing scaled");
    return;
  }
  const unsigned nbatch = (stride == 0) ? 1 : batch;
  const bool dense_cols = (ld == m) || n == 1;
  const bool dense_batch = nbatch == 1 || (unsigned long long)stride == (unsigned long long)m * n;
  const unsigned long long total_f = (unsigned long long)m * n * nbatch * ES;
  unsigned long long count_f = 0, blocks;
  if (dense_cols && dense_batch) {
    count_f = total_f;
    blocks = (total_f / 4 + kBlock * 4 - 1) / (kBlock * 4);
  } else {
    blocks = (unsigned long long)n * nbatch;
  }
  const unsigned long long cap = (unsigned long long)h->num_cus * 8;
  const unsigned grid = (unsigned)std::max<unsigned long long>(1, std::min(blocks, cap));
  ProfileScope prof(h, label);
  hipLaunchKernelGGL(scaling_kernel, dim3(grid), dim3(kBlock), 0, h->stream, kind,
                     h->flag_buffer + flag_id, h->stats_slots + slot_a, h->stats_slots + slot_b,
                     reinterpret_cast<float *>(ptr), count_f, m * ES, n,
                     (unsigned long long)ld * ES, nbatch, (unsigned long long)stride * ES);
}

__global__ void combine_flag_kernel(int *flag, const StatsSlot *a, const StatsSlot *b) {
  *flag = combine_launch_flag(a->mode, b->mode);
}

int read_flag(cuMpSGEMM_handle *h, unsigned id) {
  int v = 0;
  check_hip(hipMemcpyAsync(&v, h->flag_buffer + id, sizeof(int), hipMemcpyDeviceToHost, h->stream),
            "read launch flag");
  check_hip(hipStreamSynchronize(h->stream), "sync after flag read");
  return v;
}
} // namespace
} // namespace cumpsgemm_amd

namespace cumpsgemm_amd {
// C *= 1 / (scale_C's coefficient).  The stand-alone form of the scaled
// pipelines runs this on C before a GEMM with beta != 0, so that the scale_C
// pass that follows the GEMM -- which multiplies all of C, beta * C_old
// included -- leaves beta * C_old as it was: every factor is a power of two,
// hence exact unless C_old / coefficient leaves FP32's range.
template <class T>
void unscale_C(cuMpSGEMM_handle *h, unsigned slot_a, unsigned slot_b, unsigned flag_id, unsigned m, unsigned n,
               T *ptr, unsigned ld, unsigned batch, unsigned stride) {
  launch_scaling<T>(h, UNSCALE_C, slot_a, slot_b, flag_id, m, n, ptr, ld, batch, stride, "scaling_C");
}
template void unscale_C<float>(cuMpSGEMM_handle *, unsigned, unsigned, unsigned, unsigned, unsigned, float *,
                               unsigned, unsigned, unsigned);
template void unscale_C<hipComplex>(cuMpSGEMM_handle *, unsigned, unsigned, unsigned, unsigned, unsigned,
                                    hipComplex *, unsigned, unsigned, unsigned);
} // namespace cumpsgemm_amd

using namespace cumpsgemm_amd;

template <class T>
void cumpsgemm::scale_A(handle_t h, unsigned exp_stats_buffer_id, unsigned flag_id, unsigned m,
                        unsigned n, T *ptr, unsigned ld, unsigned batch_size, unsigned stride) {
  launch_scaling<T>(h, SCALE_A, exp_stats_buffer_id, exp_stats_buffer_id, flag_id, m, n, ptr, ld,
                    batch_size, stride, "scaling_AB");
}
template <class T>
void cumpsgemm::scale_B(handle_t h, unsigned exp_stats_buffer_id, unsigned flag_id, unsigned m,
                        unsigned n, T *ptr, unsigned ld, unsigned batch_size, unsigned stride) {
  launch_scaling<T>(h, SCALE_B, exp_stats_buffer_id, exp_stats_buffer_id, flag_id, m, n, ptr, ld,
                    batch_size, stride, "scaling_AB");
}
template <class T>
void cumpsgemm::scale_C(handle_t h, unsigned exp_stats_buffer_A_id, unsigned exp_stats_buffer_B_id,
                        unsigned flag_id, unsigned m, unsigned n, T *ptr, unsigned ld,
                        unsigned batch_size, unsigned stride) {
  launch_scaling<T>(h, SCALE_C, exp_stats_buffer_A_id, exp_stats_buffer_B_id, flag_id, m, n, ptr,
                    ld, batch_size, stride, "scaling_C");
}
template <class T>
void cumpsgemm::reset_scale_A(handle_t h, unsigned exp_stats_buffer_id, unsigned flag_id,
                              unsigned m, unsigned n, T *ptr, unsigned ld, unsigned batch_size,
                              unsigned stride) {
  launch_scaling<T>(h, RESET_A, exp_stats_buffer_id, exp_stats_buffer_id, flag_id, m, n, ptr, ld,
                    batch_size, stride, "reset_scaling_AB");
}
template <class T>
void cumpsgemm::reset_scale_B(handle_t h, unsigned exp_stats_buffer_id, unsigned flag_id,
                              unsigned m, unsigned n, T *ptr, unsigned ld, unsigned batch_size,
                              unsigned stride) {
  launch_scaling<T>(h, RESET_B, exp_stats_buffer_id, exp_stats_buffer_id, flag_id, m, n, ptr, ld,
                    batch_size, stride, "reset_scaling_AB");
}

#define INST(T)                                                                                   \
  template void cumpsgemm::scale_A<T>(handle_t, unsigned, unsigned, unsigned, unsigned, T *,      \
                                      unsigned, unsigned, unsigned);                              \
  template void cumpsgemm::scale_B<T>(handle_t, unsigned, unsigned, unsigned, unsigned, T *,      \
                                      unsigned, unsigned, unsigned);                              \
  template void cumpsgemm::scale_C<T>(handle_t, unsigned, unsigned, unsigned, unsigned, unsigned, \
                                      T *, unsigned, unsigned, unsigned);                         \
  template void cumpsgemm::reset_scale_A<T>(handle_t, unsigned, unsigned, unsigned, unsigned,     \
                                            T *, unsigned, unsigned, unsigned);                   \
  template void cumpsgemm::reset_scale_B<T>(handle_t, unsigned, unsigned, unsigned, unsigned,     \
                                            T *, unsigned, unsigned, unsigned);
INST(float)
INST(hipComplex)
#undef INST

unsigned cumpsgemm::get_current_dynamic_launch_buffer_id(handle_t h) { return h->flag_current_id; }
unsigned cumpsgemm::get_next_dynamic_launch_buffer_id(handle_t h) {
  // slots 0 / 1 are presets; 2..length-1 cycle (the index wraps, the length stays)
  h->flag_current_id++;
  if (h->flag_current_id >= h->flag_ring_length) h->flag_current_id = 2;
  return h->flag_current_id;
}
cuMpSGEMM_compute_mode_t cumpsgemm::get_dynamic_launch_gemm_compute_mode(handle_t h,
                                                                         unsigned buffer_id) {
  return (cuMpSGEMM_compute_mode_t)(read_flag(h, buffer_id) & kModeMask);
}
std::pair<int, int> cumpsgemm::get_dynamic_launch_scaling_mode_AB(handle_t h, unsigned buffer_id) {
  const int f = read_flag(h, buffer_id);
  return {(f & kScaleABit) ? 1 : 0, (f & kScaleBBit) ? 1 : 0};
}
void cumpsgemm::set_dynamic_launch_buffer_by_exp_stats(handle_t h, unsigned flag_id,
                                                       unsigned A_exp_stats_buffer_id,
                                                       unsigned B_exp_stats_buffer_id) {
  hipLaunchKernelGGL(combine_flag_kernel, dim3(1), dim3(1), 0, h->stream, h->flag_buffer + flag_id,
                     h->stats_slots + A_exp_stats_buffer_id,
                     h->stats_slots + B_exp_stats_buffer_id);
}
void cumpsgemm::set_dynamic_launch_flag_buffer_id(handle_t h, unsigned id) {
  h->flag_enabled_id = id;
  h->flag_enabled = true;
}
void cumpsgemm::unset_dynamic_launch_flag_buffer_id(handle_t h) {
  h->flag_enabled_id = 0;
  h->flag_enabled = false;
}

extern "C" {
#define SCALE_C_ABI(NAME, FN, T)                                                                  \
  void NAME(cuMpSGEMM_handle_t h, unsigned stats_id, unsigned flag_id, unsigned m, unsigned n,    \
            T *ptr, unsigned ld, unsigned batch, unsigned stride) {                               \
    cumpsgemm::FN<T>(h, stats_id, flag_id, m, n, ptr, ld, batch, stride);                         \
  }
SCALE_C_ABI(cuMpSGEMM_scale_A_s, scale_A, float)
SCALE_C_ABI(cuMpSGEMM_scale_A_c, scale_A, hipComplex)
SCALE_C_ABI(cuMpSGEMM_scale_B_s, scale_B, float)
SCALE_C_ABI(cuMpSGEMM_scale_B_c, scale_B, hipComplex)
SCALE_C_ABI(cuMpSGEMM_reset_scale_A_s, reset_scale_A, float)
SCALE_C_ABI(cuMpSGEMM_reset_scale_A_c, reset_scale_A, hipComplex)
SCALE_C_ABI(cuMpSGEMM_reset_scale_B_s, reset_scale_B, float)
SCALE_C_ABI(cuMpSGEMM_reset_scale_B_c, reset_scale_B, hipComplex)
#undef SCALE_C_ABI
void cuMpSGEMM_scale_C_s(cuMpSGEMM_handle_t h, unsigned stats_a, unsigned stats_b, unsigned flag_id,
                         unsigned m, unsigned n, float *ptr, unsigned ld, unsigned batch,
                         unsigned stride) {
  cumpsgemm::scale_C<float>(h, stats_a, stats_b, flag_id, m, n, ptr, ld, batch, stride);
}
void cuMpSGEMM_scale_C_c(cuMpSGEMM_handle_t h, unsigned stats_a, unsigned stats_b, unsigned flag_id,
                         unsigned m, unsigned n, hipComplex *ptr, unsigned ld, unsigned batch,
                         unsigned stride) {
  cumpsgemm::scale_C<hipComplex>(h, stats_a, stats_b, flag_id, m, n, ptr, ld, batch, stride);
}
unsigned cuMpSGEMM_get_current_dynamic_launch_buffer_id(cuMpSGEMM_handle_t h) {
  return cumpsgemm::get_current_dynamic_launch_buffer_id(h);
}
unsigned cuMpSGEMM_get_next_dynamic_launch_buffer_id(cuMpSGEMM_handle_t h) {
  return cumpsgemm::get_next_dynamic_launch_buffer_id(h);
}
int cuMpSGEMM_get_dynamic_launch_flag(cuMpSGEMM_handle_t h, unsigned id) {
  try { // no exception may cross the C boundary
    return read_flag(h, id);
  } catch (const std::exception &) {
    return 0;
  }
}
void cuMpSGEMM_set_dynamic_launch_buffer_by_exp_stats(cuMpSGEMM_handle_t h, unsigned flag_id,
                                                      unsigned a_id, unsigned b_id) {
  cumpsgemm::set_dynamic_launch_buffer_by_exp_stats(h, flag_id, a_id, b_id);
}
void cuMpSGEMM_set_dynamic_launch_flag_buffer_id(cuMpSGEMM_handle_t h, unsigned id) {
  cumpsgemm::set_dynamic_launch_flag_buffer_id(h, id);
}
void cuMpSGEMM_unset_dynamic_launch_flag_buffer_id(cuMpSGEMM_handle_t h) {
  cumpsgemm::unset_dynamic_launch_flag_buffer_id(h);
}
} // extern "C"
