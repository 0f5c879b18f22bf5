// C++ API of the MI355X mutable-precision GEMM library.
// Mirrors reference include/cumpsgemm/cumpsgemm.hpp:8-130 (namespace, names,
// argument order and meaning) with HIP types.  T is float or hipComplex.
#ifndef CUMPSGEMM_AMD_HPP
#define CUMPSGEMM_AMD_HPP
#include "cumpsgemm.h"
#include <cstddef>
#include <cstdint>
#include <string>
#include <unordered_map>
#include <utility>

namespace cumpsgemm {
using handle_t = cuMpSGEMM_handle_t;
inline void create(handle_t &handle) { cuMpSGEMM_create(&handle); }
inline void destroy(handle_t handle) { cuMpSGEMM_destroy(handle); }
inline void set_stream(handle_t &handle, hipStream_t stream) {
  cuMpSGEMM_set_stream(handle, stream);
}

// reference cumpsgemm.hpp:16-24 (src/cumpsgemm.cu:228-419).
// used_kernel_module_id receives the index into the gfx950 tile-config table
// (100 + index when the split-K path was taken, ~0u for AUTO).
template <class T>
hipblasStatus_t gemm(handle_t handle, hipblasOperation_t op_A,
                     hipblasOperation_t op_B, uint64_t m, uint64_t n, uint64_t k,
                     const T *alpha, const T *a_dmem_ptr, uint64_t lda,
                     const T *b_dmem_ptr, uint64_t ldb, const T *beta,
                     T *c_dmem_ptr, uint64_t ldc,
                     cuMpSGEMM_compute_mode_t compute_mode,
                     unsigned *used_kernel_module_id = nullptr);

// reference cumpsgemm.hpp:26-35 (src/cumpsgemm.cu:421-547)
template <class T>
hipblasStatus_t gemm_stridedBatch(
    handle_t handle, hipblasOperation_t op_A, hipblasOperation_t op_B,
    uint64_t m, uint64_t n, uint64_t k, const T *alpha, const T *a_dmem_ptr,
    uint64_t lda, uint64_t stridea, const T *b_dmem_ptr, uint64_t ldb,
    uint64_t strideb, const T *beta, T *c_dmem_ptr, uint64_t ldc,
    uint64_t stridec, uint64_t batch_count,
    cuMpSGEMM_compute_mode_t compute_mode,
    unsigned *used_kernel_module_id = nullptr);

// ---- exponent statistics (reference cumpsgemm.hpp:37-68, src/exp_stats.cu) ----
// Both return the ring slot that receives the result.  stride == 0 scans only
// the first matrix of a batch (reference src/exp_stats.cu:306).
template <class T>
unsigned exp_stats_ext(handle_t handle, unsigned m, unsigned n, const T *ptr,
                       unsigned ld, unsigned batch_size = 1, unsigned stride = 0);
template <class T>
unsigned exp_max_ext(handle_t handle, unsigned m, unsigned n, const T *ptr,
                     unsigned ld, unsigned batch_size = 1, unsigned stride = 0);

// {underflow count, total count} of a slot; synchronises the handle's stream.
std::pair<std::size_t, std::size_t> get_exp_stats(handle_t handle,
                                                  unsigned buffer_id);
unsigned get_current_exp_stats_buffer_id(handle_t handle);
void reset_exp_stats_buffer_id(handle_t handle);
void set_exp_stats_params(handle_t handle, float ignore_threshold,
                          float underflow_threshold,
                          float underflow_ratio_tolerance);
void enable_exp_stats(handle_t handle);
void disable_exp_stats(handle_t handle);
// 2^floor(log2 max|x|) of a slot (0 if the matrix is all zero/denormal)
float get_max_exp(handle_t handle, unsigned buffer_id);
cuMpSGEMM_compute_mode_t get_exp_stats_compute_mode_level(handle_t handle,
                                                          unsigned buffer_id);

// ---- power-of-two scaling (reference cumpsgemm.hpp:71-100, src/dynamic_scaling.cu) ----
template <class T>
void scale_A(handle_t handle, unsigned exp_stats_buffer_id,
             unsigned dynamic_launch_flag_buffer_id, unsigned m, unsigned n,
             T *ptr, unsigned ld, unsigned batch_size = 1, unsigned stride = 0);
template <class T>
void scale_B(handle_t handle, unsigned exp_stats_buffer_id,
             unsigned dynamic_launch_flag_buffer_id, unsigned m, unsigned n,
             T *ptr, unsigned ld, unsigned batch_size = 1, unsigned stride = 0);
template <class T>
void scale_C(handle_t handle, unsigned exp_stats_buffer_A_id,
             unsigned exp_stats_buffer_B_id,
             unsigned dynamic_launch_flag_buffer_id, unsigned m, unsigned n,
             T *ptr, unsigned ld, unsigned batch_size = 1, unsigned stride = 0);
template <class T>
void reset_scale_A(handle_t handle, unsigned exp_stats_buffer_id,
                   unsigned dynamic_launch_flag_buffer_id, unsigned m,
                   unsigned n, T *ptr, unsigned ld, unsigned batch_size = 1,
                   unsigned stride = 0);
template <class T>
void reset_scale_B(handle_t handle, unsigned exp_stats_buffer_id,
                   unsigned dynamic_launch_flag_buffer_id, unsigned m,
                   unsigned n, T *ptr, unsigned ld, unsigned batch_size = 1,
                   unsigned stride = 0);

// ---- launch-flag ring (reference cumpsgemm.hpp:104-114) ----
unsigned get_current_dynamic_launch_buffer_id(handle_t handle);
unsigned get_next_dynamic_launch_buffer_id(handle_t handle);
cuMpSGEMM_compute_mode_t get_dynamic_launch_gemm_compute_mode(handle_t handle,
                                                              unsigned buffer_id);
std::pair<int, int> get_dynamic_launch_scaling_mode_AB(handle_t handle,
                                                       unsigned buffer_id);
void set_dynamic_launch_buffer_by_exp_stats(handle_t handle,
                                            unsigned dynamic_launch_buffer_id,
                                            unsigned A_exp_stats_buffer_id,
                                            unsigned B_exp_stats_buffer_id);
// Select / deselect the flag slot that AUTO-mode GEMMs consult
// (reference src/dynamic_launch.cu:60-70, internal there; public here so the
// AUTO pipeline can be driven through the library API alone).
void set_dynamic_launch_flag_buffer_id(handle_t handle, unsigned id);
void unset_dynamic_launch_flag_buffer_id(handle_t handle);

// ---- wall-clock profiling of the stats / scaling / GEMM launches
//      (reference cumpsgemm.hpp:116-129, src/cumpsgemm.cu:814-849) ----
void enable_exp_stats_profiling(handle_t handle);
void disable_exp_stats_profiling(handle_t handle);
void reset_exp_stats_profiling(handle_t handle);
void print_exp_stats_profiling(handle_t handle, unsigned csv = false);
namespace debug {
struct stats_t {
  double time_sum; // seconds
  std::uint64_t n;
};
std::unordered_map<std::string, stats_t>
get_exp_stats_profiling_result(handle_t handle);
} // namespace debug
} // namespace cumpsgemm
#endif
