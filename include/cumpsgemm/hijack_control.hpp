// Run-time control of the hipBLAS interposer that lives in libcumpsgemm.so.
// Mirrors reference include/cumpsgemm/hijack_control.hpp:9-32
// (implementation there: src/cumpsgemm_cublas.cu:1189-1271).
#ifndef CUMPSGEMM_AMD_HIJACK_CONTROL_HPP
#define CUMPSGEMM_AMD_HIJACK_CONTROL_HPP
#include "detail/common.h"
#include <functional>
#include <string>

namespace cumpsgemm {
namespace hijack_control {
// the lazily created handle all intercepted calls run on
cuMpSGEMM_handle_t get_internal_global_handle();

// pin every intercepted GEMM to `mode` (throws for CUMPSGEMM_FP32_SIMT) /
// go back to asking the rule
void set_compute_mode(cuMpSGEMM_compute_mode_t mode);
void unset_compute_mode();

// route (2^p, 2, 2) and (2, 2^p, 2) shapes to the HBM-streaming kernels
void enable_custom_gemm_Mx2x2();
void disable_custom_gemm_Mx2x2();

void reset_exp_stats_buffer_id();
void set_exp_stats_params(float ignore_threshold, float underflow_threshold,
                          float underflow_tolerance_rate);
void enable_restoring_AB_after_scaling();
void disable_restoring_AB_after_scaling();

// "func,opA,opB,m,n,k,batch,MODE" of the last intercepted call
std::string get_last_called_function_str();
void set_last_called_function_str(const std::string func_str);
void clear_last_called_function_str();

bool is_library_loaded();

// (op_A, op_B, m, n, k) -> mode; takes precedence over the rule library
using control_function_t = std::function<cuMpSGEMM_compute_mode_t(
    const int, const int, const unsigned, const unsigned, const unsigned)>;
void set_control_function(const control_function_t control_function);
void unset_control_function();
} // namespace hijack_control
} // namespace cumpsgemm
#endif
