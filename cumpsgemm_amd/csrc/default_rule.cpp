// Default mode rule.  Compiled into libcumpsgemm.so and, on its own, into
// libcumpsgemm_rule.so -- the library a user replaces to install a custom rule.
// Behaviour follows reference src/default_cumpsgemm_rule.cu:6-49:
//   any of m, n, k <= 1024  -> CUBLAS_SIMT (forward to hipBLAS), before the
//                              environment is even looked at;
//   otherwise CUMPSGEMM_COMPUTE_MODE selects the mode; an unknown value logs an
//   error and forwards; an unset variable forwards silently (the reference
//   dereferences a null pointer there).
#include "utils.hpp"
#include <cstdlib>
#include <cstring>
#include <cumpsgemm/cumpsgemm.h>

extern "C" cuMpSGEMM_compute_mode_t
cuMpSGEMM_get_compute_mode(const char * /*func_name*/, hipblasHandle_t /*hipblas_handle*/,
                           hipblasOperation_t /*op_A*/, hipblasOperation_t /*op_B*/, unsigned m,
                           unsigned n, unsigned k) {
  if (m <= 1024 || n <= 1024 || k <= 1024) return CUMPSGEMM_CUBLAS_SIMT;
  const char *env = std::getenv("CUMPSGEMM_COMPUTE_MODE");
  if (env == nullptr) return CUMPSGEMM_CUBLAS;
  static const struct {
    const char *name;
    cuMpSGEMM_compute_mode_t mode;
  } known[] = {
      {"FP16TCEC", CUMPSGEMM_FP16TCEC},           {"TF32TCEC", CUMPSGEMM_TF32TCEC},
      {"FP16TC", CUMPSGEMM_FP16TC},               {"TF32TC", CUMPSGEMM_TF32TC},
      {"CUBLAS_TF32TC", CUMPSGEMM_CUBLAS_TF32TC}, {"CUBLAS_FP16TC", CUMPSGEMM_CUBLAS_FP16TC},
      {"CUBLAS_SIMT", CUMPSGEMM_CUBLAS_SIMT},     {"CUBLAS", CUMPSGEMM_CUBLAS},
      {"DRY_RUN", CUMPSGEMM_DRY_RUN},             {"AUTO", CUMPSGEMM_AUTO},
      {"FP16TCEC_SCALING", CUMPSGEMM_FP16TCEC_SCALING},
  };
  for (const auto &e : known)
    if (std::strcmp(env, e.name) == 0) return e.mode;
  cumpsgemm_amd::log_error(std::string("Unknown CUMPSGEMM_COMPUTE_MODE = ") + env + ". Ignored");
  return CUMPSGEMM_CUBLAS;
}
