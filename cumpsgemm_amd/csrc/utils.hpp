// Environment-gated logging, same prefixes and gates as the reference
// (src/utils.hpp:5-42): CUMPSGEMM_INFO enables LOG lines (default off),
// CUMPSGEMM_ERROR_LOG gates ERROR (default on) and WARNING (default off).
// Lines go to stdout because the reference's log-replay tool parses them there.
#pragma once
#include <cstdio>
#include <cstdlib>
#include <string>

namespace cumpsgemm_amd {
inline bool env_flag(const char *name, bool when_unset) {
  const char *v = std::getenv(name);
  if (v == nullptr) return when_unset;
  return std::string(v) != "0";
}
inline void log_info(const std::string &s) {
  if (env_flag("CUMPSGEMM_INFO", false)) {
    std::fprintf(stdout, "[cuMpSGEMM LOG] %s\n", s.c_str());
    std::fflush(stdout);
  }
}
inline void log_error(const std::string &s) {
  if (env_flag("CUMPSGEMM_ERROR_LOG", true)) {
    std::fprintf(stdout, "[cuMpSGEMM ERROR] %s\n", s.c_str());
    std::fflush(stdout);
  }
}
inline void log_warning(const std::string &s) {
  if (env_flag("CUMPSGEMM_ERROR_LOG", false)) {
    std::fprintf(stdout, "[cuMpSGEMM WARNING] %s\n", s.c_str());
    std::fflush(stdout);
  }
}
} // namespace cumpsgemm_amd
