// hipBLAS interposer.  When libcumpsgemm.so is LD_PRELOADed the six symbols
// below shadow hipBLAS's; each call asks the mode rule what to do and either
// forwards to the real hipBLAS function (found with dlsym(RTLD_NEXT)) or runs
// the TCEC pipeline on the library's global handle, on the caller's stream.
//
// Takes the place of reference src/cumpsgemm_cublas.cu: mode query :198-220,
// per-call flow :222-593 / :595-976, intercepted symbols :979-1187,
// hijack_control :1189-1271, global handle and env configuration :101-157.
#include "handle.hpp"
#include "pipeline.hpp"
#include "utils.hpp"
#include <cumpsgemm/cumpsgemm.hpp>
#include <cumpsgemm/cumpsgemm_ext.h>
#include <cumpsgemm/hijack_control.hpp>
#include <ctime>
#include <dlfcn.h>
#include <mutex>
#include <sstream>
#include <stdexcept>
#include <type_traits>

namespace {
using namespace cumpsgemm_amd;

// one library handle per device, created at the first intercepted call made
// with that device current (the reference keeps a single one for the process,
// src/cumpsgemm_cublas.cu:101-157)
constexpr int kMaxDevices = 64;
cuMpSGEMM_handle_t g_handles[kMaxDevices] = {};
std::once_flag g_handle_once[kMaxDevices];
int current_device() {
  int d = 0;
  if (hipGetDevice(&d) != hipSuccess) {
    (void)hipGetLastError();
    d = 0;
  }
  return (d >= 0 && d < kMaxDevices) ? d : 0;
}
// Record of the last intercepted call; its text form is only made when somebody
// asks for it (an intercepted call that is forwarded must stay cheap).
struct LastCall {
  bool from_call = false;
  const char *func_name = "";
  hipblasOperation_t op_A = HIPBLAS_OP_N, op_B = HIPBLAS_OP_N;
  int m = 0, n = 0, k = 0, batch = 1;
  cuMpSGEMM_compute_mode_t mode = CUMPSGEMM_CUBLAS;
  std::string text; // set through the control API, or cached
} g_last;
const char *op_str(hipblasOperation_t op);
const std::string &last_called_text() {
  if (g_last.from_call) {
    g_last.text = std::string(g_last.func_name) + "," + op_str(g_last.op_A) + "," + op_str(g_last.op_B) + "," +
                  std::to_string(g_last.m) + "," + std::to_string(g_last.n) + "," + std::to_string(g_last.k) +
                  "," + std::to_string(g_last.batch) + "," + cuMpSGEMM_get_compute_mode_string(g_last.mode);
    g_last.from_call = false;
  }
  return g_last.text;
}
void set_last_called_text(const std::string &s) {
  g_last.from_call = false;
  g_last.text = s;
}
bool g_mx2x2_enabled = false;
bool g_restore_AB = true;
cumpsgemm::hijack_control::control_function_t g_control_func;
enum { STATIC_MODE, DYNAMIC_MODE } g_hijack_mode = DYNAMIC_MODE;
cuMpSGEMM_compute_mode_t g_static_mode = CUMPSGEMM_CUBLAS;

std::string sci(double v) {
  std::stringstream ss;
  ss << std::scientific << v;
  return ss.str();
}

const char *op_str(hipblasOperation_t op) {
  switch (op) {
  case HIPBLAS_OP_N: return "N";
  case HIPBLAS_OP_T: return "T";
  case HIPBLAS_OP_C: return "C";
  default: return "?";
  }
}

// The next definition of `name` after this library in the lookup order (the
// real hipBLAS when we are preloaded); falls back to opening libhipblas.so.
void *real_symbol(const char *name) {
  void *p = dlsym(RTLD_NEXT, name);
  if (p == nullptr) {
    static void *lib = dlopen("libhipblas.so", RTLD_NOW | RTLD_GLOBAL);
    if (lib == nullptr) lib = dlopen("libhipblas.so.3", RTLD_NOW | RTLD_GLOBAL);
    if (lib != nullptr) p = dlsym(lib, name);
  }
  if (p == nullptr)
    log_error(std::string("Could not load the hipBLAS function \"") + name + "\"");
  return p;
}

hipStream_t caller_stream(hipblasHandle_t hb) {
  using fn_t = hipblasStatus_t (*)(hipblasHandle_t, hipStream_t *);
  static fn_t fn = reinterpret_cast<fn_t>(real_symbol("hipblasGetStream"));
  hipStream_t s = nullptr;
  if (fn != nullptr && hb != nullptr) (void)fn(hb, &s);
  return s;
}

// Whether the caller's hipBLAS handle takes alpha and beta from device memory.
// This library's entry points read them on the host (as the reference does,
// src/cumpsgemm.cu:266, with no cublasGetPointerMode anywhere in
// src/cumpsgemm_cublas.cu), so such calls are left to hipBLAS.
bool device_pointer_mode(hipblasHandle_t hb) {
  using fn_t = hipblasStatus_t (*)(hipblasHandle_t, hipblasPointerMode_t *);
  static fn_t fn = reinterpret_cast<fn_t>(real_symbol("hipblasGetPointerMode"));
  hipblasPointerMode_t pm = HIPBLAS_POINTER_MODE_HOST;
  if (fn == nullptr || hb == nullptr || fn(hb, &pm) != HIPBLAS_STATUS_SUCCESS) return false;
  return pm == HIPBLAS_POINTER_MODE_DEVICE;
}

bool mx2x2_enabled() {
  if (g_mx2x2_enabled) return true;
  return env_flag("CUMPSGEMM_CUSTOM_GEMM_MX2X2", false);
}

float env_float(const char *name, float dflt) {
  const char *v = std::getenv(name);
  return v ? std::stof(v) : dflt;
}
int env_int(const char *name, int dflt) {
  const char *v = std::getenv(name);
  return v ? std::stoi(v) : dflt;
}

cuMpSGEMM_handle_t global_handle() {
  const int dev = current_device();
  std::call_once(g_handle_once[dev], [dev]() {
    cuMpSGEMM_handle_t &g_handle = g_handles[dev];
    log_info("Initialize cuMpSGEMM handle...");
    if (cuMpSGEMM_create(&g_handle) != HIPBLAS_STATUS_SUCCESS) {
      log_error("Initialization failed.");
      g_handle = nullptr;
      return;
    }
    const float ignore_thr = env_float("CUMPSGEMM_AUTO_IGNORE_THRESHOLD", 0.0f);
    const float under_thr = env_float("CUMPSGEMM_AUTO_UNDERFLOW_THRESHOLD", 1.0f / 32768);
    const float tol = env_float("CUMPSGEMM_AUTO_UNDERFLOW_TOLERANCE_RATE", 0.0f);
    const int restore = env_int("CUMPSGEMM_AUTO_RESTORE_AB_SCALING", 1);
    log_info("AUTO config: ignore_threshold=" + sci(ignore_thr) + " @Init");
    log_info("AUTO config: underflow_threshold=" + sci(under_thr) + " @Init");
    log_info("AUTO config: underflow_tolerance_rate=" + sci(tol) + " @Init");
    log_info("AUTO config: restore_AB_scaling=" + std::to_string(restore) + " @Init");
    log_info(std::string("CUSTOM_GEMM_MX2X2: ") + (mx2x2_enabled() ? "enabled" : "disabled") +
             " @Init");
    cumpsgemm::set_exp_stats_params(g_handle, ignore_thr, under_thr, tol);
    g_restore_AB = restore != 0;
  });
  return g_handles[dev];
}

using rule_fn_t = cuMpSGEMM_compute_mode_t (*)(const char *, hipblasHandle_t, hipblasOperation_t,
                                               hipblasOperation_t, unsigned, unsigned, unsigned);

// The user's rule library, looked up once.  The documented contract is that a
// libcumpsgemm_rule.so on the loader path which defines
// cuMpSGEMM_get_compute_mode replaces the built-in rule.
rule_fn_t user_rule() {
  static rule_fn_t fn = []() -> rule_fn_t {
    void *lib = dlopen("libcumpsgemm_rule.so", RTLD_NOW | RTLD_LOCAL);
    if (lib == nullptr) {
      log_warning("Failed to load libcumpsgemm_rule.so. Default rule will be used.");
      return nullptr;
    }
    void *p = dlsym(lib, "cuMpSGEMM_get_compute_mode");
    if (p == nullptr) {
      log_warning("Failed to load a function cuMpSGEMM_get_compute_mode during selecting "
                  "hijacking function. Default rule will be used.");
      return nullptr;
    }
    return reinterpret_cast<rule_fn_t>(p);
  }();
  return fn;
}

cuMpSGEMM_compute_mode_t query_mode(const char *func_name, hipblasHandle_t hb,
                                    hipblasOperation_t op_A, hipblasOperation_t op_B, unsigned m,
                                    unsigned n, unsigned k) {
  if (g_hijack_mode == STATIC_MODE) return g_static_mode;
  if (g_control_func) return g_control_func((int)op_A, (int)op_B, m, n, k);
  if (rule_fn_t fn = user_rule()) return fn(func_name, hb, op_A, op_B, m, n, k);
  return cuMpSGEMM_get_compute_mode(func_name, hb, op_A, op_B, m, n, k);
}

bool forwards_to_hipblas(cuMpSGEMM_compute_mode_t mode) {
  return mode == CUMPSGEMM_CUBLAS || mode == CUMPSGEMM_CUBLAS_FP16TC ||
         mode == CUMPSGEMM_CUBLAS_TF32TC || mode == CUMPSGEMM_CUBLAS_SIMT;
}

bool is_pow2(uint64_t v) { return (v & (v - 1)) == 0; }

template <class T> struct ffi;
template <> struct ffi<float> {
  static constexpr const char *gemm = "hipblasSgemm";
  static constexpr const char *gemm_sb = "hipblasSgemmStridedBatched";
};
template <> struct ffi<hipComplex> {
  static constexpr const char *gemm = "hipblasCgemm";
  static constexpr const char *gemm_sb = "hipblasCgemmStridedBatched";
};

template <class T>
hipblasStatus_t forward_gemm(hipblasHandle_t hb, hipblasOperation_t op_A, hipblasOperation_t op_B,
                             int m, int n, int k, const T *alpha, const T *a, int lda, const T *b,
                             int ldb, const T *beta, T *c, int ldc) {
  using fn_t = hipblasStatus_t (*)(hipblasHandle_t, hipblasOperation_t, hipblasOperation_t, int,
                                   int, int, const T *, const T *, int, const T *, int, const T *,
                                   T *, int);
  static fn_t fn = reinterpret_cast<fn_t>(real_symbol(ffi<T>::gemm));
  if (fn == nullptr) return HIPBLAS_STATUS_NOT_SUPPORTED;
  return fn(hb, op_A, op_B, m, n, k, alpha, a, lda, b, ldb, beta, c, ldc);
}

template <class T>
hipblasStatus_t forward_gemm_sb(hipblasHandle_t hb, hipblasOperation_t op_A,
                                hipblasOperation_t op_B, int m, int n, int k, const T *alpha,
                                const T *a, int lda, long long sa, const T *b, int ldb,
                                long long sb, const T *beta, T *c, int ldc, long long sc,
                                int batch) {
  using fn_t = hipblasStatus_t (*)(hipblasHandle_t, hipblasOperation_t, hipblasOperation_t, int,
                                   int, int, const T *, const T *, int, long long, const T *, int,
                                   long long, const T *, T *, int, long long, int);
  static fn_t fn = reinterpret_cast<fn_t>(real_symbol(ffi<T>::gemm_sb));
  if (fn == nullptr) return HIPBLAS_STATUS_NOT_SUPPORTED;
  return fn(hb, op_A, op_B, m, n, k, alpha, a, lda, sa, b, ldb, sb, beta, c, ldc, sc, batch);
}

// One intercepted call.  batched == false: strides are ignored, batch == 1.
// Per-call wall-clock profiling of intercepted GEMMs, switched on by
// CUMPSGEMM_ENABLE_CULIP_PROFILING (any value but "0").  The stream is drained
// before the first and after the second timestamp, and one line
//   [CULiP Result][<label>] <nanoseconds>ns
// goes to stdout, with the labels of reference src/cumpsgemm_cublas.cu:270-297,
// :393-416, :430-441, :648-677, :780-806, :812-822 and the line format of
// src/culip.cu:19-33 (existing log parsers keep working).
bool culip_enabled() {
  const char *v = std::getenv("CUMPSGEMM_ENABLE_CULIP_PROFILING");
  return v != nullptr && std::string(v) != "0";
}
struct CulipScope {
  bool on;
  hipStream_t stream;
  std::string label;
  struct timespec t0;
  CulipScope(bool enabled, hipStream_t st, const std::string &name, hipblasOperation_t op_A,
             hipblasOperation_t op_B, long m, long n, long k, bool batched, long batch)
      : on(enabled), stream(st) {
    if (!on) return;
    char buf[128];
    if (batched)
      std::snprintf(buf, sizeof(buf), "%s-%s%s-m%lu-n%lu-k%lu-batchCount%lu", name.c_str(), op_str(op_A),
                    op_str(op_B), (unsigned long)m, (unsigned long)n, (unsigned long)k,
                    (unsigned long)batch);
    else
      std::snprintf(buf, sizeof(buf), "%s-%s%s-m%lu-n%lu-k%lu", name.c_str(), op_str(op_A), op_str(op_B),
                    (unsigned long)m, (unsigned long)n, (unsigned long)k);
    label = buf;
    (void)hipStreamSynchronize(stream);
    clock_gettime(CLOCK_MONOTONIC, &t0);
  }
  ~CulipScope() {
    if (!on) return;
    (void)hipStreamSynchronize(stream);
    struct timespec t1;
    clock_gettime(CLOCK_MONOTONIC, &t1);
    const long ns = ((long)t1.tv_sec - (long)t0.tv_sec) * 1000000000L + ((long)t1.tv_nsec - (long)t0.tv_nsec);
    std::printf("[CULiP Result][%s] %luns\n", label.c_str(), (unsigned long)ns);
    std::fflush(stdout);
  }
};

template <class T>
hipblasStatus_t hijack_core(const char *func_name, hipblasHandle_t hb, hipblasOperation_t op_A,
                            hipblasOperation_t op_B, int m, int n, int k, const T *alpha,
                            const T *a, int lda, long long sa, const T *b, int ldb, long long sb,
                            const T *beta, T *c, int ldc, long long sc, int batch, bool batched) {
  if (m <= 0 || n <= 0 || k <= 0 || lda <= 0 || ldb <= 0 || ldc <= 0 || (batched && batch <= 0)) {
    return HIPBLAS_STATUS_INVALID_VALUE;
  }
  const cuMpSGEMM_compute_mode_t mode = query_mode(func_name, hb, op_A, op_B, m, n, k);
  // scalars in device memory: nothing here can read them, the call goes to hipBLAS
  const bool device_scalars = mode != CUMPSGEMM_DRY_RUN && device_pointer_mode(hb);
  const bool gate_shape = mx2x2_enabled() && !device_scalars && k == 2 &&
                          ((n == 2 && is_pow2((uint64_t)m)) || (m == 2 && is_pow2((uint64_t)n)));
  const bool forward = mode != CUMPSGEMM_DRY_RUN && !gate_shape && (forwards_to_hipblas(mode) || device_scalars);
  // One intercepted call at a time from here on: the process-wide handle, the
  // record of the last call and the stream it runs on are shared by all host
  // threads.  (The rule hook above runs outside the lock: it may call back
  // into user code.  Recursive, in case the vendor library's own GEMM entry
  // points call each other through the dynamic symbol table.)
  static std::recursive_mutex call_mutex;
  std::unique_lock<std::recursive_mutex> lock(call_mutex);
  // a dry run only logs: it must not need a device, so the handle is created
  // after it; a forwarded call uses the handle only if there is one already
  // (statistics of C are switched on through a handle)
  cuMpSGEMM_handle_t h =
      (mode == CUMPSGEMM_DRY_RUN || forward) ? g_handles[current_device()] : global_handle();

  if (env_flag("CUMPSGEMM_INFO", false)) {
    log_info(std::string(func_name) + " op=(" + op_str(op_A) + ", " + op_str(op_B) + "), shape=(" +
             std::to_string(m) + ", " + std::to_string(n) + ", " + std::to_string(k) + ")" +
             (batched ? ", batch=" + std::to_string(batch) : std::string()) +
             ", mode=" + cuMpSGEMM_get_compute_mode_string(mode) + "[" +
             (g_hijack_mode == DYNAMIC_MODE ? "dynamic" : "static") +
             "][exp_stats:" + ((h && h->exp_stats_enabled) ? "1" : "0") + "]");
  }
  g_last.from_call = true;
  g_last.func_name = func_name;
  g_last.op_A = op_A;
  g_last.op_B = op_B;
  g_last.m = m;
  g_last.n = n;
  g_last.k = k;
  g_last.batch = batched ? batch : 1;
  g_last.mode = mode;

  if (mode == CUMPSGEMM_DRY_RUN) return HIPBLAS_STATUS_SUCCESS;

  if (forward) {
    // The vendor library does this call; unless statistics of C are wanted
    // nothing of this library is involved, so other threads' calls need not wait.
    const bool stats_of_c = h != nullptr && h->exp_stats_enabled;
    if (!stats_of_c) lock.unlock();
    if (device_scalars && !forwards_to_hipblas(mode)) {
      log_warning("alpha / beta are in device memory (HIPBLAS_POINTER_MODE_DEVICE): forwarding to hipBLAS");
      log_info(" +---> forwarded to hipBLAS (device pointer mode)");
    }
    CulipScope prof(culip_enabled(), caller_stream(hb), func_name, op_A, op_B, m, n, k, batched, batch);
    const hipblasStatus_t st =
        batched ? forward_gemm_sb<T>(hb, op_A, op_B, m, n, k, alpha, a, lda, sa, b, ldb, sb, beta,
                                     c, ldc, sc, batch)
                : forward_gemm<T>(hb, op_A, op_B, m, n, k, alpha, a, lda, b, ldb, beta, c, ldc);
    if (stats_of_c) {
      // statistics of the result, as the reference does for forwarded calls
      // (src/cumpsgemm_cublas.cu:420-425); the statistics take a 32-bit stride
      if (batched && (sc < 0 || sc > 0xffffffffll)) {
        log_warning("exp_stats of C skipped: the batch stride does not fit 32 bits");
      } else {
        cuMpSGEMM_set_stream(h, caller_stream(hb));
        cumpsgemm::exp_stats_ext<T>(h, (unsigned)m, (unsigned)n, c, (unsigned)ldc,
                                    batched ? (unsigned)batch : 1u, batched ? (unsigned)sc : 0u);
      }
    }
    return st;
  }
  if (h == nullptr) return HIPBLAS_STATUS_NOT_INITIALIZED;

  if (batched && (sa < 0 || sb < 0 || sc < 0)) {
    // not something this library's kernels address; the vendor library decides what it means
    log_warning("negative batch stride: forwarding to hipBLAS");
    return forward_gemm_sb<T>(hb, op_A, op_B, m, n, k, alpha, a, lda, sa, b, ldb, sb, beta, c, ldc, sc, batch);
  }
  // kernels of this library run on the caller's stream so that ordering with
  // the application's other work is preserved
  cuMpSGEMM_set_stream(h, caller_stream(hb));
  const uint64_t nb = batched ? (uint64_t)batch : 1;
  const uint64_t usa = batched ? (uint64_t)sa : 0, usb = batched ? (uint64_t)sb : 0,
                 usc = batched ? (uint64_t)sc : 0;

  const bool culip = culip_enabled();
  const std::string sc_prefix = std::is_same<T, float>::value ? "s" : "c";
  const hipStream_t cstream = caller_stream(hb);

  if (mx2x2_enabled() && n == 2 && k == 2 && is_pow2((uint64_t)m)) {
    CulipScope prof(culip, cstream, sc_prefix + (batched ? "gemm_strided_batch_Mx2x2" : "gemm_Mx2x2"), op_A,
                    op_B, m, n, k, batched, batch);
    log_info(" +---> gemm_Mx2x2");
    if constexpr (std::is_same<T, float>::value)
      return cuMpSGEMM_sgemm_Mx2x2(h, op_A, op_B, m, alpha, a, lda, usa, b, ldb, usb, beta, c, ldc,
                                   usc, nb);
    else
      return cuMpSGEMM_cgemm_Mx2x2(h, op_A, op_B, m, alpha, a, lda, usa, b, ldb, usb, beta, c, ldc,
                                   usc, nb);
  }
  if (mx2x2_enabled() && m == 2 && k == 2 && is_pow2((uint64_t)n)) {
    CulipScope prof(culip, cstream, sc_prefix + (batched ? "gemm_strided_batch_2xNx2" : "gemm_2xNx2"), op_A,
                    op_B, m, n, k, batched, batch);
    log_info(" +---> gemm_2xNx2");
    if constexpr (std::is_same<T, float>::value)
      return cuMpSGEMM_sgemm_2xNx2(h, op_A, op_B, n, alpha, a, lda, usa, b, ldb, usb, beta, c, ldc,
                                   usc, nb);
    else
      return cuMpSGEMM_cgemm_2xNx2(h, op_A, op_B, n, alpha, a, lda, usa, b, ldb, usb, beta, c, ldc,
                                   usc, nb);
  }

  if (mode == CUMPSGEMM_FP32_SIMT || mode == CUMPSGEMM_UNDEFINED) {
    log_error(std::string("mode ") + cuMpSGEMM_get_compute_mode_string(mode) +
              " is not executable; forwarding to hipBLAS");
    return batched ? forward_gemm_sb<T>(hb, op_A, op_B, m, n, k, alpha, a, lda, sa, b, ldb, sb,
                                        beta, c, ldc, sc, batch)
                   : forward_gemm<T>(hb, op_A, op_B, m, n, k, alpha, a, lda, b, ldb, beta, c, ldc);
  }
  CulipScope prof(culip, cstream,
                  sc_prefix + (batched ? "gemm_stridedBatch_" : "gemm_") +
                      cuMpSGEMM_get_compute_mode_string(mode),
                  op_A, op_B, m, n, k, batched, batch);
  // unless restore_AB is off the scaled modes leave A and B untouched
  return gemm_pipeline<T>(h, op_A, op_B, m, n, k, alpha, const_cast<T *>(a), lda, usa,
                          const_cast<T *>(b), ldb, usb, beta, c, ldc, usc, nb, batched, mode,
                          g_restore_AB, nullptr);
}
} // namespace

// ---- intercepted hipBLAS symbols (prototypes of ROCm 7.2 hipblas.h) ----------
extern "C" {
hipblasStatus_t hipblasSgemm(hipblasHandle_t handle, hipblasOperation_t transA,
                             hipblasOperation_t transB, int m, int n, int k, const float *alpha,
                             const float *AP, int lda, const float *BP, int ldb, const float *beta,
                             float *CP, int ldc) {
  return hijack_core<float>(__func__, handle, transA, transB, m, n, k, alpha, AP, lda, 0, BP, ldb,
                            0, beta, CP, ldc, 0, 1, false);
}

hipblasStatus_t hipblasCgemm(hipblasHandle_t handle, hipblasOperation_t transA,
                             hipblasOperation_t transB, int m, int n, int k,
                             const hipComplex *alpha, const hipComplex *AP, int lda,
                             const hipComplex *BP, int ldb, const hipComplex *beta, hipComplex *CP,
                             int ldc) {
  return hijack_core<hipComplex>(__func__, handle, transA, transB, m, n, k, alpha, AP, lda, 0, BP,
                                 ldb, 0, beta, CP, ldc, 0, 1, false);
}

hipblasStatus_t hipblasSgemmStridedBatched(hipblasHandle_t handle, hipblasOperation_t transA,
                                           hipblasOperation_t transB, int m, int n, int k,
                                           const float *alpha, const float *AP, int lda,
                                           long long strideA, const float *BP, int ldb,
                                           long long strideB, const float *beta, float *CP,
                                           int ldc, long long strideC, int batchCount) {
  return hijack_core<float>(__func__, handle, transA, transB, m, n, k, alpha, AP, lda, strideA, BP,
                            ldb, strideB, beta, CP, ldc, strideC, batchCount, true);
}

hipblasStatus_t hipblasCgemmStridedBatched(hipblasHandle_t handle, hipblasOperation_t transA,
                                           hipblasOperation_t transB, int m, int n, int k,
                                           const hipComplex *alpha, const hipComplex *AP, int lda,
                                           long long strideA, const hipComplex *BP, int ldb,
                                           long long strideB, const hipComplex *beta,
                                           hipComplex *CP, int ldc, long long strideC,
                                           int batchCount) {
  return hijack_core<hipComplex>(__func__, handle, transA, transB, m, n, k, alpha, AP, lda,
                                 strideA, BP, ldb, strideB, beta, CP, ldc, strideC, batchCount,
                                 true);
}

// Only all-FP32-real or all-FP32-complex calls are taken over; every other
// type combination goes to hipBLAS untouched (reference :1050-1108).
hipblasStatus_t hipblasGemmEx(hipblasHandle_t handle, hipblasOperation_t transA,
                              hipblasOperation_t transB, int m, int n, int k, const void *alpha,
                              const void *A, hipDataType aType, int lda, const void *B,
                              hipDataType bType, int ldb, const void *beta, void *C,
                              hipDataType cType, int ldc, hipblasComputeType_t computeType,
                              hipblasGemmAlgo_t algo) {
  if (aType == HIP_R_32F && bType == HIP_R_32F && cType == HIP_R_32F) {
    return hijack_core<float>(__func__, handle, transA, transB, m, n, k,
                              static_cast<const float *>(alpha), static_cast<const float *>(A),
                              lda, 0, static_cast<const float *>(B), ldb, 0,
                              static_cast<const float *>(beta), static_cast<float *>(C), ldc, 0, 1,
                              false);
  }
  if (aType == HIP_C_32F && bType == HIP_C_32F && cType == HIP_C_32F) {
    return hijack_core<hipComplex>(
        __func__, handle, transA, transB, m, n, k, static_cast<const hipComplex *>(alpha),
        static_cast<const hipComplex *>(A), lda, 0, static_cast<const hipComplex *>(B), ldb, 0,
        static_cast<const hipComplex *>(beta), static_cast<hipComplex *>(C), ldc, 0, 1, false);
  }
  using fn_t = hipblasStatus_t (*)(hipblasHandle_t, hipblasOperation_t, hipblasOperation_t, int,
                                   int, int, const void *, const void *, hipDataType, int,
                                   const void *, hipDataType, int, const void *, void *,
                                   hipDataType, int, hipblasComputeType_t, hipblasGemmAlgo_t);
  static fn_t fn = reinterpret_cast<fn_t>(real_symbol("hipblasGemmEx"));
  if (fn == nullptr) return HIPBLAS_STATUS_NOT_SUPPORTED;
  return fn(handle, transA, transB, m, n, k, alpha, A, aType, lda, B, bType, ldb, beta, C, cType,
            ldc, computeType, algo);
}

hipblasStatus_t hipblasGemmStridedBatchedEx(
    hipblasHandle_t handle, hipblasOperation_t transA, hipblasOperation_t transB, int m, int n,
    int k, const void *alpha, const void *A, hipDataType aType, int lda, hipblasStride strideA,
    const void *B, hipDataType bType, int ldb, hipblasStride strideB, const void *beta, void *C,
    hipDataType cType, int ldc, hipblasStride strideC, int batchCount,
    hipblasComputeType_t computeType, hipblasGemmAlgo_t algo) {
  if (aType == HIP_R_32F && bType == HIP_R_32F && cType == HIP_R_32F) {
    return hijack_core<float>(__func__, handle, transA, transB, m, n, k,
                              static_cast<const float *>(alpha), static_cast<const float *>(A),
                              lda, strideA, static_cast<const float *>(B), ldb, strideB,
                              static_cast<const float *>(beta), static_cast<float *>(C), ldc,
                              strideC, batchCount, true);
  }
  if (aType == HIP_C_32F && bType == HIP_C_32F && cType == HIP_C_32F) {
    return hijack_core<hipComplex>(
        __func__, handle, transA, transB, m, n, k, static_cast<const hipComplex *>(alpha),
        static_cast<const hipComplex *>(A), lda, strideA, static_cast<const hipComplex *>(B), ldb,
        strideB, static_cast<const hipComplex *>(beta), static_cast<hipComplex *>(C), ldc, strideC,
        batchCount, true);
  }
  using fn_t = hipblasStatus_t (*)(hipblasHandle_t, hipblasOperation_t, hipblasOperation_t, int,
                                   int, int, const void *, const void *, hipDataType, int,
                                   hipblasStride, const void *, hipDataType, int, hipblasStride,
                                   const void *, void *, hipDataType, int, hipblasStride, int,
                                   hipblasComputeType_t, hipblasGemmAlgo_t);
  static fn_t fn = reinterpret_cast<fn_t>(real_symbol("hipblasGemmStridedBatchedEx"));
  if (fn == nullptr) return HIPBLAS_STATUS_NOT_SUPPORTED;
  return fn(handle, transA, transB, m, n, k, alpha, A, aType, lda, strideA, B, bType, ldb, strideB,
            beta, C, cType, ldc, strideC, batchCount, computeType, algo);
}
} // extern "C"

// ---- hijack_control -----------------------------------------------------------
namespace cumpsgemm {
namespace hijack_control {
cuMpSGEMM_handle_t get_internal_global_handle() { return global_handle(); }
void set_compute_mode(cuMpSGEMM_compute_mode_t mode) {
  if (mode == CUMPSGEMM_FP32_SIMT)
    throw std::runtime_error("CUMPSGEMM_FP32_SIMT mode is currently not supported.");
  g_static_mode = mode;
  g_hijack_mode = STATIC_MODE;
}
void unset_compute_mode() { g_hijack_mode = DYNAMIC_MODE; }
void enable_custom_gemm_Mx2x2() { g_mx2x2_enabled = true; }
void disable_custom_gemm_Mx2x2() { g_mx2x2_enabled = false; }
void reset_exp_stats_buffer_id() { cumpsgemm::reset_exp_stats_buffer_id(global_handle()); }
void set_exp_stats_params(float ignore_threshold, float underflow_threshold,
                          float underflow_tolerance_rate) {
  log_info("AUTO config: ignore_threshold=" + sci(ignore_threshold) + " @" + __func__);
  log_info("AUTO config: underflow_threshold=" + sci(underflow_threshold) + " @" + __func__);
  log_info("AUTO config: underflow_tolerance_rate=" + sci(underflow_tolerance_rate) + " @" +
           __func__);
  cumpsgemm::set_exp_stats_params(global_handle(), ignore_threshold, underflow_threshold,
                                  underflow_tolerance_rate);
}
void enable_restoring_AB_after_scaling() {
  g_restore_AB = true;
  log_info(std::string("AUTO config: restore_AB_scaling=True @") + __func__);
}
void disable_restoring_AB_after_scaling() {
  g_restore_AB = false;
  log_info(std::string("AUTO config: restore_AB_scaling=False @") + __func__);
}
std::string get_last_called_function_str() { return last_called_text(); }
void set_last_called_function_str(const std::string func_str) { set_last_called_text(func_str); }
void clear_last_called_function_str() { set_last_called_text(std::string()); }
bool is_library_loaded() { return true; }
void set_control_function(const control_function_t control_function) {
  g_control_func = control_function;
}
void unset_control_function() { g_control_func = nullptr; }
} // namespace hijack_control
} // namespace cumpsgemm

extern "C" {
cuMpSGEMM_handle_t cuMpSGEMM_hijack_get_internal_global_handle(void) { return global_handle(); }
int cuMpSGEMM_hijack_set_compute_mode(int mode) {
  try {
    cumpsgemm::hijack_control::set_compute_mode((cuMpSGEMM_compute_mode_t)mode);
  } catch (const std::exception &) {
    return -1;
  }
  return 0;
}
void cuMpSGEMM_hijack_unset_compute_mode(void) { cumpsgemm::hijack_control::unset_compute_mode(); }
void cuMpSGEMM_hijack_enable_custom_gemm_Mx2x2(void) { g_mx2x2_enabled = true; }
void cuMpSGEMM_hijack_disable_custom_gemm_Mx2x2(void) { g_mx2x2_enabled = false; }
void cuMpSGEMM_hijack_set_restore_AB(int enable) { g_restore_AB = enable != 0; }
size_t cuMpSGEMM_hijack_get_last_called_function_str(char *buf, size_t buf_len) {
  if (buf != nullptr && buf_len > 0) {
    std::snprintf(buf, buf_len, "%s", last_called_text().c_str());
  }
  return last_called_text().size();
}
void cuMpSGEMM_hijack_clear_last_called_function_str(void) { set_last_called_text(std::string()); }
int cuMpSGEMM_hijack_is_library_loaded(void) { return 1; }
void cuMpSGEMM_hijack_set_last_called_function_str(const char *str) {
  set_last_called_text((str != nullptr) ? str : "");
}
void cuMpSGEMM_hijack_reset_exp_stats_buffer_id(void) {
  cumpsgemm::hijack_control::reset_exp_stats_buffer_id();
}
void cuMpSGEMM_hijack_set_exp_stats_params(float ignore_threshold, float underflow_threshold,
                                           float underflow_tolerance_rate) {
  cumpsgemm::hijack_control::set_exp_stats_params(ignore_threshold, underflow_threshold,
                                                  underflow_tolerance_rate);
}
void cuMpSGEMM_hijack_set_control_function(cuMpSGEMM_control_function_t fn) {
  if (fn == nullptr) {
    cumpsgemm::hijack_control::unset_control_function();
    return;
  }
  cumpsgemm::hijack_control::set_control_function(
      [fn](const int op_A, const int op_B, const unsigned m, const unsigned n, const unsigned k) {
        return (cuMpSGEMM_compute_mode_t)fn(op_A, op_B, m, n, k);
      });
}
int cuMpSGEMM_hijack_query_compute_mode(const char *func_name, int op_A, int op_B, unsigned m,
                                        unsigned n, unsigned k) {
  return (int)query_mode(func_name, nullptr, (hipblasOperation_t)op_A, (hipblasOperation_t)op_B, m,
                         n, k);
}
}
