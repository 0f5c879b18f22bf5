// C++ client of the library's public headers, written the way a user of the
// reference's C++ API writes it (reference README.md "Usage", test/main.cu):
// create a handle, run gemm<float> / gemm<hipComplex> / gemm_stridedBatch,
// the statistics and scaling calls, and check every result on the host in
// double precision.  Built against include/ and linked with libcumpsgemm.so by
// tests/native/Makefile; run by tests/test_gpu_native_api.py.  Prints
//   RESULT <name> <value>
// lines and DONE.
#include <cumpsgemm/cumpsgemm.hpp>

#include <hip/hip_runtime.h>

#include <cmath>
#include <complex>
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <vector>

#define CHECK_HIP(x)                                                                      \
  do {                                                                                    \
    hipError_t e_ = (x);                                                                  \
    if (e_ != hipSuccess) {                                                               \
      std::printf("HIP error %s at %s:%d\n", hipGetErrorString(e_), __FILE__, __LINE__); \
      std::exit(2);                                                                       \
    }                                                                                     \
  } while (0)

static uint64_t mix(uint64_t x) {
  x += 0x9E3779B97F4A7C15ull;
  x = (x ^ (x >> 30)) * 0xBF58476D1CE4E5B9ull;
  x = (x ^ (x >> 27)) * 0x94D049BB133111EBull;
  return x ^ (x >> 31);
}
static float unif(uint64_t seed, uint64_t i) {
  return (float)((double)(mix(seed * 0x100000000ull + i) >> 40) / (1 << 24) * 2.0 - 1.0);
}

template <class T> struct dev_buf {
  T *p = nullptr;
  size_t n;
  explicit dev_buf(size_t count) : n(count) { CHECK_HIP(hipMalloc(&p, n * sizeof(T))); }
  ~dev_buf() { (void)hipFree(p); }
  void up(const std::vector<T> &h) { CHECK_HIP(hipMemcpy(p, h.data(), n * sizeof(T), hipMemcpyHostToDevice)); }
  std::vector<T> down() const {
    std::vector<T> h(n);
    CHECK_HIP(hipMemcpy(h.data(), p, n * sizeof(T), hipMemcpyDeviceToHost));
    return h;
  }
};

int main() {
  hipStream_t stream;
  CHECK_HIP(hipStreamCreate(&stream));
  cumpsgemm::handle_t handle = nullptr;
  cumpsgemm::create(handle); // returns nothing, as in the reference
  if (handle == nullptr) return 3;
  cumpsgemm::set_stream(handle, stream);

  // ---- gemm<float>, op T x N, alpha / beta, module id ----
  {
    const uint64_t m = 300, n = 200, k = 170;
    std::vector<float> a(k * m), b(k * n), c(m * n);
    for (size_t i = 0; i < a.size(); i++) a[i] = unif(1, i);
    for (size_t i = 0; i < b.size(); i++) b[i] = unif(2, i);
    for (size_t i = 0; i < c.size(); i++) c[i] = unif(3, i);
    dev_buf<float> da(a.size()), db(b.size()), dc(c.size());
    da.up(a), db.up(b), dc.up(c);
    const float alpha = 1.5f, beta = -0.5f;
    unsigned module_id = 12345;
    const auto st = cumpsgemm::gemm<float>(handle, HIPBLAS_OP_T, HIPBLAS_OP_N, m, n, k, &alpha, da.p, k, db.p, k,
                                           &beta, dc.p, m, CUMPSGEMM_FP16TCEC, &module_id);
    CHECK_HIP(hipStreamSynchronize(stream));
    const auto got = dc.down();
    double num = 0, den = 0;
    for (uint64_t j = 0; j < n; j++)
      for (uint64_t i = 0; i < m; i++) {
        double s = 0;
        for (uint64_t l = 0; l < k; l++) s += (double)a[i * k + l] * (double)b[j * k + l];
        const double ref = alpha * s + beta * (double)c[j * m + i];
        num += (ref - got[j * m + i]) * (ref - got[j * m + i]);
        den += ref * ref;
      }
    std::printf("RESULT sgemm_status %d\nRESULT sgemm_relerr %.3e\nRESULT sgemm_module %u\n", (int)st,
                std::sqrt(num / den), module_id);
  }
  // ---- gemm_stridedBatch<hipComplex>, op N x C ----
  {
    const uint64_t m = 96, n = 80, k = 72, batch = 3;
    std::vector<hipComplex> a(m * k * batch), b(n * k * batch), c(m * n * batch);
    for (size_t i = 0; i < a.size(); i++) a[i] = make_hipComplex(unif(4, 2 * i), unif(4, 2 * i + 1));
    for (size_t i = 0; i < b.size(); i++) b[i] = make_hipComplex(unif(5, 2 * i), unif(5, 2 * i + 1));
    dev_buf<hipComplex> da(a.size()), db(b.size()), dc(c.size());
    da.up(a), db.up(b);
    const hipComplex alpha = make_hipComplex(1.f, 0.f), beta = make_hipComplex(0.f, 0.f);
    const auto st = cumpsgemm::gemm_stridedBatch<hipComplex>(handle, HIPBLAS_OP_N, HIPBLAS_OP_C, m, n, k, &alpha,
                                                             da.p, m, m * k, db.p, n, n * k, &beta, dc.p, m,
                                                             m * n, batch, CUMPSGEMM_TF32TCEC);
    CHECK_HIP(hipStreamSynchronize(stream));
    const auto got = dc.down();
    double num = 0, den = 0;
    for (uint64_t t = 0; t < batch; t++)
      for (uint64_t j = 0; j < n; j++)
        for (uint64_t i = 0; i < m; i++) {
          std::complex<double> s = 0;
          for (uint64_t l = 0; l < k; l++) {
            const hipComplex x = a[t * m * k + l * m + i], y = b[t * n * k + l * n + j];
            s += std::complex<double>(x.x, x.y) * std::conj(std::complex<double>(y.x, y.y));
          }
          const hipComplex g = got[t * m * n + j * m + i];
          num += std::norm(s - std::complex<double>(g.x, g.y));
          den += std::norm(s);
        }
    std::printf("RESULT cgemm_batch_status %d\nRESULT cgemm_batch_relerr %.3e\n", (int)st, std::sqrt(num / den));
  }
  // ---- statistics, scaling round trip, launch flag ----
  {
    const unsigned m = 500, n = 40;
    std::vector<float> x(m * n);
    size_t want_under = 0;
    float want_max = 0;
    for (size_t i = 0; i < x.size(); i++) {
      x[i] = unif(6, i) * ((i % 7 == 0) ? 1e-6f : 0.01f);
      if (std::fabs(x[i]) < 1.0f / 32768.0f) want_under++;
      want_max = std::fmax(want_max, std::fabs(x[i]));
    }
    dev_buf<float> dx(x.size());
    dx.up(x);
    const unsigned id = cumpsgemm::exp_stats_ext<float>(handle, m, n, dx.p, m);
    const auto counts = cumpsgemm::get_exp_stats(handle, id); // {underflow, total} of the deciding stage
    const float max_exp = cumpsgemm::get_max_exp(handle, id);
    const auto level = cumpsgemm::get_exp_stats_compute_mode_level(handle, id);
    int e;
    std::frexp(want_max, &e);
    std::printf("RESULT stats_max_ok %d\n", max_exp == std::ldexp(1.0f, e - 1) ? 1 : 0);
    std::printf("RESULT stats_stage1_underflow_seen %d\n", want_under > 0 ? 1 : 0);
    std::printf("RESULT stats_level %d\nRESULT stats_total %zu\n", (int)level, counts.second);

    const unsigned flag = cumpsgemm::get_next_dynamic_launch_buffer_id(handle);
    cumpsgemm::set_dynamic_launch_buffer_by_exp_stats(handle, flag, id, id);
    const auto ab = cumpsgemm::get_dynamic_launch_scaling_mode_AB(handle, flag);
    std::printf("RESULT flag_mode %d\nRESULT flag_scale %d%d\n",
                (int)cumpsgemm::get_dynamic_launch_gemm_compute_mode(handle, flag), ab.first, ab.second);
    cumpsgemm::scale_A<float>(handle, id, flag, m, n, dx.p, m);
    const auto scaled = dx.down();
    cumpsgemm::reset_scale_A<float>(handle, id, flag, m, n, dx.p, m);
    CHECK_HIP(hipStreamSynchronize(stream));
    const auto back = dx.down();
    bool same = true, moved = false;
    for (size_t i = 0; i < x.size(); i++) {
      same = same && (back[i] == x[i]);
      moved = moved || (scaled[i] != x[i]);
    }
    std::printf("RESULT scale_roundtrip %d\nRESULT scale_applied %d\n", same ? 1 : 0, moved ? 1 : 0);
  }
  cumpsgemm::destroy(handle);
  CHECK_HIP(hipStreamDestroy(stream));
  std::printf("DONE\n");
  return 0;
}
