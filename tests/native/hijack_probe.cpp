// Stand-alone hipBLAS client used by tests/test_gpu_hijack.py.  It is linked
// against the real libhipblas.so; when run under LD_PRELOAD=libcumpsgemm.so the
// six GEMM entry points below resolve to the interposer instead.  For every
// call it prints one line:  RESULT <name> status=<s> relerr=<e>
// where relerr is the relative Frobenius error over sampled entries of C
// against a double-precision evaluation of the same inputs on the host.
#include <hip/hip_complex.h>
#include <hip/hip_runtime.h>
#include <hipblas/hipblas.h>

#include <cmath>
#include <complex>
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <thread>
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
  explicit dev_buf(size_t n) { CHECK_HIP(hipMalloc(&p, n * sizeof(T))); }
  ~dev_buf() { (void)hipFree(p); }
};

static void report(const char *name, hipblasStatus_t st, double num, double den) {
  std::printf("RESULT %s status=%d relerr=%.3e\n", name, (int)st, std::sqrt(num / (den > 0 ? den : 1)));
  std::fflush(stdout);
}

int main(int argc, char **argv) {
  // > 1024 so the default rule engages
  const char *env_n = std::getenv("PROBE_N");
  const int n = (argc > 1) ? std::atoi(argv[1]) : (env_n != nullptr ? std::atoi(env_n) : 1280);
  const int batch = 3;
  hipblasHandle_t hb;
  if (hipblasCreate(&hb) != HIPBLAS_STATUS_SUCCESS) {
    std::printf("hipblasCreate failed\n");
    return 2;
  }
  hipStream_t stream;
  CHECK_HIP(hipStreamCreate(&stream));
  hipblasSetStream(hb, stream);

  const size_t e = (size_t)n * n;
  std::vector<float> ha(e * batch), hb_(e * batch), hc(e * batch);
  for (size_t i = 0; i < e * batch; i++) {
    ha[i] = unif(1, i);
    hb_[i] = unif(2, i);
  }
  dev_buf<float> da(e * batch), db(e * batch), dc(e * batch);
  CHECK_HIP(hipMemcpyAsync(da.p, ha.data(), e * batch * 4, hipMemcpyHostToDevice, stream));
  CHECK_HIP(hipMemcpyAsync(db.p, hb_.data(), e * batch * 4, hipMemcpyHostToDevice, stream));
  const float one = 1.0f, zero = 0.0f;

  auto check_real = [&](const char *name, hipblasStatus_t st, int nb, bool trans_a) {
    CHECK_HIP(hipMemcpyAsync(hc.data(), dc.p, e * nb * 4, hipMemcpyDeviceToHost, stream));
    CHECK_HIP(hipStreamSynchronize(stream));
    double num = 0, den = 0;
    for (int b = 0; b < nb; b++)
      for (int s = 0; s < 400; s++) {
        const int i = (int)(mix(s * 2 + 11) % n), j = (int)(mix(s * 2 + 12) % n);
        double ref = 0;
        for (int p = 0; p < n; p++) {
          const double av = trans_a ? ha[b * e + p + (size_t)i * n] : ha[b * e + i + (size_t)p * n];
          ref += av * (double)hb_[b * e + p + (size_t)j * n];
        }
        const double d = ref - (double)hc[b * e + i + (size_t)j * n];
        num += d * d;
        den += ref * ref;
      }
    report(name, st, num, den);
  };

  CHECK_HIP(hipMemsetAsync(dc.p, 0, e * batch * 4, stream));
  hipblasStatus_t st = hipblasSgemm(hb, HIPBLAS_OP_N, HIPBLAS_OP_N, n, n, n, &one, da.p, n, db.p, n, &zero, dc.p, n);
  check_real("hipblasSgemm", st, 1, false);

  CHECK_HIP(hipMemsetAsync(dc.p, 0, e * batch * 4, stream));
  st = hipblasSgemm(hb, HIPBLAS_OP_T, HIPBLAS_OP_N, n, n, n, &one, da.p, n, db.p, n, &zero, dc.p, n);
  check_real("hipblasSgemm_TN", st, 1, true);

  CHECK_HIP(hipMemsetAsync(dc.p, 0, e * batch * 4, stream));
  st = hipblasSgemmStridedBatched(hb, HIPBLAS_OP_N, HIPBLAS_OP_N, n, n, n, &one, da.p, n, (long long)e, db.p, n,
                                  (long long)e, &zero, dc.p, n, (long long)e, batch);
  check_real("hipblasSgemmStridedBatched", st, batch, false);

  CHECK_HIP(hipMemsetAsync(dc.p, 0, e * batch * 4, stream));
  st = hipblasGemmEx(hb, HIPBLAS_OP_N, HIPBLAS_OP_N, n, n, n, &one, da.p, HIP_R_32F, n, db.p, HIP_R_32F, n, &zero,
                     dc.p, HIP_R_32F, n, HIPBLAS_COMPUTE_32F, HIPBLAS_GEMM_DEFAULT);
  check_real("hipblasGemmEx_f32", st, 1, false);

  CHECK_HIP(hipMemsetAsync(dc.p, 0, e * batch * 4, stream));
  st = hipblasGemmStridedBatchedEx(hb, HIPBLAS_OP_N, HIPBLAS_OP_N, n, n, n, &one, da.p, HIP_R_32F, n, (long long)e,
                                   db.p, HIP_R_32F, n, (long long)e, &zero, dc.p, HIP_R_32F, n, (long long)e, batch,
                                   HIPBLAS_COMPUTE_32F, HIPBLAS_GEMM_DEFAULT);
  check_real("hipblasGemmStridedBatchedEx_f32", st, batch, false);

  // zero-sized call: the interposer answers INVALID_VALUE, hipBLAS succeeds quietly
  st = hipblasSgemm(hb, HIPBLAS_OP_N, HIPBLAS_OP_N, 0, n, n, &one, da.p, n, db.p, n, &zero, dc.p, n);
  std::printf("RESULT zero_m status=%d relerr=0\n", (int)st);

  // alpha and beta in device memory: the interposer cannot read them on the host and must
  // leave the call to hipBLAS whatever the mode
  {
    dev_buf<float> dscal(2);
    const float hs[2] = {1.0f, 0.0f};
    CHECK_HIP(hipMemcpyAsync(dscal.p, hs, sizeof(hs), hipMemcpyHostToDevice, stream));
    CHECK_HIP(hipMemsetAsync(dc.p, 0, e * batch * 4, stream));
    hipblasSetPointerMode(hb, HIPBLAS_POINTER_MODE_DEVICE);
    st = hipblasSgemm(hb, HIPBLAS_OP_N, HIPBLAS_OP_N, n, n, n, dscal.p, da.p, n, db.p, n, dscal.p + 1, dc.p, n);
    hipblasSetPointerMode(hb, HIPBLAS_POINTER_MODE_HOST);
    check_real("hipblasSgemm_device_scalars", st, 1, false);
  }

  // complex: the float buffers reinterpreted as n/2-column complex matrices
  {
    const int nc = n / 2; // complex matrices are n x nc? keep them square: nc x nc
    const hipComplex cone = make_hipComplex(1.f, 0.f), czero = make_hipComplex(0.f, 0.f);
    const hipComplex *ca = reinterpret_cast<const hipComplex *>(da.p);
    const hipComplex *cb = reinterpret_cast<const hipComplex *>(db.p);
    hipComplex *cc = reinterpret_cast<hipComplex *>(dc.p);
    CHECK_HIP(hipMemsetAsync(dc.p, 0, e * batch * 4, stream));
    st = hipblasCgemm(hb, HIPBLAS_OP_C, HIPBLAS_OP_N, nc, nc, nc, &cone, ca, nc, cb, nc, &czero, cc, nc);
    CHECK_HIP(hipMemcpyAsync(hc.data(), dc.p, (size_t)nc * nc * 8, hipMemcpyDeviceToHost, stream));
    CHECK_HIP(hipStreamSynchronize(stream));
    auto A = reinterpret_cast<const std::complex<float> *>(ha.data());
    auto B = reinterpret_cast<const std::complex<float> *>(hb_.data());
    auto Cc = reinterpret_cast<const std::complex<float> *>(hc.data());
    double num = 0, den = 0;
    for (int s = 0; s < 400; s++) {
      const int i = (int)(mix(s * 2 + 31) % nc), j = (int)(mix(s * 2 + 32) % nc);
      std::complex<double> ref = 0;
      for (int p = 0; p < nc; p++)
        ref += std::conj(std::complex<double>(A[p + (size_t)i * nc])) * std::complex<double>(B[p + (size_t)j * nc]);
      num += std::norm(ref - std::complex<double>(Cc[i + (size_t)j * nc]));
      den += std::norm(ref);
    }
    report("hipblasCgemm_CN", st, num, den);

    // the other complex entry points: batches of nc x nc matrices, stride nc * nc
    const long long cs = (long long)nc * nc;
    auto check_cplx = [&](const char *name, hipblasStatus_t status, int nb) {
      CHECK_HIP(hipMemcpyAsync(hc.data(), dc.p, (size_t)cs * nb * 8, hipMemcpyDeviceToHost, stream));
      CHECK_HIP(hipStreamSynchronize(stream));
      double nu = 0, de = 0;
      for (int t = 0; t < nb; t++)
        for (int s = 0; s < 300; s++) {
          const int i = (int)(mix(s * 2 + 51) % nc), j = (int)(mix(s * 2 + 52) % nc);
          std::complex<double> ref = 0;
          for (int p = 0; p < nc; p++)
            ref += std::complex<double>(A[t * cs + i + (size_t)p * nc]) * std::complex<double>(B[t * cs + p + (size_t)j * nc]);
          nu += std::norm(ref - std::complex<double>(Cc[t * cs + i + (size_t)j * nc]));
          de += std::norm(ref);
        }
      report(name, status, nu, de);
    };
    CHECK_HIP(hipMemsetAsync(dc.p, 0, e * batch * 4, stream));
    st = hipblasCgemmStridedBatched(hb, HIPBLAS_OP_N, HIPBLAS_OP_N, nc, nc, nc, &cone, ca, nc, cs, cb, nc, cs, &czero,
                                    cc, nc, cs, 2);
    check_cplx("hipblasCgemmStridedBatched", st, 2);
    CHECK_HIP(hipMemsetAsync(dc.p, 0, e * batch * 4, stream));
    st = hipblasGemmEx(hb, HIPBLAS_OP_N, HIPBLAS_OP_N, nc, nc, nc, &cone, ca, HIP_C_32F, nc, cb, HIP_C_32F, nc, &czero,
                       cc, HIP_C_32F, nc, HIPBLAS_COMPUTE_32F, HIPBLAS_GEMM_DEFAULT);
    check_cplx("hipblasGemmEx_c32", st, 1);
    CHECK_HIP(hipMemsetAsync(dc.p, 0, e * batch * 4, stream));
    st = hipblasGemmStridedBatchedEx(hb, HIPBLAS_OP_N, HIPBLAS_OP_N, nc, nc, nc, &cone, ca, HIP_C_32F, nc, cs, cb,
                                     HIP_C_32F, nc, cs, &czero, cc, HIP_C_32F, nc, cs, 2, HIPBLAS_COMPUTE_32F,
                                     HIPBLAS_GEMM_DEFAULT);
    check_cplx("hipblasGemmStridedBatchedEx_c32", st, 2);
  }

  // a non-FP32 GemmEx must go to hipBLAS untouched whatever the mode
  {
    std::vector<uint16_t> h16(e, 0x3c00 /* 1.0 */);
    dev_buf<uint16_t> a16(e), b16(e);
    CHECK_HIP(hipMemcpyAsync(a16.p, h16.data(), e * 2, hipMemcpyHostToDevice, stream));
    CHECK_HIP(hipMemcpyAsync(b16.p, h16.data(), e * 2, hipMemcpyHostToDevice, stream));
    CHECK_HIP(hipMemsetAsync(dc.p, 0, e * 4, stream));
    st = hipblasGemmEx(hb, HIPBLAS_OP_N, HIPBLAS_OP_N, n, n, n, &one, a16.p, HIP_R_16F, n, b16.p, HIP_R_16F, n, &zero,
                       dc.p, HIP_R_32F, n, HIPBLAS_COMPUTE_32F, HIPBLAS_GEMM_DEFAULT);
    CHECK_HIP(hipMemcpyAsync(hc.data(), dc.p, e * 4, hipMemcpyDeviceToHost, stream));
    CHECK_HIP(hipStreamSynchronize(stream));
    double num = 0, den = 0;
    for (size_t i = 0; i < e; i += 997) {
      num += ((double)hc[i] - n) * ((double)hc[i] - n);
      den += (double)n * n;
    }
    report("hipblasGemmEx_f16_in", st, num, den);
  }

  // ---- gate-application shapes: (2^18 x 2) = (2^18 x 2) * (2 x 2) and its transpose-side twin ----
  if (std::getenv("PROBE_MX2X2") != nullptr) {
    const int L = 1 << 18;
    const hipComplex cone = make_hipComplex(1.f, 0.f), czero = make_hipComplex(0.f, 0.f);
    const hipComplex *ca = reinterpret_cast<const hipComplex *>(da.p); // L x 2 complex, ld L
    const hipComplex *cb = reinterpret_cast<const hipComplex *>(db.p); // 2 x 2 complex, ld 2
    hipComplex *cc = reinterpret_cast<hipComplex *>(dc.p);
    auto A = reinterpret_cast<const std::complex<float> *>(ha.data());
    auto B = reinterpret_cast<const std::complex<float> *>(hb_.data());
    auto Cc = reinterpret_cast<const std::complex<float> *>(hc.data());
    CHECK_HIP(hipMemsetAsync(dc.p, 0, (size_t)L * 2 * 8, stream));
    st = hipblasCgemm(hb, HIPBLAS_OP_N, HIPBLAS_OP_N, L, 2, 2, &cone, ca, L, cb, 2, &czero, cc, L);
    CHECK_HIP(hipMemcpyAsync(hc.data(), dc.p, (size_t)L * 2 * 8, hipMemcpyDeviceToHost, stream));
    CHECK_HIP(hipStreamSynchronize(stream));
    double num = 0, den = 0;
    for (int j = 0; j < 2; j++)
      for (int i = 0; i < L; i += 7) {
        const std::complex<double> ref = std::complex<double>(A[i]) * std::complex<double>(B[2 * j]) +
                                         std::complex<double>(A[i + L]) * std::complex<double>(B[2 * j + 1]);
        num += std::norm(ref - std::complex<double>(Cc[i + (size_t)j * L]));
        den += std::norm(ref);
      }
    report("cgemm_Mx2x2", st, num, den);
    // real, (2 x L) = (2 x 2) * (2 x L)
    CHECK_HIP(hipMemsetAsync(dc.p, 0, (size_t)L * 2 * 4, stream));
    st = hipblasSgemm(hb, HIPBLAS_OP_N, HIPBLAS_OP_N, 2, L, 2, &one, da.p, 2, db.p, 2, &zero, dc.p, 2);
    CHECK_HIP(hipMemcpyAsync(hc.data(), dc.p, (size_t)L * 2 * 4, hipMemcpyDeviceToHost, stream));
    CHECK_HIP(hipStreamSynchronize(stream));
    num = den = 0;
    for (int j = 0; j < L; j += 5)
      for (int i = 0; i < 2; i++) {
        const double ref = (double)ha[i] * hb_[2 * (size_t)j] + (double)ha[i + 2] * hb_[2 * (size_t)j + 1];
        const double d = ref - (double)hc[i + 2 * (size_t)j];
        num += d * d;
        den += ref * ref;
      }
    report("sgemm_2xNx2", st, num, den);
  }

  // ---- several host threads, each with its own hipBLAS handle and stream ----
  // (PROBE_THREADS=<count>: every thread repeats two products of different
  // shapes and compares each result with the one the main thread computed)
  if (const char *pt = std::getenv("PROBE_THREADS")) {
    const int nthreads = std::atoi(pt), reps = 12;
    const int n2 = n - 256; // a second shape, so that consecutive calls differ in their workspace use
    std::vector<float> ref1(e), ref2((size_t)n2 * n2);
    CHECK_HIP(hipMemsetAsync(dc.p, 0, e * 4, stream));
    st = hipblasSgemm(hb, HIPBLAS_OP_N, HIPBLAS_OP_T, n, n, n, &one, da.p, n, db.p, n, &zero, dc.p, n);
    CHECK_HIP(hipMemcpyAsync(ref1.data(), dc.p, e * 4, hipMemcpyDeviceToHost, stream));
    st = hipblasSgemm(hb, HIPBLAS_OP_N, HIPBLAS_OP_T, n2, n2, n2, &one, da.p, n, db.p, n, &zero, dc.p, n2);
    CHECK_HIP(hipMemcpyAsync(ref2.data(), dc.p, (size_t)n2 * n2 * 4, hipMemcpyDeviceToHost, stream));
    CHECK_HIP(hipStreamSynchronize(stream));
    std::vector<long> bad(nthreads, 0);
    std::vector<int> status(nthreads, 0);
    std::vector<std::thread> pool;
    for (int t = 0; t < nthreads; t++) {
      pool.emplace_back([&, t]() {
        hipblasHandle_t hbt;
        hipStream_t st_t;
        if (hipblasCreate(&hbt) != HIPBLAS_STATUS_SUCCESS || hipStreamCreate(&st_t) != hipSuccess) {
          status[t] = -1;
          return;
        }
        hipblasSetStream(hbt, st_t);
        dev_buf<float> dct(e);
        std::vector<float> got(e);
        for (int r = 0; r < reps; r++) {
          const bool big = ((r + t) % 2) == 0;
          const int nn = big ? n : n2;
          const size_t ee = (size_t)nn * nn;
          (void)hipMemsetAsync(dct.p, 0, ee * 4, st_t);
          const hipblasStatus_t s2 =
              hipblasSgemm(hbt, HIPBLAS_OP_N, HIPBLAS_OP_T, nn, nn, nn, &one, da.p, n, db.p, n, &zero, dct.p, nn);
          if (s2 != HIPBLAS_STATUS_SUCCESS) status[t] = (int)s2;
          (void)hipMemcpyAsync(got.data(), dct.p, ee * 4, hipMemcpyDeviceToHost, st_t);
          (void)hipStreamSynchronize(st_t);
          const std::vector<float> &ref = big ? ref1 : ref2;
          for (size_t i = 0; i < ee; i++) {
            if (std::fabs(got[i] - ref[i]) > 1e-3f) bad[t]++;
          }
        }
        hipblasDestroy(hbt);
        (void)hipStreamDestroy(st_t);
      });
    }
    for (auto &th : pool) th.join();
    long total_bad = 0;
    int worst = 0;
    for (int t = 0; t < nthreads; t++) {
      total_bad += bad[t];
      if (status[t] != 0) worst = status[t];
    }
    std::printf("RESULT threads status=%d relerr=%.3e\n", worst, (double)total_bad);
    std::fflush(stdout);
  }

  hipblasDestroy(hb);
  CHECK_HIP(hipStreamDestroy(stream));
  std::printf("DONE\n");
  return 0;
}
