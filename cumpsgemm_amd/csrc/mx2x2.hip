// HBM-streaming kernels for the gate-application shapes
//   C (M x 2) = alpha * op(A) (M x 2) * op(B) (2 x 2) + beta * C          ("Mx2x2")
//   C (2 x N) = alpha * op(A) (2 x 2) * op(B) (2 x N) + beta * C          ("2xNx2")
// The reference routes these shapes to the external cuGEMM-Mx2x2 kernels
// (src/cumpsgemm_cublas.cu:269-338, :647-722); semantics are those of a plain
// FP32 GEMM.  Both shapes reduce to one "long" operand X with L logical rows of
// 2 values, multiplied by a 2x2 matrix S held in registers:
//   Y[i][q] = alpha * (X[i][0] * S[0][q] + X[i][1] * S[1][q]) + beta * Y[i][q]
// Every element of X and Y is touched once: 16 bytes (real) or 32 bytes
// (complex) of HBM traffic per logical row, no reuse, no LDS.
#include "handle.hpp"
#include "utils.hpp"
#include <cumpsgemm/cumpsgemm_ext.h>
#include <type_traits>

namespace cumpsgemm_amd {
namespace {
constexpr int kBlock = 256;

struct cf {
  float x, y;
};
__device__ inline float mul(float a, float b) { return a * b; }
__device__ inline cf mul(cf a, cf b) { return {a.x * b.x - a.y * b.y, a.x * b.y + a.y * b.x}; }
__device__ inline float add(float a, float b) { return a + b; }
__device__ inline cf add(cf a, cf b) { return {a.x + b.x, a.y + b.y}; }
__device__ inline float cj(float a, bool) { return a; }
__device__ inline cf cj(cf a, bool c) { return {a.x, c ? -a.y : a.y}; }
__device__ inline bool is_zero(float a) { return a == 0.0f; }
__device__ inline bool is_zero(cf a) { return a.x == 0.0f && a.y == 0.0f; }

// Long operand addressing: element (i, p) at x[i * rs + p * cs]  (in elements).
template <class E> struct LongArgs {
  unsigned long long L;
  const E *x;
  unsigned long long x_rs, x_cs, x_bs;
  const E *s; // the 2x2 matrix, element (p, q) at s[p * s_rs + q * s_cs]
  unsigned long long s_rs, s_cs, s_bs;
  E *y;
  unsigned long long y_rs, y_cs, y_bs;
  E alpha, beta;
  unsigned conj_x, conj_s;
};

template <class E>
__global__ __launch_bounds__(kBlock) void long2x2_kernel(const LongArgs<E> a) {
  const unsigned b = blockIdx.y;
  const E *x = a.x + b * a.x_bs;
  const E *s = a.s + b * a.s_bs;
  E *y = a.y + b * a.y_bs;
  const E s00 = cj(s[0], a.conj_s), s01 = cj(s[a.s_cs], a.conj_s);
  const E s10 = cj(s[a.s_rs], a.conj_s), s11 = cj(s[a.s_rs + a.s_cs], a.conj_s);
  const bool bz = is_zero(a.beta);
  const unsigned long long gsz = (unsigned long long)gridDim.x * kBlock;
  unsigned long long i = (unsigned long long)blockIdx.x * kBlock + threadIdx.x;

  // streams of unit row stride: process 16 bytes per column per thread
  constexpr int V = 16 / sizeof(E); // rows per vector: 4 real, 2 complex
  struct alignas(16) vec_t { E e[V]; };
  const bool vec_ok = a.x_rs == 1 && a.y_rs == 1 && (a.L % V) == 0 &&
                      ((uintptr_t)x % 16) == 0 && ((uintptr_t)y % 16) == 0 &&
                      ((a.x_cs * sizeof(E)) % 16) == 0 && ((a.y_cs * sizeof(E)) % 16) == 0;
  if (vec_ok) {
    // Every byte is touched once: loads and stores bypass the caches' reuse
    // policy, and two vectors per column are in flight per thread.
    typedef float f4_t __attribute__((ext_vector_type(4)));
    union pack_t { f4_t f; vec_t v; };
    const unsigned long long nv = a.L / V;
    auto ldv = [](const E *p) { pack_t t; t.f = __builtin_nontemporal_load(reinterpret_cast<const f4_t *>(p)); return t.v; };
    auto stv = [](E *p, const vec_t &v) { pack_t t; t.v = v; __builtin_nontemporal_store(t.f, reinterpret_cast<f4_t *>(p)); };
    auto apply = [&](const vec_t &x0, const vec_t &x1, vec_t &y0, vec_t &y1) {
#pragma unroll
      for (int v = 0; v < V; v++) {
        const E u0 = cj(x0.e[v], a.conj_x), u1 = cj(x1.e[v], a.conj_x);
        E r0 = mul(a.alpha, add(mul(u0, s00), mul(u1, s10)));
        E r1 = mul(a.alpha, add(mul(u0, s01), mul(u1, s11)));
        if (!bz) {
          r0 = add(r0, mul(a.beta, y0.e[v]));
          r1 = add(r1, mul(a.beta, y1.e[v]));
        }
        y0.e[v] = r0;
        y1.e[v] = r1;
      }
    };
    for (; i + gsz < nv; i += 2 * gsz) {
      const unsigned long long j = i + gsz;
      const vec_t xa0 = ldv(x + i * V), xa1 = ldv(x + a.x_cs + i * V);
      const vec_t xb0 = ldv(x + j * V), xb1 = ldv(x + a.x_cs + j * V);
      vec_t ya0, ya1, yb0, yb1;
      if (!bz) {
        ya0 = ldv(y + i * V); ya1 = ldv(y + a.y_cs + i * V);
        yb0 = ldv(y + j * V); yb1 = ldv(y + a.y_cs + j * V);
      }
      apply(xa0, xa1, ya0, ya1);
      apply(xb0, xb1, yb0, yb1);
      stv(y + i * V, ya0); stv(y + a.y_cs + i * V, ya1);
      stv(y + j * V, yb0); stv(y + a.y_cs + j * V, yb1);
    }
    for (; i < nv; i += gsz) {
      const vec_t x0 = ldv(x + i * V), x1 = ldv(x + a.x_cs + i * V);
      vec_t y0, y1;
      if (!bz) {
        y0 = ldv(y + i * V);
        y1 = ldv(y + a.y_cs + i * V);
      }
      apply(x0, x1, y0, y1);
      stv(y + i * V, y0);
      stv(y + a.y_cs + i * V, y1);
    }
    return;
  }
  for (; i < a.L; i += gsz) {
    const E u0 = cj(x[i * a.x_rs], a.conj_x), u1 = cj(x[i * a.x_rs + a.x_cs], a.conj_x);
    E r0 = mul(a.alpha, add(mul(u0, s00), mul(u1, s10)));
    E r1 = mul(a.alpha, add(mul(u0, s01), mul(u1, s11)));
    E *y0 = y + i * a.y_rs, *y1 = y + i * a.y_rs + a.y_cs;
    if (!bz) {
      r0 = add(r0, mul(a.beta, *y0));
      r1 = add(r1, mul(a.beta, *y1));
    }
    *y0 = r0;
    *y1 = r1;
  }
}

template <class T> struct elem_of { using type = float; };
template <> struct elem_of<hipComplex> { using type = cf; };

// long_is_A: Mx2x2 (X = op(A), S = op(B), Y = C); else 2xNx2 expressed through
// the transposed product C^T = op(B)^T op(A)^T (X = op(B)^T, S = op(A)^T, Y = C^T).
template <class T>
hipblasStatus_t run_long2x2(cuMpSGEMM_handle *h, bool long_is_A, hipblasOperation_t op_A,
                            hipblasOperation_t op_B, uint64_t L, const T *alpha, const T *a,
                            uint64_t lda, uint64_t stridea, const T *b, uint64_t ldb,
                            uint64_t strideb, const T *beta, T *c, uint64_t ldc, uint64_t stridec,
                            uint64_t batch) {
  using E = typename elem_of<T>::type;
  if (h == nullptr || L == 0 || batch == 0 || batch > 65535) return HIPBLAS_STATUS_INVALID_VALUE;
  if (alpha == nullptr || beta == nullptr || a == nullptr || b == nullptr || c == nullptr)
    return HIPBLAS_STATUS_INVALID_VALUE; // (a null operand would fault on the device)
  LongArgs<E> args{};
  args.L = L;
  static_assert(sizeof(E) == sizeof(T), "element size");
  std::memcpy(&args.alpha, alpha, sizeof(E));
  std::memcpy(&args.beta, beta, sizeof(E));
  constexpr bool CPLX = std::is_same<T, hipComplex>::value;
  if (long_is_A) {
    args.x = reinterpret_cast<const E *>(a);
    // op(A)[i][p]: N -> a[i + p*lda]; T/C -> a[p + i*lda]
    args.x_rs = (op_A == HIPBLAS_OP_N) ? 1 : lda;
    args.x_cs = (op_A == HIPBLAS_OP_N) ? lda : 1;
    args.x_bs = stridea;
    args.conj_x = CPLX && op_A == HIPBLAS_OP_C;
    args.s = reinterpret_cast<const E *>(b);
    // op(B)[p][q]: N -> b[p + q*ldb]; T/C -> b[q + p*ldb]
    args.s_rs = (op_B == HIPBLAS_OP_N) ? 1 : ldb;
    args.s_cs = (op_B == HIPBLAS_OP_N) ? ldb : 1;
    args.s_bs = strideb;
    args.conj_s = CPLX && op_B == HIPBLAS_OP_C;
    args.y = reinterpret_cast<E *>(c);
    args.y_rs = 1;
    args.y_cs = ldc;
  } else {
    args.x = reinterpret_cast<const E *>(b);
    // X[j][p] = op(B)[p][j]: N -> b[p + j*ldb]; T/C -> b[j + p*ldb]
    args.x_rs = (op_B == HIPBLAS_OP_N) ? ldb : 1;
    args.x_cs = (op_B == HIPBLAS_OP_N) ? 1 : ldb;
    args.x_bs = strideb;
    args.conj_x = CPLX && op_B == HIPBLAS_OP_C;
    args.s = reinterpret_cast<const E *>(a);
    // S[p][r] = op(A)[r][p]: N -> a[r + p*lda]; T/C -> a[p + r*lda]
    args.s_rs = (op_A == HIPBLAS_OP_N) ? lda : 1;
    args.s_cs = (op_A == HIPBLAS_OP_N) ? 1 : lda;
    args.s_bs = stridea;
    args.conj_s = CPLX && op_A == HIPBLAS_OP_C;
    args.y = reinterpret_cast<E *>(c);
    // Y[j][r] = C[r][j] = c[r + j*ldc]
    args.y_rs = ldc;
    args.y_cs = 1;
  }
  args.y_bs = stridec;
  constexpr int V = 16 / sizeof(E);
  const uint64_t want = (L / V + kBlock - 1) / kBlock;
  // One vector per thread and column, no grid-stride loop: the workgroups in
  // flight then cover one compact window of the long operand.  With a capped
  // grid the concurrently streamed windows are a power-of-two stride apart and
  // fall on the same memory channels (measured: 4.5 TB/s capped at 16
  // workgroups per CU, 6.0 TB/s uncapped, M = 2^27).
  const unsigned grid = (unsigned)std::max<uint64_t>(1, std::min<uint64_t>(want, 0x7fffffffull));
  ProfileScope prof(h, long_is_A ? "gemm_Mx2x2" : "gemm_2xNx2");
  hipLaunchKernelGGL(long2x2_kernel<E>, dim3(grid, (unsigned)batch), dim3(kBlock), 0, h->stream,
                     args);
  return hipGetLastError() == hipSuccess ? HIPBLAS_STATUS_SUCCESS
                                         : HIPBLAS_STATUS_EXECUTION_FAILED;
}
} // namespace

} // namespace cumpsgemm_amd

using namespace cumpsgemm_amd;
extern "C" {
hipblasStatus_t cuMpSGEMM_sgemm_Mx2x2(cuMpSGEMM_handle_t handle, hipblasOperation_t op_A,
                                      hipblasOperation_t op_B, uint64_t m, const float *alpha,
                                      const float *a, uint64_t lda, uint64_t stridea,
                                      const float *b, uint64_t ldb, uint64_t strideb,
                                      const float *beta, float *c, uint64_t ldc, uint64_t stridec,
                                      uint64_t batch_count) {
  return run_long2x2<float>(handle, true, op_A, op_B, m, alpha, a, lda, stridea, b, ldb, strideb,
                            beta, c, ldc, stridec, batch_count);
}
hipblasStatus_t cuMpSGEMM_cgemm_Mx2x2(cuMpSGEMM_handle_t handle, hipblasOperation_t op_A,
                                      hipblasOperation_t op_B, uint64_t m, const hipComplex *alpha,
                                      const hipComplex *a, uint64_t lda, uint64_t stridea,
                                      const hipComplex *b, uint64_t ldb, uint64_t strideb,
                                      const hipComplex *beta, hipComplex *c, uint64_t ldc,
                                      uint64_t stridec, uint64_t batch_count) {
  return run_long2x2<hipComplex>(handle, true, op_A, op_B, m, alpha, a, lda, stridea, b, ldb,
                                 strideb, beta, c, ldc, stridec, batch_count);
}
hipblasStatus_t cuMpSGEMM_sgemm_2xNx2(cuMpSGEMM_handle_t handle, hipblasOperation_t op_A,
                                      hipblasOperation_t op_B, uint64_t n, const float *alpha,
                                      const float *a, uint64_t lda, uint64_t stridea,
                                      const float *b, uint64_t ldb, uint64_t strideb,
                                      const float *beta, float *c, uint64_t ldc, uint64_t stridec,
                                      uint64_t batch_count) {
  return run_long2x2<float>(handle, false, op_A, op_B, n, alpha, a, lda, stridea, b, ldb, strideb,
                            beta, c, ldc, stridec, batch_count);
}
hipblasStatus_t cuMpSGEMM_cgemm_2xNx2(cuMpSGEMM_handle_t handle, hipblasOperation_t op_A,
                                      hipblasOperation_t op_B, uint64_t n, const hipComplex *alpha,
                                      const hipComplex *a, uint64_t lda, uint64_t stridea,
                                      const hipComplex *b, uint64_t ldb, uint64_t strideb,
                                      const hipComplex *beta, hipComplex *c, uint64_t ldc,
                                      uint64_t stridec, uint64_t batch_count) {
  return run_long2x2<hipComplex>(handle, false, op_A, op_B, n, alpha, a, lda, stridea, b, ldb,
                                 strideb, beta, c, ldc, stridec, batch_count);
}
}
