// Pre-split of a whole FP32 operand into fp16 hi / lo planes (FP16TCEC) or three
// bf16 planes (bf16x3) for the packed kernels.  For large problems every element of A is otherwise split
// once per column of tiles (and B once per row of tiles) inside the GEMM's K
// loop; doing it once up front takes the vector arithmetic out of that loop.
//
// Output layout (the LDS image of every (tile, K-step), so that staging in the
// GEMM is a linear 16-byte copy):
//   dst[kb][plane][row][64 bytes],  kb = K-step (32 values), plane 0 = hi, 1 = lo
//   (bf16x3: the three terms in order),
//   row < rows_pad (a multiple of 256, rows >= `rows` and K-values >= `k` are
//   zero), and inside a row the 16-byte chunk c (8 K-values) sits at position
//   c ^ lds_swizzle(row).
// HBM-bound: reads 4 bytes and writes 4 (6) bytes per element.
#include "gemm_kernel.hpp"
#include "pack_split.hpp"

namespace cumpsgemm_amd {
namespace {
constexpr int kRowsPerBlock = 64;

// KC: the source is K-contiguous (element (row, kk) at src[row * ld + kk]);
// else row-contiguous (src[kk * ld + row]).
// scale_max != nullptr: the operand is multiplied by 2^14 / *scale_max (the
// bits of 2^floor(log2 max|x|) recorded by the statistics pass) while it is
// split, if that maximum is non-zero and *scale_flag has `flag_bit` set -- the
// coefficient of the stand-alone scaling kernels, read on the device.
template <bool KC, Prec P>
__global__ __launch_bounds__(256) void pack_split_kernel(const float *__restrict__ src, uint64_t ld,
                                                         uint32_t rows, uint32_t k,
                                                         char *__restrict__ dst, uint32_t rows_pad,
                                                         const uint32_t *scale_max,
                                                         const int *scale_flag, int flag_bit,
                                                         const int *launch_flag,
                                                         uint32_t flag_accept_mask) {
  // AUTO mode: nothing to do unless the launch flag names a mode this pass serves
  if (launch_flag != nullptr && ((1u << (*launch_flag & 31)) & flag_accept_mask) == 0) return;
  float coef = 1.0f;
  if (scale_max != nullptr) {
    const float mx = __uint_as_float(*scale_max);
    if ((*scale_flag & flag_bit) && mx != 0.0f) coef = 16384.0f / mx;
    coef = __uint_as_float(__builtin_amdgcn_readfirstlane(__float_as_uint(coef)));
  }
  const uint32_t kb = blockIdx.y;
  const uint32_t t = threadIdx.x;
  // lanes run along the contiguous direction of the source
  const uint32_t row = blockIdx.x * kRowsPerBlock + (KC ? t / 4 : t % kRowsPerBlock);
  const uint32_t chunk = KC ? t % 4 : t / kRowsPerBlock;
  const uint32_t k0 = kb * 32 + chunk * 8;
  f8_t x;
#pragma unroll
  for (int j = 0; j < 8; j++) {
    const uint32_t kk = k0 + j;
    float v = 0.0f;
    if (row < rows && kk < k) v = KC ? src[(uint64_t)row * ld + kk] : src[(uint64_t)kk * ld + row];
    x[j] = v;
  }
  constexpr int NP = prec_traits<P>::NP;
  u4_t out[NP];
  if constexpr (P == Prec::FP16TCEC) {
    if (scale_max != nullptr) {
      splitter<P>::run_scaled(x, out, coef, coef * 2048.0f);
    } else {
      splitter<P>::run(x, out);
    }
  } else {
    splitter<P>::run(x, out); // (bf16 has FP32's exponent range: never scaled)
  }
  char *p = dst + ((uint64_t)kb * NP * rows_pad + row) * 64 + ((chunk ^ (uint32_t)lds_swizzle((int)row)) << 4);
#pragma unroll
  for (int pl = 0; pl < NP; pl++) *reinterpret_cast<u4_t *>(p + (uint64_t)pl * rows_pad * 64) = out[pl];
}
} // namespace

void launch_pack_split(hipStream_t stream, const float *src, bool k_contiguous, uint64_t ld,
                       uint32_t rows, uint32_t k, void *dst, uint32_t rows_pad, bool bf16x3,
                       const uint32_t *scale_max, const int *scale_flag, int flag_bit,
                       const int *launch_flag, uint32_t flag_accept_mask) {
  const dim3 grid(rows_pad / kRowsPerBlock, (k + 31) / 32);
  auto launch = [&](auto kernel) {
    hipLaunchKernelGGL(kernel, grid, dim3(256), 0, stream, src, ld, rows, k, static_cast<char *>(dst),
                       rows_pad, scale_max, scale_flag, flag_bit, launch_flag, flag_accept_mask);
  };
  if (bf16x3) {
    if (k_contiguous) launch(pack_split_kernel<true, Prec::BF16X3>);
    else launch(pack_split_kernel<false, Prec::BF16X3>);
  } else {
    if (k_contiguous) launch(pack_split_kernel<true, Prec::FP16TCEC>);
    else launch(pack_split_kernel<false, Prec::FP16TCEC>);
  }
}
} // namespace cumpsgemm_amd
