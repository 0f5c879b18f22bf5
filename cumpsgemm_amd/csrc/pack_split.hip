// Pre-split of a whole FP32 / complex64 operand into fp16 hi / lo planes
// (FP16TCEC), three or two bf16 planes (bf16x3, bf16x2) or one fp16 plane
// (FP16TC) for the packed kernels.  For large problems every element of A is otherwise split
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
// HBM-bound: reads 4 bytes and writes 2 bytes per plane and element.
#include "gemm_kernel.hpp"
#include <algorithm>
#include "pack_split.hpp"

namespace cumpsgemm_amd {
namespace {
constexpr uint32_t kRowsPerBlock = 64;

// One operand of a pre-pass launch.
struct PackJob {
  const float *src;
  uint64_t ld;
  uint32_t rows, k;
  char *dst;
  uint32_t rows_pad;
  const uint32_t *scale_max; // nullptr: no scaling
  int flag_bit;
  uint32_t grid_x, grid_y, steps_per_block;
};

// KC: the source is K-contiguous (element (row, kk) at src[row * ld + kk]);
// else row-contiguous (src[kk * ld + row]).
// scale_max != nullptr: the operand is multiplied by 2^14 / *scale_max (the
// bits of 2^floor(log2 max|x|) recorded by the statistics pass) while it is
// split, if that maximum is non-zero and *scale_flag has `flag_bit` set -- the
// coefficient of the stand-alone scaling kernels, read on the device.
// `stage_mem`: LDS of the workgroup (used by the !KC form only).
template <bool KC, Prec P, bool CPLX>
__device__ inline void pack_split_body(const PackJob &job, const int *scale_flag, char *stage_mem,
                                       const uint32_t block_x, const uint32_t block_y) {
  const float *__restrict__ src = job.src;
  char *__restrict__ dst = job.dst;
  const uint64_t ld = job.ld;
  const uint32_t rows = job.rows, k = job.k, rows_pad = job.rows_pad, steps_per_block = job.steps_per_block;
  const uint32_t *scale_max = job.scale_max;
  float coef = 1.0f;
  if (scale_max != nullptr) {
    const float mx = __uint_as_float(*scale_max);
    if ((*scale_flag & job.flag_bit) && mx != 0.0f) coef = 16384.0f / mx;
    coef = __uint_as_float(__builtin_amdgcn_readfirstlane(__float_as_uint(coef)));
  }
  // One workgroup converts `steps_per_block` K-steps of 64 rows, thread = (row,
  // 16-byte chunk), two steps in flight.  Lanes run along the contiguous
  // direction of the source:
  //   KC:  4 lanes per row -> steps_per_block * 128 (complex: 256) contiguous
  //        bytes of every row; the 4 lanes of a row write its whole 64-byte
  //        plane rows;
  //   !KC: 64 lanes along the rows -> 256 (512) contiguous bytes of each
  //        K-line; a lane's chunks are 16 bytes out of every 64 of the
  //        destination, so they are gathered in LDS -- which then holds the
  //        destination image of the block, 4 KiB per plane -- and written out
  //        as a linear copy.
  // Complex sources are interleaved (re, im); their planes are re hi, re lo,
  // im hi, im lo.
  const uint32_t k_steps = (k + 31) / 32;
  const uint32_t kb0 = block_y * steps_per_block;
  const uint32_t t = threadIdx.x;
  const uint32_t lrow = KC ? t / 4 : t % kRowsPerBlock; // row within the block
  const uint32_t row = block_x * kRowsPerBlock + lrow;
  const uint32_t chunk = KC ? t % 4 : t / kRowsPerBlock;
  const bool row_in = row < rows;
  constexpr int NC = CPLX ? 2 : 1;
  constexpr int NP = prec_traits<P>::NP;
  constexpr int NPL = NP * NC; // planes per K-step
  typedef float f4u_t __attribute__((ext_vector_type(4), aligned(4)));
  typedef float f2u_t __attribute__((ext_vector_type(2), aligned(4)));
  // (!KC) two K-steps x NPL planes x the 4 KiB image of the block
  auto stage = [&](int buf, int plane) { return stage_mem + (buf * NPL + plane) * (int)(kRowsPerBlock * 64); };

  struct Vals {
    f8_t c[NC]; // the 8 K-values of the thread's chunk: real parts, imaginary parts
  };
  auto load = [&](uint32_t kb, Vals &x) {
    const uint32_t k0 = kb * 32 + chunk * 8;
    if (row_in && k0 + 8 <= k) {
      if constexpr (KC) {
        const float *p = src + ((uint64_t)row * ld + k0) * NC;
        if constexpr (!CPLX) {
          const f4u_t lo = *reinterpret_cast<const f4u_t *>(p), hi = *reinterpret_cast<const f4u_t *>(p + 4);
          x.c[0] = f8_t{lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
        } else {
#pragma unroll
          for (int j = 0; j < 4; j++) {
            const f4u_t v = *reinterpret_cast<const f4u_t *>(p + 4 * j); // two complex values
            x.c[0][2 * j] = v[0];
            x.c[1][2 * j] = v[1];
            x.c[0][2 * j + 1] = v[2];
            x.c[1][2 * j + 1] = v[3];
          }
        }
      } else {
        const float *p = src + ((uint64_t)k0 * ld + row) * NC;
#pragma unroll
        for (int j = 0; j < 8; j++) {
          if constexpr (!CPLX) {
            x.c[0][j] = p[(uint64_t)j * ld];
          } else {
            const f2u_t v = *reinterpret_cast<const f2u_t *>(p + (uint64_t)j * ld * 2);
            x.c[0][j] = v[0];
            x.c[1][j] = v[1];
          }
        }
      }
    } else {
#pragma unroll
      for (int j = 0; j < 8; j++) {
        const uint32_t kk = k0 + j;
#pragma unroll
        for (int q = 0; q < NC; q++) {
          float v = 0.0f;
          if (row_in && kk < k)
            v = KC ? src[((uint64_t)row * ld + kk) * NC + q] : src[((uint64_t)kk * ld + row) * NC + q];
          x.c[q][j] = v;
        }
      }
    }
  };
  // position of the thread's chunk inside the 64-row block image of one plane
  const uint32_t pos = lrow * 64 + ((chunk ^ (uint32_t)lds_swizzle((int)row)) << 4);
  auto split_to = [&](const Vals &x, uint32_t kb, int buf) {
#pragma unroll
    for (int q = 0; q < NC; q++) {
      u4_t out[NP];
      if constexpr (P == Prec::FP16TCEC) {
        if (scale_max != nullptr) {
          splitter<P>::run_scaled(x.c[q], out, coef, coef * 2048.0f);
        } else {
          splitter<P>::run(x.c[q], out);
        }
      } else {
        splitter<P>::run(x.c[q], out); // (bf16 has FP32's exponent range: never scaled)
      }
#pragma unroll
      for (int pl = 0; pl < NP; pl++) {
        const int plane = q * NP + pl;
        if constexpr (KC) {
          char *p = dst + (((uint64_t)kb * NPL + plane) * rows_pad + (uint64_t)block_x * kRowsPerBlock) * 64;
          *reinterpret_cast<u4_t *>(p + pos) = out[pl];
        } else {
          *reinterpret_cast<u4_t *>(stage(buf, plane) + pos) = out[pl];
        }
      }
    }
  };
  auto copy_out = [&](uint32_t kb, int buf) { // !KC: 256 threads x 16 bytes = one plane of the block
#pragma unroll
    for (int plane = 0; plane < NPL; plane++) {
      char *p = dst + (((uint64_t)kb * NPL + plane) * rows_pad + (uint64_t)block_x * kRowsPerBlock) * 64;
      *reinterpret_cast<u4_t *>(p + t * 16) = *reinterpret_cast<const u4_t *>(stage(buf, plane) + t * 16);
    }
  };
  for (uint32_t s = 0; s < steps_per_block; s += 2) {
    const uint32_t ka = kb0 + s, kb = ka + 1;
    if (ka >= k_steps) break; // uniform
    const bool two = (s + 1 < steps_per_block) && (kb < k_steps);
    Vals xa, xb;
    load(ka, xa);
    if (two) load(kb, xb);
    if constexpr (!KC) {
      if (s > 0) __syncthreads(); // the previous pair's copies have read the stage
    }
    split_to(xa, ka, 0);
    if (two) split_to(xb, kb, 1);
    if constexpr (!KC) {
      __syncthreads();
      copy_out(ka, 0);
      if (two) copy_out(kb, 1);
    }
  }
}

template <Prec P, bool CPLX> constexpr int stage_bytes(bool kc) {
  return kc ? 16 : 2 * prec_traits<P>::NP * (CPLX ? 2 : 1) * (int)kRowsPerBlock * 64;
}

// AUTO mode: nothing to do unless the launch flag names a mode this pass serves
__device__ inline bool gated_off(const int *launch_flag, uint32_t flag_accept_mask) {
  return launch_flag != nullptr && ((1u << (*launch_flag & 31)) & flag_accept_mask) == 0;
}

// Both operands of a GEMM in one launch (blockIdx.z picks the operand; the grid
// covers the larger of the two and the surplus workgroups of the other leave).
template <bool KCA, bool KCB, Prec P, bool CPLX>
__global__ __launch_bounds__(256) void pack_split_pair_kernel(const PackJob job_a, const PackJob job_b,
                                                              const int *scale_flag, const int *launch_flag,
                                                              uint32_t flag_accept_mask) {
  if (gated_off(launch_flag, flag_accept_mask)) return;
  __shared__ __attribute__((aligned(16))) char stage_mem[stage_bytes<P, CPLX>(KCA && KCB)];
  if (blockIdx.z == 0) {
    if (blockIdx.x < job_a.grid_x && blockIdx.y < job_a.grid_y)
      pack_split_body<KCA, P, CPLX>(job_a, scale_flag, stage_mem, blockIdx.x, blockIdx.y);
  } else {
    if (blockIdx.x < job_b.grid_x && blockIdx.y < job_b.grid_y)
      pack_split_body<KCB, P, CPLX>(job_b, scale_flag, stage_mem, blockIdx.x, blockIdx.y);
  }
}

PackJob make_job(const PackOperand &o, uint32_t k, int flag_bit) {
  PackJob j{};
  j.src = o.src;
  j.ld = o.ld;
  j.rows = o.rows;
  j.k = k;
  j.dst = static_cast<char *>(o.dst);
  j.rows_pad = o.rows_pad;
  j.scale_max = o.scale_max;
  j.flag_bit = flag_bit;
  // up to 8 K-steps per workgroup, fewer while that would leave under ~2048 workgroups
  const unsigned k_steps = (k + 31) / 32, row_blocks = o.rows_pad / kRowsPerBlock;
  const unsigned spb = (unsigned)std::max<uint64_t>(1, std::min<uint64_t>(8, (uint64_t)k_steps * row_blocks / 2048));
  j.grid_x = row_blocks;
  j.grid_y = (k_steps + spb - 1) / spb;
  j.steps_per_block = spb;
  return j;
}

template <Prec P, bool CPLX>
void launch_pair_of(hipStream_t stream, const PackJob &ja, bool a_kc, const PackJob &jb, bool b_kc,
                    const int *scale_flag, const int *launch_flag, uint32_t flag_accept_mask) {
  const dim3 grid(std::max(ja.grid_x, jb.grid_x), std::max(ja.grid_y, jb.grid_y), 2);
  auto launch = [&](auto kernel) {
    hipLaunchKernelGGL(kernel, grid, dim3(256), 0, stream, ja, jb, scale_flag, launch_flag, flag_accept_mask);
  };
  if (a_kc && b_kc) launch(pack_split_pair_kernel<true, true, P, CPLX>);
  else if (a_kc) launch(pack_split_pair_kernel<true, false, P, CPLX>);
  else if (b_kc) launch(pack_split_pair_kernel<false, true, P, CPLX>);
  else launch(pack_split_pair_kernel<false, false, P, CPLX>);
}
} // namespace

// Loads the real pre-pass kernels onto the current device (a first launch would
// otherwise do that, allocating device memory for the code).
void prepare_pack_split_real() {
  hipFuncAttributes attr;
  auto touch = [&](auto kernel) { (void)hipFuncGetAttributes(&attr, reinterpret_cast<const void *>(kernel)); };
  touch(pack_split_pair_kernel<true, true, Prec::FP16TCEC, false>);
  touch(pack_split_pair_kernel<true, false, Prec::FP16TCEC, false>);
  touch(pack_split_pair_kernel<false, true, Prec::FP16TCEC, false>);
  touch(pack_split_pair_kernel<false, false, Prec::FP16TCEC, false>);
  touch(pack_split_pair_kernel<true, true, Prec::BF16X3, false>);
  touch(pack_split_pair_kernel<true, false, Prec::BF16X3, false>);
  touch(pack_split_pair_kernel<false, true, Prec::BF16X3, false>);
  touch(pack_split_pair_kernel<false, false, Prec::BF16X3, false>);
  (void)hipGetLastError();
}

void launch_pack_split_pair(hipStream_t stream, const PackOperand &a, const PackOperand &b, uint32_t k,
                            PackKind kind, const int *scale_flag, const int *launch_flag,
                            uint32_t flag_accept_mask) {
  // (the scale bits of the launch flag: 0x40 for A, 0x20 for B)
  const PackJob ja = make_job(a, k, 0x40), jb = make_job(b, k, 0x20);
  switch (kind) {
  case PackKind::BF16X3_REAL:
    launch_pair_of<Prec::BF16X3, false>(stream, ja, a.k_contiguous, jb, b.k_contiguous, scale_flag, launch_flag,
                                        flag_accept_mask);
    break;
  case PackKind::FP16TC_REAL:
    launch_pair_of<Prec::FP16TC, false>(stream, ja, a.k_contiguous, jb, b.k_contiguous, scale_flag, launch_flag,
                                        flag_accept_mask);
    break;
  case PackKind::BF16X2_REAL:
    launch_pair_of<Prec::BF16X2, false>(stream, ja, a.k_contiguous, jb, b.k_contiguous, scale_flag, launch_flag,
                                        flag_accept_mask);
    break;
  case PackKind::FP16TC_COMPLEX:
    launch_pair_of<Prec::FP16TC, true>(stream, ja, a.k_contiguous, jb, b.k_contiguous, scale_flag, launch_flag,
                                       flag_accept_mask);
    break;
  case PackKind::BF16X3_COMPLEX:
    launch_pair_of<Prec::BF16X3, true>(stream, ja, a.k_contiguous, jb, b.k_contiguous, scale_flag, launch_flag,
                                       flag_accept_mask);
    break;
  case PackKind::BF16X2_COMPLEX:
    launch_pair_of<Prec::BF16X2, true>(stream, ja, a.k_contiguous, jb, b.k_contiguous, scale_flag, launch_flag,
                                       flag_accept_mask);
    break;
  case PackKind::FP16_COMPLEX:
    launch_pair_of<Prec::FP16TCEC, true>(stream, ja, a.k_contiguous, jb, b.k_contiguous, scale_flag, launch_flag,
                                         flag_accept_mask);
    break;
  default:
    launch_pair_of<Prec::FP16TCEC, false>(stream, ja, a.k_contiguous, jb, b.k_contiguous, scale_flag,
                                          launch_flag, flag_accept_mask);
    break;
  }
}
} // namespace cumpsgemm_amd
