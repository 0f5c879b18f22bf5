// gfx950 (CDNA4, wave64) split-and-correct GEMM kernels.
//
// One workgroup computes a BM x BN tile of C = alpha*op(A)*op(B) + beta*C.
// FP32 operands are read from HBM with coalesced loads, split in registers
// into low-precision planes (fp16 hi/lo, or bf16 b0/b1/b2) and staged in LDS
// as K-contiguous rows, so that one ds_read_b128 yields the 8 K-values a lane
// feeds to v_mfma_f32_32x32x16_{f16,bf16}.  The leading product (plane 0 x
// plane 0) accumulates in `main`, every correction product in a separate
// `corr` accumulator; they are merged once, in FP32, in the epilogue:
//   C_acc = main + corr * corr_scale        (corr_scale = 2^-11 for fp16 hi/lo)
//
// Takes the place of the reference's gemm_core / mma_smem / dmem loaders
// (src/cumpsgemm_kernel.cuh:58-585, src/dmem_accessor.hpp) and of the external
// mtk::wmma::tcec fragment arithmetic (src/device_tcec_wrapper.hpp:64-106).
#pragma once
#include <algorithm>
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <type_traits>

// Instruction mix dripped in after each MFMA of the interleaved K loop (tuning
// knobs; the defaults are the measured optimum on MI355X).
#ifndef CUMPSGEMM_SCHED_VALU
#define CUMPSGEMM_SCHED_VALU 4
#endif
#ifndef CUMPSGEMM_SCHED_DS
#define CUMPSGEMM_SCHED_DS 1
#endif
#ifndef CUMPSGEMM_SCHED_VMEM
#define CUMPSGEMM_SCHED_VMEM 1
#endif
// Edge of the MFMA output block: 32 (v_mfma_f32_32x32x16_*) or 16
// (v_mfma_f32_16x16x32_*), for the kernels that read pre-split operands (and
// the in-loop complex bf16x3 ones) and for the other kernels that split in the
// K loop.
#ifndef CUMPSGEMM_MFMA_EDGE_PACKED
#define CUMPSGEMM_MFMA_EDGE_PACKED 16
#endif
#ifndef CUMPSGEMM_MFMA_EDGE_INLOOP
#define CUMPSGEMM_MFMA_EDGE_INLOOP 32
#endif
// Diagnostic build (-DCUMPSGEMM_WALK_STAMPS=1): the tile-walking pre-split
// kernel records the shader clock in front of and behind every K-step's barrier
// and after every write-out (first wave of two workgroups), see
// cuMpSGEMM_set_walk_stamp_buffer.  Off in the library that is shipped.
#ifndef CUMPSGEMM_WALK_STAMPS
#define CUMPSGEMM_WALK_STAMPS 0
#endif

namespace cumpsgemm_amd {

enum class Prec : int { FP16TCEC = 0, FP16TC = 1, BF16X3 = 2, BF16X2 = 3 };

typedef _Float16 h8_t __attribute__((ext_vector_type(8)));
typedef __bf16 b8_t __attribute__((ext_vector_type(8)));
typedef float f8_t __attribute__((ext_vector_type(8)));
typedef float f16v_t __attribute__((ext_vector_type(16)));
typedef float f4v_t __attribute__((ext_vector_type(4)));
typedef uint32_t u4_t __attribute__((ext_vector_type(4)));

template <Prec P> struct prec_traits;
template <> struct prec_traits<Prec::FP16TCEC> {
  static constexpr int NP = 2;    // planes per operand
  static constexpr int NPROD = 3; // MFMA products per logical product
  static constexpr int NACC = 2;
  static constexpr bool IS_BF16 = false;
  static constexpr float CORR_SCALE = 1.0f / 2048.0f;
  // {plane of A, plane of B, accumulator}
  static constexpr int PA[6] = {0, 1, 0, 0, 0, 0};
  static constexpr int PB[6] = {0, 0, 1, 0, 0, 0};
  static constexpr int ACC[6] = {0, 1, 1, 0, 0, 0};
};
template <> struct prec_traits<Prec::FP16TC> {
  static constexpr int NP = 1;
  static constexpr int NPROD = 1;
  static constexpr int NACC = 1;
  static constexpr bool IS_BF16 = false;
  static constexpr float CORR_SCALE = 1.0f;
  static constexpr int PA[6] = {0, 0, 0, 0, 0, 0};
  static constexpr int PB[6] = {0, 0, 0, 0, 0, 0};
  static constexpr int ACC[6] = {0, 0, 0, 0, 0, 0};
};
template <> struct prec_traits<Prec::BF16X3> {
  static constexpr int NP = 3;
  static constexpr int NPROD = 6;
  static constexpr int NACC = 2;
  static constexpr bool IS_BF16 = true;
  static constexpr float CORR_SCALE = 1.0f;
  // smallest terms first so they meet in the correction accumulator before
  // the larger ones
  static constexpr int PA[6] = {0, 2, 0, 1, 1, 0};
  static constexpr int PB[6] = {0, 0, 2, 1, 0, 1};
  static constexpr int ACC[6] = {0, 1, 1, 1, 1, 1};
};
template <> struct prec_traits<Prec::BF16X2> {
  static constexpr int NP = 2;
  static constexpr int NPROD = 3;
  static constexpr int NACC = 2;
  static constexpr bool IS_BF16 = true;
  static constexpr float CORR_SCALE = 1.0f;
  static constexpr int PA[6] = {0, 1, 0, 0, 0, 0};
  static constexpr int PB[6] = {0, 0, 1, 0, 0, 0};
  static constexpr int ACC[6] = {0, 1, 1, 0, 0, 0};
};

// Arguments shared by every GEMM kernel (passed by value as one struct).
struct GemmArgs {
  uint32_t m, n, k;
  uint32_t k_chunk;  // K range handled by one blockIdx.z (== k when no split-K)
  const void *a;
  const void *b;
  void *c;
  uint64_t lda, ldb, ldc;                // in elements
  uint64_t stride_a, stride_b, stride_c; // in elements, per blockIdx.y
  float alpha_re, alpha_im, beta_re, beta_im;
  uint32_t conj_a, conj_b; // complex only: op C (the sign is applied when the partial products are combined)
  uint32_t tiles_m, tiles_n;
  uint32_t batch;      // persistent kernels walk (tile, batch) pairs themselves
  uint32_t atomic_out; // split-K: C += alpha*acc with float atomics
  uint32_t raster_group; // tile rows per column group of the tile order (0: 8); | kFetchFromOnePatch
  // AUTO mode: device flag consulted before doing any work.  The kernel runs
  // only if ((1u << (flag & 31)) & flag_accept_mask) != 0.
  const int *launch_flag;
  uint32_t flag_accept_mask;
  // SCALED kernels: power-of-two scaling fused into the split (A, B) and the
  // write-out (C).  The coefficients come from device memory -- the maximum
  // exponents recorded by the statistics passes and the scale bits of a launch
  // flag -- so that no host synchronisation is needed.
  const uint32_t *scale_max_a, *scale_max_b; // bits of 2^floor(log2 max|x|)
  const int *scale_flag;                     // bit 6: scale A, bit 5: scale B
#if CUMPSGEMM_WALK_STAMPS
  unsigned long long *stamps; // 2 x 512 words: [count, stamps...] of workgroups 0 and 101
#endif
};

// Bit of GemmArgs::raster_group understood by the tile-walking pre-split kernel
// only: a profiler experiment (see there), never set by a normal call.
constexpr uint32_t kFetchFromOnePatch = 0x80000000u;

// ---- split one group of 8 FP32 values into NP packed 16-byte plane chunks ----
template <Prec P> struct splitter;

// hi = fp16(x); lo = fp16((x - hi) * 2^11).  (x - hi) is exact in FP32 and so is
// the scaling, hence lo = fp16(fma(hi, -2^11, x * 2^11)) is the same value; it
// is evaluated with the mixed-precision FMA that reads hi straight from its
// packed fp16 register and writes the fp16 result into the low / high half of
// the destination: 2.5 vector instructions per element instead of 4.
__device__ inline uint32_t split_pair_fp16(const float x0, const float x1, uint32_t &lo) {
  typedef _Float16 h2_t __attribute__((ext_vector_type(2)));
  typedef float f2_t __attribute__((ext_vector_type(2)));
  f2_t x = {x0, x1};
  const uint32_t hi = __builtin_bit_cast(uint32_t, __builtin_convertvector(x, h2_t));
  const float t0 = x0 * 2048.0f, t1 = x1 * 2048.0f;
  const float k = -2048.0f;
  uint32_t l;
  asm("v_fma_mixlo_f16 %0, %1, %2, %3 op_sel_hi:[1,0,0]" : "=v"(l) : "v"(hi), "s"(k), "v"(t0));
  asm("v_fma_mixhi_f16 %0, %1, %2, %3 op_sel:[1,0,0] op_sel_hi:[1,0,0]"
      : "+v"(l)
      : "v"(hi), "s"(k), "v"(t1));
  lo = l;
  return hi;
}

// The same split of (x * s), s a power of two held in a scalar register (s2048
// = s * 2^11): hi = fp16(x * s) comes from the mixed-precision FMA as well, so
// the scaling costs one more instruction per pair, not one per element.
__device__ inline uint32_t split_pair_fp16_scaled(const float x0, const float x1, const float s,
                                                  const float s2048, uint32_t &lo) {
  uint32_t hi;
  asm("v_fma_mixlo_f16 %0, %1, %2, 0 op_sel_hi:[0,0,0]" : "=v"(hi) : "v"(x0), "s"(s));
  asm("v_fma_mixhi_f16 %0, %1, %2, 0 op_sel_hi:[0,0,0]" : "+v"(hi) : "v"(x1), "s"(s));
  const float t0 = x0 * s2048, t1 = x1 * s2048;
  const float k = -2048.0f;
  uint32_t l;
  asm("v_fma_mixlo_f16 %0, %1, %2, %3 op_sel_hi:[1,0,0]" : "=v"(l) : "v"(hi), "s"(k), "v"(t0));
  asm("v_fma_mixhi_f16 %0, %1, %2, %3 op_sel:[1,0,0] op_sel_hi:[1,0,0]"
      : "+v"(l)
      : "v"(hi), "s"(k), "v"(t1));
  lo = l;
  return hi;
}

template <> struct splitter<Prec::FP16TCEC> {
  __device__ static inline void run(const f8_t x, u4_t (&out)[2]) {
#pragma unroll
    for (int i = 0; i < 4; i++) {
      uint32_t lo;
      out[0][i] = split_pair_fp16(x[2 * i], x[2 * i + 1], lo);
      out[1][i] = lo;
    }
  }
  __device__ static inline void run_scaled(const f8_t x, u4_t (&out)[2], const float s,
                                           const float s2048) {
#pragma unroll
    for (int i = 0; i < 4; i++) {
      uint32_t lo;
      out[0][i] = split_pair_fp16_scaled(x[2 * i], x[2 * i + 1], s, s2048, lo);
      out[1][i] = lo;
    }
  }
};
template <> struct splitter<Prec::FP16TC> {
  __device__ static inline void run(const f8_t x, u4_t (&out)[1]) {
    out[0] = __builtin_bit_cast(u4_t, __builtin_convertvector(x, h8_t));
  }
};
template <> struct splitter<Prec::BF16X3> {
  __device__ static inline void run(const f8_t x, u4_t (&out)[3]) {
    const b8_t b0 = __builtin_convertvector(x, b8_t);
    const f8_t r1 = x - __builtin_convertvector(b0, f8_t);
    const b8_t b1 = __builtin_convertvector(r1, b8_t);
    const f8_t r2 = r1 - __builtin_convertvector(b1, f8_t);
    const b8_t b2 = __builtin_convertvector(r2, b8_t);
    out[0] = __builtin_bit_cast(u4_t, b0);
    out[1] = __builtin_bit_cast(u4_t, b1);
    out[2] = __builtin_bit_cast(u4_t, b2);
  }
};
template <> struct splitter<Prec::BF16X2> {
  __device__ static inline void run(const f8_t x, u4_t (&out)[2]) {
    const b8_t b0 = __builtin_convertvector(x, b8_t);
    const f8_t r1 = x - __builtin_convertvector(b0, f8_t);
    const b8_t b1 = __builtin_convertvector(r1, b8_t);
    out[0] = __builtin_bit_cast(u4_t, b0);
    out[1] = __builtin_bit_cast(u4_t, b1);
  }
};

template <bool IS_BF16>
__device__ inline f16v_t mfma_block(const u4_t a, const u4_t b, const f16v_t c) {
  if constexpr (IS_BF16) {
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(
        __builtin_bit_cast(b8_t, a), __builtin_bit_cast(b8_t, b), c, 0, 0, 0);
  } else {
    return __builtin_amdgcn_mfma_f32_32x32x16_f16(
        __builtin_bit_cast(h8_t, a), __builtin_bit_cast(h8_t, b), c, 0, 0, 0);
  }
}
template <bool IS_BF16>
__device__ inline f4v_t mfma_block(const u4_t a, const u4_t b, const f4v_t c) {
  if constexpr (IS_BF16) {
    return __builtin_amdgcn_mfma_f32_16x16x32_bf16(
        __builtin_bit_cast(b8_t, a), __builtin_bit_cast(b8_t, b), c, 0, 0, 0);
  } else {
    return __builtin_amdgcn_mfma_f32_16x16x32_f16(
        __builtin_bit_cast(h8_t, a), __builtin_bit_cast(h8_t, b), c, 0, 0, 0);
  }
}

// Tile configuration.  BK is fixed at 32 (4 chunks of 8 K-values per row).
//   A_KC: op(A) is stored K-contiguous (op T / C); else M-contiguous (op N)
//   B_KC: op(B) is stored K-contiguous (op N);     else N-contiguous (op T / C)
//   OCC : waves per SIMD the register allocator must leave room for
//   DEEP: three LDS buffers and an interleaved instruction schedule (MFMAs with
//         the staging work dripped in between); otherwise two buffers and
//         plain program order.
//   PERSIST (DEEP only): one workgroup per CU slot walks a list of tiles and
//         keeps the load pipeline running across tile boundaries, so that the
//         first K-steps of the next tile are already in LDS when the current
//         tile's results are written out.  Interior tiles only (the host
//         checks divisibility and alignment).
//   SCALED (FP16TCEC only): op(A), op(B) are multiplied by powers of two read
//         from device memory while they are split, and the result by the
//         inverse product when it is written out (see GemmArgs).
//   PACKED (three-buffer kernels; complex bf16x3: two buffers): A
//         and B were split beforehand into fp16 / bf16 planes laid out as the
//         LDS image of every (tile, K-step), see pack_split_kernel; staging is
//         a plain 16-byte copy, no arithmetic.
//   KS2 (two-buffer kernels): twice the waves; the two wave groups take
//         one 16-wide K-slice of every step each and add their accumulators
//         through LDS at the end, and one group stages A, the other B (complex
//         half-unit loaders: every thread half a unit of each).  For a
//         problem of no more tiles than CUs: two waves per SIMD instead of one
//         shorten the chain LDS read -> MFMA -> split -> LDS write of a step.
template <Prec P_, bool CPLX_, bool A_KC_, bool B_KC_, int BM_, int BN_, int WM_,
          int WN_, int OCC_ = 1, bool DEEP_ = false, bool PERSIST_ = false, bool SCALED_ = false,
          bool PACKED_ = false, bool KS2_ = false, bool E16_ = false>
struct GemmCfg {
  static_assert(!KS2_ || (!DEEP_ && !PACKED_), "K-slice split: two-buffer kernels");
  static constexpr bool KS2 = KS2_;
  // (PACKED + SCALED: the operands were scaled when they were pre-split; the
  // kernel only folds the inverse scaling of C into alpha)
  // (three buffers of pre-split planes, except for complex bf16x3, whose six
  // planes per operand leave room for two: its pre-split kernel is the
  // two-buffer, one-tile form)
  static_assert(!PACKED_ || (DEEP_ != (P_ == Prec::BF16X3 && CPLX_)), "packed form");
  static_assert(!(PACKED_ && !DEEP_) || !PERSIST_, "two-buffer packed form: one tile per workgroup");
  static constexpr bool PACKED = PACKED_;
  static_assert(!PERSIST_ || DEEP_, "persistent kernels use the three-buffer pipeline");
  static_assert(!SCALED_ || P_ == Prec::FP16TCEC, "scaling guards the fp16 range only");
  using persistent_type =
      GemmCfg<P_, CPLX_, A_KC_, B_KC_, BM_, BN_, WM_, WN_, OCC_, DEEP_, DEEP_, SCALED_, false, false, E16_>;
  using scaled_type = GemmCfg<P_, CPLX_, A_KC_, B_KC_, BM_, BN_, WM_, WN_, OCC_, DEEP_, PERSIST_,
                              P_ == Prec::FP16TCEC, false, false, E16_>;
  // the same kernel on 16x16x32 MFMAs (E16_: asked for by the table)
  using edge16_type = GemmCfg<P_, CPLX_, A_KC_, B_KC_, BM_, BN_, WM_, WN_, OCC_, DEEP_, PERSIST_, SCALED_,
                              PACKED_, KS2_, true>;
  static constexpr bool SCALED = SCALED_;
  static constexpr int OCC = OCC_;
  static constexpr bool DEEP = DEEP_;
  static constexpr bool PERSIST = PERSIST_;
  static constexpr Prec P = P_;
  static constexpr bool CPLX = CPLX_;
  static constexpr bool A_KC = A_KC_;
  static constexpr bool B_KC = B_KC_;
  static constexpr int BM = BM_, BN = BN_, BK = 32, WM = WM_, WN = WN_;
  static constexpr int TILE_WAVES = (BM / WM) * (BN / WN); // waves that cover the tile once
  static constexpr int NWAVES = TILE_WAVES * (KS2_ ? 2 : 1);
  static constexpr int NT = NWAVES * 64;
  // MFMA block edge, blocks per wave tile, accumulator registers per block
  // (in-loop kernels measured with edge 16 over 34 shapes x 3 layouts, single
  // and strided-batch, every tile class forced: complex bf16x3 + 5 - 7 %
  // throughout; the 256x128 kernels of bf16x2, which spill 230 - 260 B per
  // lane with edge 32 and nothing with 16, x 1.2 - 2.4; the 128x256 kernel of
  // FP16TCEC for two M/N-contiguous operands + 15 - 35 %; the others between
  // - 8 % and + 9 % with a mean of zero, so they keep 32)
  static constexpr bool EDGE16_INLOOP =
      (P_ == Prec::BF16X3 && CPLX_) || (P_ == Prec::BF16X2 && !CPLX_ && BM_ * BN_ >= 256 * 128) ||
      (P_ == Prec::FP16TCEC && !CPLX_ && !A_KC_ && !B_KC_ && BM_ == 128 && BN_ == 256);
  static constexpr int MT = PACKED_ ? CUMPSGEMM_MFMA_EDGE_PACKED
                            : (EDGE16_INLOOP || E16_) ? CUMPSGEMM_MFMA_EDGE_PACKED
                                                      : CUMPSGEMM_MFMA_EDGE_INLOOP;
  // Real FP16TCEC, 256x128 and 128x128, tile-walking: a second instance on 16x16x32
  // MFMAs for launches that keep every CU busy.  There the part runs against its power
  // limit and the 16x16x32 form, which needs less energy per flop, measures
  // 3 - 9 % faster (512^3 x 64 279 -> 296, 4096^2 x 512 284 -> 301, 256^3 x 512
  // 222 -> 243 TFLOP/s; 128x128: 1152^2 x 384 x 16 236 -> 244, 768^2 x 256 x 64 229 -> 234);
  // on launches that leave CUs idle the clock is higher and 32x32x16 wins by 4 - 8 %
  // (2304^2 x 768 242 -> 223).
  // (the same for the 128x128 kernel of real bf16x3 -- 512^3 x 64 176 -> 182 / 174 -> 188 NN / TN,
  // 384^3 x 128 158 -> 166 / 157 -> 169 -- and the 256x128 one of FP16TC -- 1024^3 x 8 553 -> 567 / 558 -> 609)
  static constexpr bool HAS_EDGE16_TWIN =
      !CPLX_ && !PACKED_ && DEEP_ && !KS2_ && !EDGE16_INLOOP && !E16_ &&
      ((P_ == Prec::FP16TCEC && BM_ * BN_ >= 128 * 128) || (P_ == Prec::BF16X3 && BM_ * BN_ == 128 * 128) ||
       (P_ == Prec::FP16TC && BM_ * BN_ >= 256 * 128));
  static_assert(MT == 32 || MT == 16, "MFMA block edge");
  static constexpr int TM = WM / MT, TN = WN / MT;
  static constexpr int NV = MT * MT / 64;
  static constexpr int NP = prec_traits<P>::NP;
  static constexpr int NCOMP = CPLX ? 2 : 1;
  // LDS row: 32 K-values * 2 bytes = four 16-byte chunks, stored at chunk
  // position (chunk ^ lds_swizzle(row)); see lds_offset().
  static constexpr int ROW_BYTES = 64;
  // DEEP workgroups keep three tiles in LDS so that a tile is complete one full
  // step before it is multiplied and its first fragments can be fetched ahead
  // of the barrier; the others double-buffer.
  static constexpr int NSTAGE = DEEP_ ? 3 : 2;
  static constexpr int A_PLANE_BYTES = BM * ROW_BYTES;
  static constexpr int B_PLANE_BYTES = BN * ROW_BYTES;
  static constexpr int A_STAGE_BYTES = A_PLANE_BYTES * NP * NCOMP;
  static constexpr int B_STAGE_BYTES = B_PLANE_BYTES * NP * NCOMP;
  static constexpr int STAGE_BYTES = A_STAGE_BYTES + B_STAGE_BYTES;
  // (KS2: the second wave group's accumulators pass through LDS once)
  static constexpr int REDUCE_BYTES =
      KS2_ ? TILE_WAVES * 64 * (CPLX_ ? 4 : 1) * prec_traits<P>::NACC * TM * TN * NV * 4 : 0;
  static constexpr int LDS_BYTES = NSTAGE * STAGE_BYTES > REDUCE_BYTES ? NSTAGE * STAGE_BYTES : REDUCE_BYTES;
  static_assert(!KS2_ || (MT == 32 && BM * 4 + BN * 4 == NT), "one staging unit per thread: A then B");
  // staging units: one unit = (row, chunk of 8 K-values)
  // (when a tile has fewer units than the workgroup has threads, the surplus
  // waves simply stage nothing for that operand)
  static constexpr int UA = (BM * 4 + NT - 1) / NT;
  static constexpr int UB = (BN * 4 + NT - 1) / NT;
  static_assert((BM * 4) % NT == 0 || (BM * 4) < NT, "tile/threads");
  static_assert((BN * 4) % NT == 0 || (BN * 4) < NT, "tile/threads");
  static_assert(BM % WM == 0 && BN % WN == 0 && WM % 32 == 0 && WN % 32 == 0,
                "wave tile");
  static_assert(LDS_BYTES <= 160 * 1024, "LDS budget");
};

// Byte offset of (row, 16-byte chunk) inside one LDS plane.  Rows are 64 bytes,
// i.e. 16 banks; the chunk is XOR-swizzled with row bits.  The swizzle was
// picked by measurement (SQ_LDS_BANK_CONFLICT over all 256 swizzles whose two
// bits are parities of the low four row bits): it is one of the 16 that take
// every access pattern of these kernels without a conflict cycle --
//  - fragment reads, ds_read_b128: lane l at row l % 32, chunk l / 32
//    (32x32x16 MFMAs) or at row l % 16, chunk l / 16 (16x16x32 MFMAs),
//  - staging writes, ds_write_b128: 16 consecutive rows x 4 chunks (a
//    K-contiguous tile) or 64 consecutive rows at one chunk (a row-contiguous
//    one), and their 8-byte half-unit forms.
__device__ inline int lds_swizzle(int row) {
  return (((row >> 1) ^ (row >> 3)) & 1) | ((((row >> 2) ^ (row >> 3)) & 1) << 1);
}
__device__ inline int lds_offset(int row, int chunk) {
  return row * 64 + ((chunk ^ lds_swizzle(row)) << 4);
}

// Workgroup barrier that orders LDS traffic only.  __syncthreads() also fences
// global memory, which makes every wave wait for its outstanding global loads
// -- the prefetch of a later K-step -- before it may pass the barrier.
__device__ inline void block_sync_lds() {
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup", "local");
  __builtin_amdgcn_s_barrier();
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup", "local");
}

// Immediate of s_waitcnt that waits until at most `n` vector-memory operations
// of the wave are in flight and leaves the other counters alone.  gfx9 family
// encoding: vmcnt[3:0] in bits 3:0 and vmcnt[5:4] in bits 15:14; expcnt (bits
// 6:4) and lgkmcnt (bits 11:8) at their maxima mean "do not wait".
constexpr int waitcnt_vm(int n) { return (n & 15) | ((n >> 4) << 14) | (7 << 4) | (15 << 8); }
static_assert(waitcnt_vm(6) == 0x0f76 && waitcnt_vm(63) == 0xcf7f, "s_waitcnt vmcnt immediate");

// The tile-walking pre-split kernel keeps global -> LDS loads in flight across
// a tile's write-out, and a wave learns that a load has landed only from its
// vector-memory counter, which counts loads and stores alike and retires them
// in issue order: "at most n in flight" means everything but the n youngest
// operations is complete.  Seen from one wave, around a write-out (L(i): the
// `ndma` loads of the next tile's K-step i):
//     last step of a tile:  L(1), MFMAs, wait(ndma), barrier
//     write-out:            S stores
//     first step:           L(2), MFMAs, wait(w), barrier; step 1 is read next -> L(1) complete?
//     second step on:       L(i + 2), MFMAs, wait(ndma), barrier
// Younger than L(1) at the first step's wait: the stores and L(2), so that
// wait is safe iff w <= ndma + S.  This function plays the sequence for three
// tiles of `nk` steps with S stores after each and reports whether every
// buffer is complete when the barrier before its first read is passed.
constexpr bool walk_waits_cover(int ndma, int stores, int w, int nk) {
  int issued = 0;        // operations issued so far
  int complete = 0;      // operations known complete (a prefix, by the in-order rule)
  int load_end[64] = {}; // issue count right after the loads of step i
  if (3 * nk + 2 > 64 || nk < 2) return false;
  auto issue_loads = [&](int step) {
    issued += ndma;
    load_end[step] = issued;
  };
  auto wait = [&](int n) {
    if (issued - n > complete) complete = issued - n;
  };
  issue_loads(0);
  issue_loads(1);
  wait(0);
  for (int t = 0; t < 3; t++) {
    for (int s = 0; s < nk; s++) {
      const int step = t * nk + s;
      issue_loads(step + 2);
      wait(t > 0 && s == 0 ? w : ndma);
      // barrier; the next step reads the planes of step + 1
      if (load_end[step + 1] > complete) return false;
    }
    issued += stores; // write-out
  }
  return true;
}
constexpr bool walk_waits_cover_range(int ndma, int stores_lo, int stores_hi, int w) {
  for (int s = stores_lo; s <= stores_hi; s++)
    for (int nk = 2; nk <= 6; nk++)
      if (!walk_waits_cover(ndma, s, w, nk)) return false;
  return true;
}
// (the model itself: one store fewer than the wait allows for must fail it)
static_assert(walk_waits_cover_range(6, 57, 128, 63) && !walk_waits_cover(6, 56, 63, 4) &&
                  walk_waits_cover_range(6, 0, 64, 6) && !walk_waits_cover(6, 0, 7, 4),
              "model of the in-order vector-memory counter");

// Map a linear workgroup id to a tile so that (a) workgroups that the
// dispatcher places on the same XCD (id mod 8) work on neighbouring tiles and
// share that XCD's L2, (b) tiles are walked in column groups of GROUP tile
// rows so that the A rows / B columns in flight stay small.
__device__ inline void map_tile(uint32_t bid, uint32_t tiles_m, uint32_t tiles_n,
                                uint32_t &tm, uint32_t &tn, const uint32_t GROUP = 8) {
  const uint32_t total = tiles_m * tiles_n;
  constexpr uint32_t NXCD = 8;
  uint32_t id = bid;
  if (total >= NXCD * 4) {
    const uint32_t q = total / NXCD, r = total % NXCD;
    const uint32_t xcd = bid % NXCD, loc = bid / NXCD;
    // XCD x owns a contiguous range; the first r XCDs own one tile more
    id = xcd * q + (xcd < r ? xcd : r) + loc;
  }
  const uint32_t per_group = GROUP * tiles_n;
  const uint32_t g = id / per_group;
  const uint32_t first_m = g * GROUP;
  const uint32_t gsz = (tiles_m - first_m < GROUP) ? (tiles_m - first_m) : GROUP;
  const uint32_t in = id % per_group;
  tm = first_m + in % gsz;
  tn = in / gsz;
}

// The same for a list of (tile, batch) pairs: the XCD ranges are cut from the
// whole list, so that one XCD works on neighbouring tiles of one matrix.
__device__ inline void map_tile_batched(uint32_t vid, uint32_t tiles_m, uint32_t tiles_n,
                                        uint32_t batch, uint32_t &tm, uint32_t &tn,
                                        uint32_t &bat, const uint32_t GROUP = 8) {
  const uint32_t per_batch = tiles_m * tiles_n;
  const uint32_t total = per_batch * batch;
  constexpr uint32_t NXCD = 8;
  uint32_t id = vid;
  if (total >= NXCD * 4) {
    const uint32_t q = total / NXCD, r = total % NXCD;
    const uint32_t xcd = vid % NXCD, loc = vid / NXCD;
    id = xcd * q + (xcd < r ? xcd : r) + loc;
  }
  bat = id / per_batch;
  id -= bat * per_batch;
  const uint32_t per_group = GROUP * tiles_n;
  const uint32_t g = id / per_group;
  const uint32_t first_m = g * GROUP;
  const uint32_t gsz = (tiles_m - first_m < GROUP) ? (tiles_m - first_m) : GROUP;
  const uint32_t in = id % per_group;
  tm = first_m + in % gsz;
  tn = in / gsz;
}

// ---------------------------------------------------------------------------
// Global -> register staging of one operand tile.
//   ROWS rows (M for A, N for B) x 32 K-values; U units per thread.
//   KC:   memory is K-contiguous  -> unit = (row, chunk), chunk fastest over
//         lanes; each thread reads 8 consecutive elements (16-byte loads).
//   !KC:  memory is row-contiguous -> unit = (row, chunk), row fastest over
//         lanes; each thread reads 8 elements `ld` apart, consecutive lanes
//         read consecutive addresses.
// All addresses are "uniform base + per-thread 32-bit offset": the bases live
// in scalar registers, the offsets are computed once per kernel.
// Out-of-range elements read as zero, which contributes nothing to the sums.
// ---------------------------------------------------------------------------
//   TID0: with fewer units than threads, the first thread that stages this
//         operand (the ROWS * 4 threads from there on do).
template <bool CPLX, bool KC, int ROWS, int U, int NT, bool HALF_UNITS = false, int TID0 = 0>
struct tile_loader {
  static constexpr int NC = CPLX ? 2 : 1;
  static constexpr int ES = CPLX ? 2 : 1;
  static constexpr bool PARTIAL = (ROWS * 4) < NT; // fewer units than threads
  // An operand with half as many units as threads: every thread takes
  // half a unit (4 of its 8 K-values; even threads the lower four, odd threads
  // the upper four, so that a pair of lanes fills one 16-byte chunk of a plane
  // and a wave's 8-byte LDS writes cover all banks), so that all waves have the
  // same work and the K loop no branch around an idle half.
  // (HALF_UNITS: the precisions this pays for, measured -- FP16TCEC and bf16x2; the
  // costlier bf16x3 split and the single-product FP16TC kernels keep whole units)
  static constexpr bool HALF = HALF_UNITS && (ROWS * 4 * 2 == NT);
  static_assert(TID0 == 0 || (PARTIAL && !HALF), "TID0: partial tiles of whole units");
  static constexpr int KV = HALF ? 4 : 8; // K-values a thread handles per unit

  // whether this thread stages anything of this operand (wave-uniform)
  __device__ static inline bool active(int tid) {
    return !PARTIAL || HALF || (tid >= TID0 && tid < TID0 + ROWS * 4);
  }
  // ... in the register-staged copy of pre-split planes (whole 16-byte chunks)
  __device__ static inline bool copy_active(int tid) { return !PARTIAL || tid < ROWS * 4; }
  // which half of its unit (0 unless HALF)
  __device__ static inline int half_of(int tid) { return HALF ? (tid & 1) : 0; }

  __device__ static inline void unit_coords(int u, int tid, int &row, int &chunk) {
    const int id = (HALF ? tid >> 1 : tid - TID0) + u * NT;
    if constexpr (KC) {
      chunk = id & 3;
      row = id >> 2;
    } else {
      row = id % ROWS;
      chunk = id / ROWS;
    }
  }

  // element offset of unit u from the tile origin
  __device__ static inline uint32_t unit_offset(int u, int tid, uint32_t ld) {
    int row, chunk;
    unit_coords(u, tid, row, chunk);
    const uint32_t k0 = (uint32_t)chunk * 8 + (uint32_t)half_of(tid) * 4;
    return KC ? (uint32_t)row * ld + k0 : k0 * ld + (uint32_t)row;
  }

  // whether every per-thread byte offset of a tile fits 32 bits
  __device__ static inline bool offsets_fit(uint64_t ld) {
    const uint64_t span = KC ? (uint64_t)ROWS * ld + 32 : 32 * ld + ROWS;
    return span * ES * 4 < 0x7fffffffull;
  }

  // byte offset of unit u from the tile origin
  __device__ static inline uint32_t unit_byte_offset(int u, int tid, uint32_t ld) {
    return unit_offset(u, tid, ld) * (uint32_t)(ES * 4);
  }

  // Staging registers of one thread: the 8 K-values (re, im) of each unit.
  struct Regs {
    f8_t v[U][NC];
    u4_t third[U]; // pre-split operands with three planes: the third chunk
  };

  // interior tile: base points at element (row 0 of the tile, k 0 of the K-step).
  //   !KC: buffer loads -- the descriptor (scalar registers) carries the uniform
  //        base, the vector offset is the thread's constant byte offset and the
  //        scalar offset selects the K-line, so no vector ALU work goes into
  //        addressing; consecutive lanes read consecutive addresses.
  //   KC:  16-byte global loads at base + constant per-thread offset.
  // (16-byte *buffer* loads are avoided on purpose: this toolchain narrows them
  // incorrectly when the loaded vector is taken apart element-wise.)
  __device__ static inline void load_fast(Regs &reg, const float *__restrict__ base, uint64_t ld,
                                          const uint32_t (&boff)[U]) {
    if (!active(threadIdx.x)) return;
    if constexpr (KC) {
#pragma unroll
      for (int u = 0; u < U; u++) {
        // rows of a K-contiguous operand are 16-byte aligned only if ld is a
        // multiple of 4: the vector type promises 4-byte alignment and leaves
        // the choice of instruction to the compiler
        typedef float f4u_t __attribute__((ext_vector_type(4), aligned(4)));
        const f4u_t *p = reinterpret_cast<const f4u_t *>(reinterpret_cast<const char *>(base) + boff[u]);
        if constexpr (!CPLX) {
          const f4u_t lo = p[0];
          reg.v[u][0][0] = lo.x; reg.v[u][0][1] = lo.y; reg.v[u][0][2] = lo.z; reg.v[u][0][3] = lo.w;
          if constexpr (!HALF) {
            const f4u_t hi = p[1];
            reg.v[u][0][4] = hi.x; reg.v[u][0][5] = hi.y; reg.v[u][0][6] = hi.z; reg.v[u][0][7] = hi.w;
          }
        } else {
#pragma unroll
          for (int q = 0; q < KV / 2; q++) {
            const f4u_t t = p[q];
            reg.v[u][0][2 * q] = t.x; reg.v[u][1][2 * q] = t.y;
            reg.v[u][0][2 * q + 1] = t.z; reg.v[u][1][2 * q + 1] = t.w;
          }
        }
      }
    } else {
      const __amdgpu_buffer_rsrc_t rsrc = __builtin_amdgcn_make_buffer_rsrc(
          const_cast<float *>(base), 0, 0xffffffff, 0x00020000);
      const uint32_t line = (uint32_t)ld * (uint32_t)(ES * 4); // bytes between K-lines
#pragma unroll
      for (int u = 0; u < U; u++) {
#pragma unroll
        for (int j = 0; j < KV; j++) {
          if constexpr (!CPLX) {
            reg.v[u][0][j] = __builtin_bit_cast(
                float, __builtin_amdgcn_raw_buffer_load_b32(rsrc, boff[u], j * line, 0));
          } else {
            // one 8-byte load per complex element.  The loaded pair is taken
            // apart as a 64-bit integer: extracting the elements of the vector
            // result directly is what this toolchain mis-narrows.
            typedef unsigned int u2_t __attribute__((ext_vector_type(2)));
            const u2_t t = __builtin_amdgcn_raw_buffer_load_b64(rsrc, boff[u], j * line, 0);
            const uint64_t w = __builtin_bit_cast(uint64_t, t);
            reg.v[u][0][j] = __builtin_bit_cast(float, (uint32_t)w);
            reg.v[u][1][j] = __builtin_bit_cast(float, (uint32_t)(w >> 32));
          }
        }
      }
    }
  }

  // Pre-split operand: the planes of one (tile, K-step) are stored as their LDS
  // image, ROWS * 64 bytes each, `plane_bytes` apart.  Unit u of thread t is the
  // 16-byte chunk number t + u * NT of every plane; the two chunks (hi, lo)
  // travel in the unit's staging registers.
  template <int NPL>
  __device__ static inline void load_packed(Regs &reg, const float *__restrict__ base,
                                            uint32_t plane_bytes) {
    static_assert((NPL >= 1 && NPL <= 3) || (NPL == 4 && NC == 2), "1, 2, 3 or (complex) 2 x 2 planes");
    if (!copy_active(threadIdx.x)) return;
    const char *p = reinterpret_cast<const char *>(base);
#pragma unroll
    for (int u = 0; u < U; u++) {
      const uint32_t off = (uint32_t)(threadIdx.x + u * NT) * 16u;
#pragma unroll
      for (int q = 0; q < (NPL == 4 ? 2 : 1); q++) { // complex: (re hi, re lo), (im hi, im lo)
        const float4 hi = *reinterpret_cast<const float4 *>(p + (2u * q) * plane_bytes + off);
        reg.v[u][q][0] = hi.x; reg.v[u][q][1] = hi.y; reg.v[u][q][2] = hi.z; reg.v[u][q][3] = hi.w;
        if constexpr (NPL >= 2) {
          const float4 lo = *reinterpret_cast<const float4 *>(p + (2u * q + 1u) * plane_bytes + off);
          reg.v[u][q][4] = lo.x; reg.v[u][q][5] = lo.y; reg.v[u][q][6] = lo.z; reg.v[u][q][7] = lo.w;
        }
      }
      if constexpr (NPL == 3)
        reg.third[u] = *reinterpret_cast<const u4_t *>(p + 2u * plane_bytes + off);
    }
  }
  // The same copy without the round trip through registers: 16-byte global ->
  // LDS loads (gfx950).  The 64 lanes of a wave fill 1 KiB of contiguous LDS,
  // which is what the planes' layout (the linear LDS image) asks for.  Returns
  // nothing; completion is tracked by the wave's vector-memory counter.
  template <int NPL>
  __device__ static inline void dma_packed(const float *__restrict__ base, uint32_t plane_bytes, char *lds_op,
                                           int wave) {
    typedef const void __attribute__((address_space(1))) *gptr_t;
    typedef void __attribute__((address_space(3))) *lptr_t;
    constexpr int PLANE = ROWS * 64;
    const char *p = reinterpret_cast<const char *>(base);
    if constexpr (!PARTIAL) {
#pragma unroll
      for (int u = 0; u < U; u++) {
        const uint32_t off = (uint32_t)(threadIdx.x + u * NT) * 16u;
#pragma unroll
        for (int pl = 0; pl < NPL; pl++) {
          __builtin_amdgcn_global_load_lds((gptr_t)(p + (uint32_t)pl * plane_bytes + off),
                                           (lptr_t)(lds_op + pl * PLANE + (wave * 64 + u * NT) * 16), 16, 0, 0);
        }
      }
    } else {
      // Fewer chunks per plane than threads: the threads form NT / (ROWS * 4)
      // groups and each group takes its share of the planes, so that every wave
      // issues the same number of loads and waits for them with the same
      // constant -- idle waves or masked lanes would put branches into the K loop
      // and with them an end to the interleaving of its LDS reads and MFMAs.
      constexpr int GROUPS = NT / (ROWS * 4);
      static_assert(NT % (ROWS * 4) == 0 && (ROWS * 4) % 64 == 0 && NPL % GROUPS == 0, "plane groups");
      const int group = wave / ((ROWS * 4) / 64);   // wave-uniform
      const int wave_in = wave % ((ROWS * 4) / 64);
      const uint32_t off = (uint32_t)(threadIdx.x % (ROWS * 4)) * 16u;
#pragma unroll
      for (int i = 0; i < NPL / GROUPS; i++) {
        const int pl = group * (NPL / GROUPS) + i;
        __builtin_amdgcn_global_load_lds((gptr_t)(p + (uint32_t)pl * plane_bytes + off),
                                         (lptr_t)(lds_op + pl * PLANE + wave_in * 64 * 16), 16, 0, 0);
      }
    }
  }
  // global -> LDS loads that dma_packed issues per wave
  template <int NPL> static constexpr int dma_loads() { return PARTIAL ? NPL / (NT / (ROWS * 4)) : U * NPL; }
  template <int NPL>
  __device__ static inline void store_packed(Regs &reg, char *lds_op, int tid) {
    constexpr int PLANE = ROWS * 64;
    if (!copy_active(tid)) return;
#pragma unroll
    for (int u = 0; u < U; u++) {
      const int off = (tid + u * NT) * 16;
#pragma unroll
      for (int q = 0; q < (NPL == 4 ? 2 : 1); q++) {
        const f8_t v = reg.v[u][q];
        *reinterpret_cast<float4 *>(lds_op + 2 * q * PLANE + off) = make_float4(v[0], v[1], v[2], v[3]);
        if constexpr (NPL >= 2)
          *reinterpret_cast<float4 *>(lds_op + (2 * q + 1) * PLANE + off) = make_float4(v[4], v[5], v[6], v[7]);
      }
      if constexpr (NPL == 3) *reinterpret_cast<u4_t *>(lds_op + 2 * PLANE + off) = reg.third[u];
    }
  }

  // The 8 K-values (re, im) of unit u, ready to be split.
  __device__ static inline void fetch(Regs &reg, int u, f8_t &re, f8_t &im) {
    re = reg.v[u][0];
    if constexpr (CPLX) im = reg.v[u][1];
  }

  // edge tile / unaligned / huge ld: element-wise and guarded.  The branches
  // keep only one load in flight per thread, which keeps this rarely used path
  // from dictating the kernel's register budget.
  __device__ static inline void load_guarded(Regs &reg, const float *__restrict__ base, uint64_t ld,
                                             int rows_left, int k_left, int tid) {
    if (!active(tid)) return;
#pragma unroll
    for (int u = 0; u < U; u++) {
      int row, chunk;
      unit_coords(u, tid, row, chunk);
      const int k0 = chunk * 8 + half_of(tid) * 4;
      if constexpr (KC) {
        // a unit that lies inside the matrix is 8 (complex: 16) consecutive
        // floats: wide loads, like an interior tile (a narrow operand next to a
        // long one -- C with a few columns -- sends both through this loader)
        if (row < rows_left && k0 + KV <= k_left) {
          typedef float f4u_t __attribute__((ext_vector_type(4), aligned(4)));
          const f4u_t *p = reinterpret_cast<const f4u_t *>(base + ((uint64_t)row * ld + k0) * ES);
          if constexpr (!CPLX) {
            const f4u_t lo = p[0];
            reg.v[u][0][0] = lo.x; reg.v[u][0][1] = lo.y; reg.v[u][0][2] = lo.z; reg.v[u][0][3] = lo.w;
            if constexpr (!HALF) {
              const f4u_t hi = p[1];
              reg.v[u][0][4] = hi.x; reg.v[u][0][5] = hi.y; reg.v[u][0][6] = hi.z; reg.v[u][0][7] = hi.w;
            }
          } else {
#pragma unroll
            for (int q = 0; q < KV / 2; q++) {
              const f4u_t t = p[q];
              reg.v[u][0][2 * q] = t.x; reg.v[u][1][2 * q] = t.y;
              reg.v[u][0][2 * q + 1] = t.z; reg.v[u][1][2 * q + 1] = t.w;
            }
          }
          continue;
        }
      }
#pragma unroll
      for (int j = 0; j < KV; j++) {
        const uint64_t idx = KC ? (uint64_t)row * ld + (k0 + j) : (uint64_t)(k0 + j) * ld + row;
        float tx = 0.0f, ty = 0.0f;
        if (row < rows_left && k0 + j < k_left) {
          if constexpr (!CPLX) {
            tx = base[idx];
          } else {
            const float2 t = reinterpret_cast<const float2 *>(base)[idx];
            tx = t.x;
            ty = t.y;
          }
        }
        reg.v[u][0][j] = tx;
        if constexpr (CPLX) reg.v[u][1][j] = ty;
      }
    }
  }

  // split and write to LDS: planes laid out [comp][plane][row][chunk]
  // SCALED: the values are multiplied by s (s2048 = s * 2^11) on the way
  template <Prec P, bool SCALED = false>
  __device__ static inline void store(Regs &reg, char *lds_op, int tid, float s = 1.0f,
                                      float s2048 = 2048.0f) {
    constexpr int NP = prec_traits<P>::NP;
    constexpr int PLANE = ROWS * 64;
    if (!active(tid)) return;
#pragma unroll
    for (int u = 0; u < U; u++) {
      int row, chunk;
      unit_coords(u, tid, row, chunk);
      f8_t part[2];
      fetch(reg, u, part[0], part[1]);
      if constexpr (HALF) {
        // four K-values per component: the lower half of each plane chunk is
        // computed (the upper half of the staging vector is unused) and written
        // as 8 bytes into this thread's half of the chunk
#pragma unroll
        for (int c = 0; c < NC; c++) {
#pragma unroll
          for (int j = 4; j < 8; j++) part[c][j] = 0.0f;
          u4_t out[NP];
          if constexpr (SCALED) {
            splitter<P>::run_scaled(part[c], out, s, s2048);
          } else {
            splitter<P>::run(part[c], out);
          }
#pragma unroll
          for (int p = 0; p < NP; p++) {
            typedef uint32_t u2v_t __attribute__((ext_vector_type(2)));
            const u2v_t lo2 = {out[p][0], out[p][1]};
            *reinterpret_cast<u2v_t *>(lds_op + (c * NP + p) * PLANE + lds_offset(row, chunk) + half_of(tid) * 8) = lo2;
          }
        }
        continue;
      }
#pragma unroll
      for (int c = 0; c < NC; c++) {
        u4_t out[NP];
        if constexpr (SCALED) {
          splitter<P>::run_scaled(part[c], out, s, s2048);
        } else {
          splitter<P>::run(part[c], out);
        }
#pragma unroll
        for (int p = 0; p < NP; p++) {
          *reinterpret_cast<u4_t *>(lds_op + (c * NP + p) * PLANE + lds_offset(row, chunk)) = out[p];
        }
      }
    }
  }
};

template <class Cfg>
__global__ __launch_bounds__(Cfg::NT)
__attribute__((amdgpu_waves_per_eu(Cfg::OCC, Cfg::OCC))) void gemm_tcec_kernel(const GemmArgs args) {
  constexpr Prec P = Cfg::P;
  using PT = prec_traits<P>;
  constexpr bool CPLX = Cfg::CPLX;
  constexpr int BM = Cfg::BM, BN = Cfg::BN, BK = Cfg::BK;
  constexpr int TM = Cfg::TM, TN = Cfg::TN, NP = Cfg::NP, NCOMP = Cfg::NCOMP;
  constexpr int NT = Cfg::NT;
  constexpr int ES = CPLX ? 2 : 1; // floats per element

  if (args.launch_flag != nullptr) {
    const int flag = *args.launch_flag;
    if (((1u << (flag & 31)) & args.flag_accept_mask) == 0) return;
  }

  // Fused power-of-two scaling (same coefficients as the stand-alone scaling
  // kernels: 2^14 / max for a flagged, non-zero operand, and the inverse
  // product for C).  All uniform, in scalar registers.
  float coef_a = 1.0f, coef_b = 1.0f, coef_c = 1.0f;
  if constexpr (Cfg::SCALED) {
    const int sflag = *args.scale_flag;
    const float ma = __uint_as_float(*args.scale_max_a), mb = __uint_as_float(*args.scale_max_b);
    if ((sflag & 0x40) && ma != 0.0f) {
      coef_a = 16384.0f / ma;
      coef_c *= ma / 16384.0f;
    }
    if ((sflag & 0x20) && mb != 0.0f) {
      coef_b = 16384.0f / mb;
      coef_c *= mb / 16384.0f;
    }
  }
  if constexpr (Cfg::SCALED) {
    // loaded through vector memory, so the compiler cannot see that they are
    // uniform: say so, or each costs every lane a register for the whole kernel
    auto uniform = [](float x) {
      return __uint_as_float(__builtin_amdgcn_readfirstlane(__float_as_uint(x)));
    };
    coef_a = uniform(coef_a);
    coef_b = uniform(coef_b);
    coef_c = uniform(coef_c);
  }
  const float coef_a2048 = coef_a * 2048.0f, coef_b2048 = coef_b * 2048.0f;
  // alpha with the inverse scaling of C folded in (exact: a power of two)
  const float alpha_re = args.alpha_re * coef_c, alpha_im = args.alpha_im * coef_c;

  extern __shared__ __attribute__((aligned(16))) char lds[];

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  // (KS2: two groups of waves cover the tile, each with one K-slice of every step)
  const int wave_t = Cfg::KS2 ? wave % Cfg::TILE_WAVES : wave;
  const int kgrp = Cfg::KS2 ? wave / Cfg::TILE_WAVES : 0;
  const int wm = wave_t % (BM / Cfg::WM);
  const int wn = wave_t / (BM / Cfg::WM);

  // (persistent kernels: the first tile of this workgroup's list; see below)
  uint32_t tile_m, tile_n, tile_b = blockIdx.y;
  if constexpr (Cfg::PERSIST) {
    // (the walk over pre-split operands takes its column-group height from the host)
    const uint32_t rg = args.raster_group & ~kFetchFromOnePatch;
    const uint32_t group = (Cfg::PACKED && rg) ? rg : 8u;
    map_tile_batched(blockIdx.x, args.tiles_m, args.tiles_n, args.batch, tile_m, tile_n, tile_b, group);
  } else {
    map_tile(blockIdx.x, args.tiles_m, args.tiles_n, tile_m, tile_n, args.raster_group ? args.raster_group : 8u);
  }
  const uint32_t m0 = tile_m * BM, n0 = tile_n * BN;
  // A tile that sticks out over the edge of C is computed from an origin moved
  // back so that it ends exactly at the edge (when the matrix is at least one
  // tile wide): every load stays in bounds and unguarded, the rows / columns it
  // shares with its neighbour are simply not stored again.
  // (pre-split operands are padded to whole tiles instead)
  const bool shift_m = !Cfg::PACKED && args.m >= (uint32_t)BM;
  const bool shift_n = !Cfg::PACKED && args.n >= (uint32_t)BN;
  auto load_origin_m = [&](uint32_t o) { return (shift_m && o + BM > args.m) ? args.m - BM : o; };
  auto load_origin_n = [&](uint32_t o) { return (shift_n && o + BN > args.n) ? args.n - BN : o; };
  const uint32_t ml0 = load_origin_m(m0), nl0 = load_origin_n(n0);
  const uint32_t kbeg = blockIdx.z * args.k_chunk;
  const uint32_t kend = (kbeg + args.k_chunk < args.k) ? kbeg + args.k_chunk : args.k;
  if (kbeg >= kend) return;

  const float *a = reinterpret_cast<const float *>(args.a) +
                   (uint64_t)tile_b * args.stride_a * ES;
  const float *b = reinterpret_cast<const float *>(args.b) +
                   (uint64_t)tile_b * args.stride_b * ES;
  float *c = reinterpret_cast<float *>(args.c) +
             (uint64_t)tile_b * args.stride_c * ES;

  // operand tile origins at k = kbeg
  const float *a_tile = Cfg::A_KC ? a + ((uint64_t)ml0 * args.lda + kbeg) * ES
                                  : a + ((uint64_t)kbeg * args.lda + ml0) * ES;
  const float *b_tile = Cfg::B_KC ? b + ((uint64_t)nl0 * args.ldb + kbeg) * ES
                                  : b + ((uint64_t)kbeg * args.ldb + nl0) * ES;
  // (not const: a persistent kernel moves them from tile to tile)
  // Pre-split operands: lda / ldb are the padded row counts; one K-step holds
  // NP planes of (rows x 64 bytes), i.e. 16 floats per row and plane.
  auto packed_origin = [&](const float *base, uint64_t rows_pad, uint32_t row0) {
    return base + ((uint64_t)(kbeg / BK) * (NP * NCOMP) * rows_pad + row0) * 16;
  };
  if constexpr (Cfg::PACKED) {
    a_tile = packed_origin(a, args.lda, ml0);
    b_tile = packed_origin(b, args.ldb, nl0);
  }
  const uint64_t a_kstep = Cfg::PACKED ? (uint64_t)(NP * NCOMP) * args.lda * 16
                           : Cfg::A_KC ? (uint64_t)BK * ES : (uint64_t)BK * args.lda * ES;
  const uint64_t b_kstep = Cfg::PACKED ? (uint64_t)(NP * NCOMP) * args.ldb * 16
                           : Cfg::B_KC ? (uint64_t)BK * ES : (uint64_t)BK * args.ldb * ES;

  // (real data: only the two-wave-group kernels have tiles of half as many units
  // as threads; there it pays when op(A) is K-contiguous -- 1024^3, us, one
  // operand per group -> half units: op(A) = T 14.8 -> 14.0, with op(B) = T as
  // well 17.8 -> 16.1, but op(A) = N 16.3 -> 18.0)
  constexpr bool HALF_UNITS = (P == Prec::FP16TCEC || P == Prec::BF16X2) && (CPLX || Cfg::A_KC);
  // KS2: every thread takes half a unit of each operand (above), or the first
  // wave group stages one operand and the second the other.  A row-contiguous
  // operand (eight 4-byte loads per thread) then goes to the first group:
  // measured at 1024^3, op(A) = T with op(B) = T, 17.9 us that way and 19.7 us
  // the other.
  constexpr bool HALF_B = HALF_UNITS && (BN * 4 * 2 == NT);
  constexpr bool SPLIT_AB = Cfg::KS2 && !HALF_B;
  constexpr bool B_FIRST = Cfg::A_KC && !Cfg::B_KC;
  using LA = tile_loader<CPLX, Cfg::A_KC, BM, Cfg::UA, NT, HALF_UNITS, (SPLIT_AB && B_FIRST) ? BN * 4 : 0>;
  using LB = tile_loader<CPLX, Cfg::B_KC, BN, Cfg::UB, NT, HALF_UNITS, (SPLIT_AB && !B_FIRST) ? BM * 4 : 0>;

  const int rows_a = (int)((args.m - ml0 < (uint32_t)BM) ? args.m - ml0 : BM);
  const int rows_b = (int)((args.n - nl0 < (uint32_t)BN) ? args.n - nl0 : BN);
  // unguarded loads: the (moved) tile lies inside the matrix and every
  // per-thread offset fits 31 bits
  // (pre-split operands are padded to whole tiles and K-steps: always unguarded)
  const bool a_full = Cfg::PACKED || ((rows_a == BM) && LA::offsets_fit(args.lda));
  const bool b_full = Cfg::PACKED || ((rows_b == BN) && LB::offsets_fit(args.ldb));

  uint32_t offa[Cfg::UA], offb[Cfg::UB];
#pragma unroll
  for (int u = 0; u < Cfg::UA; u++) offa[u] = LA::unit_byte_offset(u, tid, (uint32_t)args.lda);
#pragma unroll
  for (int u = 0; u < Cfg::UB; u++) offb[u] = LB::unit_byte_offset(u, tid, (uint32_t)args.ldb);

  // staging registers: the next tile this wave will split and write to LDS
  typename LA::Regs ra;
  typename LB::Regs rb;

  // accumulators: [component][main/corr][TN][TM]; MFMA rows run along N and
  // MFMA columns along M so that a lane's 64 outputs of one register are 32
  // consecutive M-values -> coalesced column-major stores.
  // Complex: the four real products ar*br, ai*bi, ar*bi, ai*br are kept apart
  // and combined -- with the signs that op C asks for -- when the tile is
  // written out, so neither the subtraction nor a conjugation costs a single
  // vector instruction in the K loop.
  constexpr int NACCSET = CPLX ? 4 : 1;
  constexpr int MT = Cfg::MT, NV = Cfg::NV;
  typedef float accv_t __attribute__((ext_vector_type(NV)));
  accv_t acc[NACCSET][PT::NACC][TN][TM];
#pragma unroll
  for (int q = 0; q < NACCSET; q++)
#pragma unroll
    for (int s = 0; s < PT::NACC; s++)
#pragma unroll
      for (int j = 0; j < TN; j++)
#pragma unroll
        for (int i = 0; i < TM; i++)
#pragma unroll
          for (int v = 0; v < NV; v++) acc[q][s][j][i][v] = 0.0f;

  const int klen = (int)(kend - kbeg);

  // FAST: interior tile, aligned, full K-step -> unguarded wide loads
  auto gload = [&](int kt, auto fast_tag) {
    constexpr bool FAST = decltype(fast_tag)::value;
    const float *ap = a_tile + (uint64_t)kt * a_kstep;
    const float *bp = b_tile + (uint64_t)kt * b_kstep;
    if constexpr (Cfg::PACKED) {
      // (register-staged copy of the planes: the three-buffer forms only; the
      // two-buffer form never comes here)
      if constexpr (Cfg::DEEP) {
        LA::template load_packed<NP * NCOMP>(ra, ap, (uint32_t)args.lda * 64u);
        LB::template load_packed<NP * NCOMP>(rb, bp, (uint32_t)args.ldb * 64u);
      }
    } else if constexpr (FAST) {
      LA::load_fast(ra, ap, args.lda, offa);
      LB::load_fast(rb, bp, args.ldb, offb);
    } else {
      const int k_left = klen - kt * BK;
      LA::load_guarded(ra, ap, args.lda, rows_a, k_left, tid);
      LB::load_guarded(rb, bp, args.ldb, rows_b, k_left, tid);
    }
  };
  auto lstore = [&](int stage) {
    char *sa = lds + stage * Cfg::STAGE_BYTES;
    char *sb = sa + Cfg::A_STAGE_BYTES;
    if constexpr (Cfg::PACKED) {
      if constexpr (Cfg::DEEP) {
        LA::template store_packed<NP * NCOMP>(ra, sa, tid);
        LB::template store_packed<NP * NCOMP>(rb, sb, tid);
      }
    } else {
      LA::template store<P, Cfg::SCALED>(ra, sa, tid, coef_a, coef_a2048);
      LB::template store<P, Cfg::SCALED>(rb, sb, tid, coef_b, coef_b2048);
    }
  };

  // Per-lane fragment addresses.  Lane l of a 32x32x16 MFMA supplies row
  // (l % 32) of its operand tile and K-values 8*(l/32).. of the 16-wide slice
  // kk, i.e. 16-byte chunk 2*kk + l/32.  The swizzle only looks at the low four
  // row bits, which are the lane's own, so the two slices differ by one XOR.
  // (Edge 16: lane l of a 16x16x32 MFMA supplies row (l % 16) and K-values
  // 8*(l/16).. of the whole 32-wide step, i.e. chunk l/16.)
  const int frag_row = lane & (MT - 1);
  const int frag_g = lane / MT;
  int a_frag_off[2], b_frag_off[2];
#pragma unroll
  for (int kk = 0; kk < 2; kk++) {
    const int chunk = MT == 32 ? 2 * (Cfg::KS2 ? kgrp : kk) + frag_g : frag_g;
    a_frag_off[kk] = lds_offset(wm * Cfg::WM + frag_row, chunk);
    b_frag_off[kk] = lds_offset(wn * Cfg::WN + frag_row, chunk);
  }

  // A K-step's MFMAs are issued from two sets of fragment registers, so that
  // one set's LDS reads run beside the MFMAs that use the other.
  //   edge 32: set h = the 16-wide K-slice h of every block of the wave tile;
  //   edge 16: set h = half h of the wave tile's row blocks and half h of its
  //            column blocks over the whole 32-wide step; the four quadrants
  //            are multiplied in the order (0,0) (0,1) (1,1) (1,0), so that
  //            each one shares an operand half with the one before it.
  // [component][plane][block]
  constexpr int FA = MT == 32 ? TM : TM / 2, FB = MT == 32 ? TN : TN / 2;
  static_assert(MT == 32 || (TM % 2 == 0 && TN % 2 == 0), "quadrants");
  struct Frags {
    u4_t a[NCOMP][NP][FA];
    u4_t b[NCOMP][NP][FB];
  };
  auto frag_load = [&](Frags &f, int stage, int h) {
    const char *sa = lds + stage * Cfg::STAGE_BYTES;
    const char *sb = sa + Cfg::A_STAGE_BYTES;
    const int ib = MT == 32 ? 0 : h * FA, jb = MT == 32 ? 0 : h * FB;
#pragma unroll
    for (int q = 0; q < NCOMP; q++)
#pragma unroll
      for (int p = 0; p < NP; p++) {
#pragma unroll
        for (int i = 0; i < FA; i++)
          f.a[q][p][i] = *reinterpret_cast<const u4_t *>(sa + (q * NP + p) * Cfg::A_PLANE_BYTES +
                                                         a_frag_off[h] + (ib + i) * MT * 64);
#pragma unroll
        for (int j = 0; j < FB; j++)
          f.b[q][p][j] = *reinterpret_cast<const u4_t *>(sb + (q * NP + p) * Cfg::B_PLANE_BYTES +
                                                         b_frag_off[h] + (jb + j) * MT * 64);
      }
  };
  // blocks [ib, ib + FA) x [jb, jb + FB) of the wave tile += fb.b x fa.a
  // (one product after the other, so that the two correction products of a
  // block are FA * FB MFMAs apart)
  auto frag_mma_part = [&](Frags &fa, Frags &fb, const int ib, const int jb) {
#pragma unroll
    for (int t = 0; t < PT::NPROD; t++)
#pragma unroll
      for (int j = 0; j < FB; j++)
#pragma unroll
        for (int i = 0; i < FA; i++) {
          const int s = PT::ACC[t], pa = PT::PA[t], pb = PT::PB[t], jj = jb + j, ii = ib + i;
          if constexpr (!CPLX) {
            acc[0][s][jj][ii] = mfma_block<PT::IS_BF16>(fb.b[0][pb][j], fa.a[0][pa][i], acc[0][s][jj][ii]);
          } else {
            acc[0][s][jj][ii] = mfma_block<PT::IS_BF16>(fb.b[0][pb][j], fa.a[0][pa][i], acc[0][s][jj][ii]);
            acc[1][s][jj][ii] = mfma_block<PT::IS_BF16>(fb.b[1][pb][j], fa.a[1][pa][i], acc[1][s][jj][ii]);
            acc[2][s][jj][ii] = mfma_block<PT::IS_BF16>(fb.b[1][pb][j], fa.a[0][pa][i], acc[2][s][jj][ii]);
            acc[3][s][jj][ii] = mfma_block<PT::IS_BF16>(fb.b[0][pb][j], fa.a[1][pa][i], acc[3][s][jj][ii]);
          }
        }
  };
  // all MFMAs of a step: f0 holds set 0, f1 set 1
  auto frag_mma = [&](Frags &f0, Frags &f1) {
    if constexpr (MT == 32) {
      frag_mma_part(f0, f0, 0, 0);
      frag_mma_part(f1, f1, 0, 0);
    } else {
      frag_mma_part(f0, f0, 0, 0);
      frag_mma_part(f0, f1, 0, FB);
      frag_mma_part(f1, f1, FA, FB);
      frag_mma_part(f1, f0, FA, 0);
    }
  };
  static_assert(BK == 32, "two 16-wide K-slices, or one 32-wide, per step");
  // MFMAs per K-step, and the vector instructions dripped in after each (half
  // as many after a 16x16x32 MFMA, which is half as long)
  constexpr int SCHED_VALU = MT == 32 ? CUMPSGEMM_SCHED_VALU : (CUMPSGEMM_SCHED_VALU + 1) / 2;
  constexpr int STEP_MFMAS = (MT == 32 ? 2 : 1) * PT::NPROD * TM * TN * (CPLX ? 4 : 1);
  // a whole K-step from one LDS buffer (KS2: this wave group's K-slice of it)
  auto mma_tile = [&](int stage) {
    Frags f0, f1;
    frag_load(f0, stage, 0);
    if constexpr (Cfg::KS2) {
      frag_mma_part(f0, f0, 0, 0);
    } else {
      frag_load(f1, stage, 1);
      frag_mma(f0, f1);
    }
  };

  // ---- epilogue -----------------------------------------------------------
  // 32x32 accumulator layout: register v of lane l holds
  //   MFMA row (-> n) = 8*(v/4) + 4*(l/32) + v%4,  MFMA column (-> m) = l%32
  // so the 32 lanes of a half-wave write 128 contiguous bytes of a C column.
  // 16x16: MFMA row (-> n) = 4*(l/16) + v, MFMA column (-> m) = l%16.
  // FULL: interior tile, no bounds checks.
  // Vector-memory operations every wave issues in an unguarded (FULL) write-out,
  // at least: one store (or atomic, or load + store) per result register; a
  // complex result is one 8-byte store.  The loops below are tied to it.
  constexpr int EPI_VMEM = TN * TM * Cfg::NV;
  const bool beta_zero = (args.beta_re == 0.0f) && (!CPLX || args.beta_im == 0.0f);
  const float sgn_a = args.conj_a ? -1.0f : 1.0f, sgn_b = args.conj_b ? -1.0f : 1.0f;
  const float sgn_ab = sgn_a * sgn_b;
  // (em0, en0): origin the tile was computed from; (lo_m, lo_n): first row /
  // column this tile owns (differs from the origin for a moved edge tile).
  // How a result reaches C is the same for every element of a launch, so it is
  // decided once per tile, outside the element loops (decided per element, the
  // write-out is a chain of scalar branches, two taken per store):
  constexpr int OUT_STORE = 0, OUT_BETA = 1, OUT_ATOMIC = 2; // C = x | C = x + beta * C | C += x (split-K)
  auto epilogue_body = [&](float *cb, const uint32_t em0, const uint32_t en0, const uint32_t lo_m,
                           const uint32_t lo_n, auto full_tag, auto out_tag) {
    constexpr bool FULL = decltype(full_tag)::value;
    constexpr int OUT = decltype(out_tag)::value;
    // Addresses: every lane keeps the 64-bit address of the first result it
    // holds (row lane_m, column lane_n of C); every other result of the lane is
    // dm rows and dn columns further on, the same dm, dn for all lanes and
    // known at compile time, so that its address is that base plus a wave-uniform
    // offset -- one 64-bit vector add per column instead of a 64-bit multiply by
    // ldc per element.
    //   16x16 blocks, real (after the lane swap below): lane l holds rows l % 32, columns 8 * (l / 32) + ...
    //   32x32 blocks: rows l % 32, columns 4 * (l / 32) + ...;  16x16, complex: rows l % 16, columns 4 * (l / 16) + ...
    constexpr bool SWAPPED = !CPLX && MT == 16;
    const uint32_t lane_m = em0 + wm * Cfg::WM + (SWAPPED ? (lane & 31) : (lane & (MT - 1)));
    const uint32_t lane_n = en0 + wn * Cfg::WN + (SWAPPED ? 8 * (lane >> 5) : 4 * (lane / MT));
    float *const lane_base = cb + ((uint64_t)lane_n * args.ldc + lane_m) * ES;
    // (taken by the kernels over pre-split operands; the kernels that split in the K loop are at their
    // register limit and measure 2 - 4 % slower with the extra base address live: they multiply per element)
    auto address = [&](const int dm, const int dn) {
      if constexpr (Cfg::PACKED) return lane_base + ((uint64_t)dn * args.ldc + (uint64_t)dm) * ES;
      else return cb + ((uint64_t)(lane_n + dn) * args.ldc + (lane_m + dm)) * ES;
    };
    auto inside = [&](const int dm, const int dn) {
      const uint32_t mm = lane_m + dm, nn = lane_n + dn;
      return FULL || (mm < args.m && nn < args.n && mm >= lo_m && nn >= lo_n);
    };
    // C = x + beta * C: the old values of a group of results are fetched first,
    // all loads in flight together, then the group is combined and stored.  (One
    // element at a time, every load would have to wait for the store before it,
    // which the compiler cannot tell apart from it, and every store for its load:
    // a round trip to memory per element.)
    auto old_value = [&](const int dm, const int dn) {
      float o = 0.0f;
      if constexpr (OUT == OUT_BETA) {
        if (inside(dm, dn)) o = *address(dm, dn);
      }
      return o;
    };
    // one real result
    auto put = [&](const float x, const float old, const int dm, const int dn) {
      if (inside(dm, dn)) {
        float *cp = address(dm, dn);
        if constexpr (OUT == OUT_ATOMIC) {
          atomicAdd(cp, x * alpha_re);
        } else if constexpr (OUT == OUT_STORE) {
          // the result is not read again by this kernel: streaming store
          __builtin_nontemporal_store(x * alpha_re, cp);
        } else {
          *cp = x * alpha_re + args.beta_re * old;
        }
      }
    };
    auto real_value = [&](const int j, const int i, const int v) {
      float x = acc[0][0][j][i][v];
      if constexpr (PT::NACC == 2) x += acc[0][1][j][i][v] * PT::CORR_SCALE;
      return x;
    };
    if constexpr (SWAPPED) {
      static_assert(TN * (TM / 2) * 4 * 2 == EPI_VMEM, "stores of the write-out");
      // Two neighbouring row blocks trade their odd / even 16-lane rows, after
      // which register v of lane l holds column 4*(2*(l/32) + w) + v, row l%32
      // of the block pair (w = 0, 1: the first / second register of the pair):
      // 32 lanes write 128 contiguous bytes, as with the 32x32 blocks.
#pragma unroll
      for (int j = 0; j < TN; j++) {
        float old[TM / 2][4][2];
#pragma unroll
        for (int i = 0; i < TM; i += 2)
#pragma unroll
          for (int v = 0; v < 4; v++)
#pragma unroll
            for (int w = 0; w < 2; w++) old[i / 2][v][w] = old_value(i * 16, j * 16 + 4 * w + v);
#pragma unroll
        for (int i = 0; i < TM; i += 2) {
#pragma unroll
          for (int v = 0; v < 4; v++) {
            const auto r = __builtin_amdgcn_permlane16_swap(__float_as_uint(real_value(j, i, v)),
                                                            __float_as_uint(real_value(j, i + 1, v)), false, false);
#pragma unroll
            for (int w = 0; w < 2; w++) put(__uint_as_float(r[w]), old[i / 2][v][w], i * 16, j * 16 + 4 * w + v);
          }
        }
      }
      return;
    }
#pragma unroll
    for (int j = 0; j < TN; j++)
#pragma unroll
      for (int i = 0; i < TM; i++) {
        auto offsets = [&](const int v, int &dm, int &dn) {
          dm = i * MT;
          dn = j * MT + (MT == 32 ? 8 * (v / 4) + (v & 3) : v);
        };
        // (groups of four: the kernels that split in the K loop have no registers to spare)
        if constexpr (!CPLX) {
#pragma unroll
          for (int g = 0; g < NV; g += 4) {
            float old[4];
#pragma unroll
            for (int v = g; v < g + 4; v++) {
              int dm, dn;
              offsets(v, dm, dn);
              old[v - g] = old_value(dm, dn);
            }
#pragma unroll
            for (int v = g; v < g + 4; v++) {
              int dm, dn;
              offsets(v, dm, dn);
              put(real_value(j, i, v), old[v - g], dm, dn);
            }
          }
        } else {
#pragma unroll
          for (int g = 0; g < NV; g += 4) {
          float2 old[4];
          if constexpr (OUT == OUT_BETA) {
#pragma unroll
            for (int v = g; v < g + 4; v++) {
              int dm, dn;
              offsets(v, dm, dn);
              old[v - g] = make_float2(0.0f, 0.0f);
              if (inside(dm, dn)) old[v - g] = *reinterpret_cast<const float2 *>(address(dm, dn));
            }
          }
#pragma unroll
          for (int v = g; v < g + 4; v++) {
            int dm, dn;
            offsets(v, dm, dn);
            if (!inside(dm, dn)) continue;
            float *cp = address(dm, dn);
            // re = ar*br - sa*sb*ai*bi, im = sb*ar*bi + sa*ai*br with
            // sa (sb) = -1 when op(A) (op(B)) conjugates
            float p[4];
#pragma unroll
            for (int q = 0; q < 4; q++) {
              p[q] = acc[q][0][j][i][v];
              if constexpr (PT::NACC == 2) p[q] += acc[q][1][j][i][v] * PT::CORR_SCALE;
            }
            const float x = p[0] - sgn_ab * p[1];
            const float y = sgn_b * p[2] + sgn_a * p[3];
            float rx = x * alpha_re - y * alpha_im;
            float ry = y * alpha_re + x * alpha_im;
            if constexpr (OUT == OUT_ATOMIC) {
              atomicAdd(cp, rx);
              atomicAdd(cp + 1, ry);
            } else {
              if constexpr (OUT == OUT_BETA) {
                rx = x * alpha_re - y * alpha_im + (args.beta_re * old[v - g].x - args.beta_im * old[v - g].y);
                ry = y * alpha_re + x * alpha_im + (args.beta_im * old[v - g].x + args.beta_re * old[v - g].y);
              }
              // the result is not read again by this kernel: streaming store
              typedef float f2v_t __attribute__((ext_vector_type(2)));
              f2v_t out2 = {rx, ry};
              __builtin_nontemporal_store(out2, reinterpret_cast<f2v_t *>(cp));
            }
          }
          }
        }
      }
  };
  auto epilogue = [&](float *cb, const uint32_t em0, const uint32_t en0, const uint32_t lo_m, const uint32_t lo_n,
                      auto full_tag) {
    if (args.atomic_out) {
      epilogue_body(cb, em0, en0, lo_m, lo_n, full_tag, std::integral_constant<int, OUT_ATOMIC>{});
    } else if (beta_zero) {
      epilogue_body(cb, em0, en0, lo_m, lo_n, full_tag, std::integral_constant<int, OUT_STORE>{});
    } else {
      epilogue_body(cb, em0, en0, lo_m, lo_n, full_tag, std::integral_constant<int, OUT_BETA>{});
    }
  };
  auto zero_acc = [&]() {
#pragma unroll
    for (int q = 0; q < NACCSET; q++)
#pragma unroll
      for (int s = 0; s < PT::NACC; s++)
#pragma unroll
        for (int j = 0; j < TN; j++)
#pragma unroll
          for (int i = 0; i < TM; i++)
#pragma unroll
            for (int v = 0; v < NV; v++) acc[q][s][j][i][v] = 0.0f;
  };

  if constexpr (Cfg::PERSIST && Cfg::PACKED) {
    // ---- persistent walk over pre-split operands with global -> LDS loads -----
    // One workgroup walks its list of tiles; the planes of step t + 2 are asked
    // for before the MFMAs of step t, across tile boundaries.  The first step of
    // a tile is peeled off the K loop: the previous tile's write-out stands
    // between its loads and the next ones in the (in-order) vector-memory
    // counter, so its wait differs -- as a constant, not a branch inside the loop
    // (see walk_waits_cover).  After an interior tile, whose write-out issues at
    // least EPI_VMEM operations in every wave, that many more may stay in flight;
    // after an edge tile -- guarded stores, none at all from a wave that lies
    // outside C -- nothing is assumed and the plain count is used.
    const uint32_t total = args.tiles_m * args.tiles_n * args.batch;
    const uint32_t my_tiles = (total - blockIdx.x + gridDim.x - 1) / gridDim.x;
    const int nk = klen / BK;
    // (profiler experiment, kFetchFromOnePatch: every workgroup reads the planes
    // of the tile that its slot has in the first round of XCD 0, first K-step
    // only -- 32 tiles' worth of operands that every L2 keeps, so that nothing
    // but the first touch goes over the fabric -- while C is written where it
    // belongs.  The results are meaningless; the time is that of the same
    // instruction stream without operand traffic beyond the L2.)
    const bool one_patch = (args.raster_group & kFetchFromOnePatch) != 0;
    const uint32_t group = (args.raster_group & ~kFetchFromOnePatch) ? (args.raster_group & ~kFetchFromOnePatch) : 8u;
    auto tile_at = [&](uint32_t i, const float *&at, const float *&bt, float *&ct, uint32_t &om0, uint32_t &on0) {
      uint32_t tm, tn, bat;
      map_tile_batched(blockIdx.x + (i < my_tiles ? i : my_tiles - 1) * gridDim.x, args.tiles_m,
                       args.tiles_n, args.batch, tm, tn, bat, group);
      om0 = tm * BM;
      on0 = tn * BN;
      if (one_patch) {
        const uint32_t slot = blockIdx.x / 8u; // position among the workgroups of one XCD
        tm = slot % group;
        tn = slot / group;
      }
      at = packed_origin(reinterpret_cast<const float *>(args.a), args.lda, tm * BM);
      bt = packed_origin(reinterpret_cast<const float *>(args.b), args.ldb, tn * BN);
      ct = reinterpret_cast<float *>(args.c);
    };
    const uint64_t a_adv = one_patch ? 0 : a_kstep, b_adv = one_patch ? 0 : b_kstep;
    constexpr int NDMA = LA::template dma_loads<NP * NCOMP>() + LB::template dma_loads<NP * NCOMP>();
    static_assert(NDMA <= 15, "a K-step's loads must leave room in the 6-bit counter");
    constexpr int WAIT_AFTER_FULL = NDMA + EPI_VMEM > 63 ? 63 : NDMA + EPI_VMEM;
    static_assert(walk_waits_cover_range(NDMA, EPI_VMEM, 2 * EPI_VMEM, WAIT_AFTER_FULL),
                  "first-step wait after an interior write-out");
    static_assert(walk_waits_cover_range(NDMA, 0, 2 * EPI_VMEM, NDMA), "first-step wait after an edge write-out");
    const float *la = a_tile, *lb = b_tile, *la_next, *lb_next;
    float *c_cur = c, *c_ignored;
    uint32_t cm0 = m0, cn0 = n0, i0, i1;
    if (one_patch) tile_at(0, la, lb, c_ignored, i0, i1);
    tile_at(1, la_next, lb_next, c_ignored, i0, i1);
    int lk = 0;
    auto dma_next = [&](int stage) {
      char *sa = lds + stage * Cfg::STAGE_BYTES;
      char *sb = sa + Cfg::A_STAGE_BYTES;
      LA::template dma_packed<NP * NCOMP>(la, (uint32_t)args.lda * 64u, sa, wave);
      LB::template dma_packed<NP * NCOMP>(lb, (uint32_t)args.ldb * 64u, sb, wave);
      lk++;
      const bool wrap = (lk == nk);
      la = wrap ? la_next : la + a_adv;
      lb = wrap ? lb_next : lb + b_adv;
      lk = wrap ? 0 : lk;
    };
    Frags f0, f1;
    int b0 = 0, b1 = 1, b2 = 2;
#if CUMPSGEMM_WALK_STAMPS
    unsigned long long *stamp_buf = nullptr;
    if (args.stamps != nullptr && tid == 0 && (blockIdx.x == 0 || blockIdx.x == 101))
      stamp_buf = args.stamps + (blockIdx.x == 0 ? 0 : 512);
    int stamp_n = 0;
    // tag 1: this wave's MFMAs and wait are done; 0: past the barrier; 2: write-out issued
    auto stamp = [&](unsigned long long tag) {
      if (stamp_buf != nullptr && stamp_n < 500) {
        stamp_buf[1 + stamp_n] = (__builtin_readcyclecounter() & 0x0fffffffffffffffull) | (tag << 60);
        stamp_buf[0] = ++stamp_n;
      }
    };
#else
    auto stamp = [](unsigned long long) {};
#endif
    bool after_full = false; // the previous tile was written out by the unguarded epilogue
    // one K-step.  AFTER_WRITEOUT: the stores of the previous tile's write-out
    // stand between the loads it waits for and this step's own, so the number of
    // operations that may stay in flight depends on which epilogue ran (one
    // scalar branch around the wait, outside the K loop proper).
    auto step = [&](auto after_writeout_tag) {
      frag_load(f1, b0, 1);
      dma_next(b2);
      frag_mma(f0, f1);
      if constexpr (decltype(after_writeout_tag)::value) {
        if (after_full) __builtin_amdgcn_s_waitcnt(waitcnt_vm(WAIT_AFTER_FULL));
        else __builtin_amdgcn_s_waitcnt(waitcnt_vm(NDMA));
      } else {
        __builtin_amdgcn_s_waitcnt(waitcnt_vm(NDMA));
      }
      stamp(1);
      asm volatile("s_barrier" ::: "memory");
      stamp(0);
      const int tmp = b0;
      b0 = b1;
      b1 = b2;
      b2 = tmp;
      frag_load(f0, b0, 0);
    };
    dma_next(0);
    dma_next(1);
    __builtin_amdgcn_s_waitcnt(0);
    __syncthreads();
    frag_load(f0, 0, 0);
    for (uint32_t ct = 0; ct < my_tiles; ct++) {
      step(std::true_type{});
      for (int kk = 1; kk < nk; kk++) step(std::false_type{});
      const bool interior = cm0 + BM <= args.m && cn0 + BN <= args.n;
      if (interior) epilogue(c_cur, cm0, cn0, cm0, cn0, std::true_type{});
      else epilogue(c_cur, cm0, cn0, cm0, cn0, std::false_type{});
      after_full = interior;
      stamp(2);
      zero_acc();
      const float *ua, *ub;
      tile_at(ct + 1, ua, ub, c_cur, cm0, cn0);
      tile_at(ct + 2, la_next, lb_next, c_ignored, i0, i1);
    }
    __builtin_amdgcn_s_waitcnt(0);
    return;
  }
  if constexpr (Cfg::PERSIST) {
    // ---- persistent walk over this workgroup's tiles ----------------------
    // Tile i of the list is virtual workgroup blockIdx.x + i * gridDim.x.  The
    // K-steps of all tiles form one stream: the loader runs three steps ahead
    // of the multiplier straight across tile boundaries, so when a tile's
    // results are written out the next tile's first steps are already in LDS.
    // Requires >= 4 K-steps per tile (the loader's "next tile" origin is
    // refreshed when the multiplier changes tile, three steps after the loader
    // did).  The matrix is at least one tile wide and high and every K-chunk a
    // multiple of the K-step (checked by the host), so no load needs a guard.
    const uint32_t total = args.tiles_m * args.tiles_n * args.batch;
    const uint32_t my_tiles = (total - blockIdx.x + gridDim.x - 1) / gridDim.x;
    const int nk = klen / BK;
    // origin of tile i of the list: operand pointers, C, the (possibly moved)
    // origin it is computed from and the first row / column it owns
    auto origin = [&](uint32_t i, const float *&at, const float *&bt, float *&ct, uint32_t &om0,
                      uint32_t &on0, uint32_t &olo_m, uint32_t &olo_n) {
      uint32_t tm, tn, bat;
      map_tile_batched(blockIdx.x + (i < my_tiles ? i : my_tiles - 1) * gridDim.x, args.tiles_m,
                       args.tiles_n, args.batch, tm, tn, bat);
      olo_m = tm * BM;
      olo_n = tn * BN;
      om0 = load_origin_m(olo_m);
      on0 = load_origin_n(olo_n);
      const float *ab = reinterpret_cast<const float *>(args.a) + (uint64_t)bat * args.stride_a * ES;
      const float *bb = reinterpret_cast<const float *>(args.b) + (uint64_t)bat * args.stride_b * ES;
      ct = reinterpret_cast<float *>(args.c) + (uint64_t)bat * args.stride_c * ES;
      if constexpr (Cfg::PACKED) {
        at = packed_origin(ab, args.lda, om0);
        bt = packed_origin(bb, args.ldb, on0);
      } else {
        at = Cfg::A_KC ? ab + ((uint64_t)om0 * args.lda + kbeg) * ES
                       : ab + ((uint64_t)kbeg * args.lda + om0) * ES;
        bt = Cfg::B_KC ? bb + ((uint64_t)on0 * args.ldb + kbeg) * ES
                       : bb + ((uint64_t)kbeg * args.ldb + on0) * ES;
      }
    };
    const float *a_next, *b_next; // origin of the tile after the one being loaded
    const float *a_unused, *b_unused;
    float *c_cur = c, *c_unused;
    uint32_t cm0 = ml0, cn0 = nl0, clo_m = m0, clo_n = n0, u0, u1, u2, u3;
    origin(1, a_next, b_next, c_unused, u0, u1, u2, u3);
    int lk = 0;
    auto gnext = [&]() {
      gload(0, std::true_type{});
      lk++;
      const bool wrap = (lk == nk);
      a_tile = wrap ? a_next : a_tile + a_kstep;
      b_tile = wrap ? b_next : b_tile + b_kstep;
      lk = wrap ? 0 : lk;
    };
    Frags f0, f1;
    gnext();
    lstore(0);
    gnext();
    lstore(1);
    gnext();
    block_sync_lds();
    frag_load(f0, 0, 0);
    int b0 = 0, b1 = 1, b2 = 2;
    auto kstep = [&]() {
      frag_load(f1, b0, 1);
      frag_mma(f0, f1);
      lstore(b2);
      gnext();
      frag_load(f0, b1, 0);
#pragma unroll
      for (int g = 0; g < STEP_MFMAS; g++) {
        __builtin_amdgcn_sched_group_barrier(0x008, 1, 0); // MFMA
        __builtin_amdgcn_sched_group_barrier(0x002, SCHED_VALU, 0); // VALU
        __builtin_amdgcn_sched_group_barrier(0x080, CUMPSGEMM_SCHED_DS, 0); // DS
        __builtin_amdgcn_sched_group_barrier(0x020, CUMPSGEMM_SCHED_VMEM, 0); // VMEM read
      }
      block_sync_lds();
      const int tmp = b0;
      b0 = b1;
      b1 = b2;
      b2 = tmp;
    };
    auto tile_done = [&](uint32_t next) { // write the finished tile out, move on to tile `next`
      if (cm0 == clo_m && cn0 == clo_n && cm0 + BM <= args.m && cn0 + BN <= args.n) {
        epilogue(c_cur, cm0, cn0, clo_m, clo_n, std::true_type{});
      } else {
        epilogue(c_cur, cm0, cn0, clo_m, clo_n, std::false_type{});
      }
      zero_acc();
      origin(next, a_unused, b_unused, c_cur, cm0, cn0, clo_m, clo_n);
      origin(next + 1, a_next, b_next, c_unused, u0, u1, u2, u3);
    };
    if constexpr (CPLX) {
      // tiles outside, K-steps inside: measured + 3 - 5 % for the complex kernels
      // (batch 64 x 512^3 CGEMM 321 -> 335 TFLOP/s) ...
      for (uint32_t ct = 0; ct < my_tiles; ct++) {
        for (int kk = 0; kk < nk; kk++) kstep();
        tile_done(ct + 1);
      }
    } else {
      // ... and - 5 - 25 % for the real ones, which keep one flat loop over all steps
      int ck = 0;
      uint32_t ct = 0;
      const uint32_t steps = my_tiles * (uint32_t)nk;
      for (uint32_t s = 0; s < steps; s++) {
        kstep();
        if (++ck == nk) {
          ck = 0;
          tile_done(++ct);
        }
      }
    }
    return;
  }

  // The K loop over `nk` steps.  Two separate instances (fast / guarded loads)
  // keep the rarely used guarded code out of the hot loop.  Loads past the last
  // tile re-read the last one (never staged), which keeps the loop body free of
  // conditionals that touch the staging registers.
  auto pipeline = [&](const int nk, auto fast_tag) {
    const int last = nk - 1;
    auto clamp = [&](int kt) { return kt < last ? kt : last; };
    Frags f0, f1;
    if constexpr (!Cfg::DEEP) {
      // Double-buffered: every wave multiplies tile t from one LDS buffer,
      // stages tile t+1 into the other and prefetches tile t+2 into registers;
      // one barrier per step.  Overlap of vector and matrix work comes from
      // co-resident workgroups.
      gload(0, fast_tag);
      lstore(0);
      gload(clamp(1), fast_tag);
      block_sync_lds();
      for (int t = 0; t < nk; t++) {
        const int cur = t & 1;
        mma_tile(cur);
        if (t + 1 < nk) lstore(cur ^ 1);
        gload(clamp(t + 2), fast_tag);
        block_sync_lds();
      }
    } else {
      // Three LDS buffers, one barrier per step, every wave does the same work.
      // In step t a wave
      //   - multiplies tile t (buffer t%3): the first K-slice from fragments it
      //     fetched during step t-1, the second from fragments fetched now;
      //   - splits the tile it holds in registers (t+2) into buffer (t+2)%3,
      //     last read in step t-1, and reloads the registers with tile t+3;
      //   - fetches the first K-slice of its fragments of tile t+1, complete
      //     since the barrier that ended step t-1.
      // The body is one basic block and the scheduler is told to drip the
      // vector and memory instructions in between the MFMAs, so that each wave
      // keeps the matrix pipe busy while it does its share of the staging; the
      // second wave on the SIMD fills what gaps remain.
      gload(0, fast_tag);
      lstore(0);
      gload(clamp(1), fast_tag);
      lstore(1);
      gload(clamp(2), fast_tag);
      block_sync_lds();
      frag_load(f0, 0, 0);
      int b0 = 0, b1 = 1, b2 = 2; // buffers of tiles t, t+1, t+2
      for (int t = 0; t < nk; t++) {
        frag_load(f1, b0, 1);
        frag_mma(f0, f1);
        lstore(b2);
        gload(clamp(t + 3), fast_tag);
        frag_load(f0, b1, 0);
        if constexpr (decltype(fast_tag)::value) {
          // 24 (real) MFMAs per step: after each one up to 4 vector ALU
          // instructions, one LDS access and one global load
#pragma unroll
          for (int g = 0; g < STEP_MFMAS; g++) {
            __builtin_amdgcn_sched_group_barrier(0x008, 1, 0); // MFMA
            __builtin_amdgcn_sched_group_barrier(0x002, SCHED_VALU, 0); // VALU
            __builtin_amdgcn_sched_group_barrier(0x080, CUMPSGEMM_SCHED_DS, 0); // DS
            __builtin_amdgcn_sched_group_barrier(0x020, CUMPSGEMM_SCHED_VMEM, 0); // VMEM read
          }
        }
        block_sync_lds();
        const int tmp = b0;
        b0 = b1;
        b1 = b2;
        b2 = tmp;
      }
    }
  };

  if constexpr (Cfg::PACKED && !Cfg::DEEP) {
    // ---- pre-split operands, two LDS buffers, one tile per workgroup -----------
    // (complex bf16x3: twelve planes per K-step, 72 KB.)  The planes of step
    // t + 1 are asked for at the start of step t, into the buffer that step
    // t - 1 was read from (free since the barrier that ended it), and must have
    // landed when step t ends: one whole step of MFMAs -- 96 per wave here --
    // covers the latency.
    const int nk = klen / BK; // (pre-split operands are padded to whole K-steps)
    const int last = nk - 1;
    auto dma = [&](int kt, int stage) {
      const int kc = kt < last ? kt : last;
      char *sa = lds + stage * Cfg::STAGE_BYTES;
      char *sb = sa + Cfg::A_STAGE_BYTES;
      LA::template dma_packed<NP * NCOMP>(a_tile + (uint64_t)kc * a_kstep, (uint32_t)args.lda * 64u, sa, wave);
      LB::template dma_packed<NP * NCOMP>(b_tile + (uint64_t)kc * b_kstep, (uint32_t)args.ldb * 64u, sb, wave);
    };
    Frags f0, f1;
    dma(0, 0);
    __builtin_amdgcn_s_waitcnt(0);
    __syncthreads();
    frag_load(f0, 0, 0);
    for (int t = 0; t < nk; t++) {
      const int cur = t & 1;
      frag_load(f1, cur, 1);
      dma(t + 1, cur ^ 1); // (past the end: a re-read of the last step, unused)
      frag_mma(f0, f1);
      __builtin_amdgcn_s_waitcnt(waitcnt_vm(0));
      asm volatile("s_barrier" ::: "memory");
      frag_load(f0, cur ^ 1, 0);
    }
    if (ml0 == m0 && nl0 == n0 && rows_a == BM && rows_b == BN) {
      epilogue(c, ml0, nl0, m0, n0, std::true_type{});
    } else {
      epilogue(c, ml0, nl0, m0, n0, std::false_type{});
    }
    return;
  }
  if constexpr (Cfg::PACKED && !Cfg::PERSIST) {
    // ---- pre-split operands, one tile per workgroup: global -> LDS loads ------
    // The planes go from memory straight into the LDS buffers: no staging
    // registers, no ds_write.  In step t a wave
    //   - asks for its share of tile t + 2 (into the buffer that tile t - 1 was
    //     read from, free since the barrier that ended step t - 1),
    //   - multiplies tile t (first set of fragments fetched right after that
    //     barrier, second fetched now),
    //   - waits until its share of tile t + 1 -- asked for a whole step ago -- has
    //     landed, then at the barrier for everybody else's.
    // Same arithmetic in the same order as the register-staged pipeline
    // (bit-identical results); measured against it at 8192^3: + 2 % for the
    // fp16 kernel, + 0.5 % for bf16x3.
    const int nk = klen / BK; // (pre-split operands are padded to whole K-steps)
    const int last = nk - 1;
    auto dma = [&](int kt, int stage) {
      const int kc = kt < last ? kt : last;
      char *sa = lds + stage * Cfg::STAGE_BYTES;
      char *sb = sa + Cfg::A_STAGE_BYTES;
      LA::template dma_packed<NP * NCOMP>(a_tile + (uint64_t)kc * a_kstep, (uint32_t)args.lda * 64u, sa, wave);
      LB::template dma_packed<NP * NCOMP>(b_tile + (uint64_t)kc * b_kstep, (uint32_t)args.ldb * 64u, sb, wave);
    };
    // loads every wave issues per step
    constexpr int NDMA_A = LA::template dma_loads<NP * NCOMP>(), NDMA_B = LB::template dma_loads<NP * NCOMP>();
    static_assert(NDMA_A + NDMA_B <= 15, "a K-step's loads must leave room in the 6-bit counter");
    auto wait_previous_step = [&]() {
      // at most this step's loads still in flight <=> the previous step's have landed
      __builtin_amdgcn_s_waitcnt(waitcnt_vm(NDMA_A + NDMA_B));
    };
    Frags f0, f1;
    dma(0, 0);
    dma(1, 1);
    __builtin_amdgcn_s_waitcnt(0);
    __syncthreads();
    int b0 = 0, b1 = 1, b2 = 2;
    frag_load(f0, 0, 0);
    for (int t = 0; t < nk; t++) {
      frag_load(f1, b0, 1);
      dma(t + 2, b2);
      frag_mma(f0, f1);
      wait_previous_step();
      // (a plain barrier: a workgroup-scope fence on LDS would make the compiler
      // wait for the loads just issued as well; the "memory" clobber keeps it
      // from moving the fragment reads below to this side)
      asm volatile("s_barrier" ::: "memory");
      const int tmp = b0;
      b0 = b1;
      b1 = b2;
      b2 = tmp;
      frag_load(f0, b0, 0); // first K-slice of the next tile (past the end: a re-read, unused)
    }
    __builtin_amdgcn_s_waitcnt(0);
    if (ml0 == m0 && nl0 == n0 && rows_a == BM && rows_b == BN) {
      epilogue(c, ml0, nl0, m0, n0, std::true_type{});
    } else {
      epilogue(c, ml0, nl0, m0, n0, std::false_type{});
    }
    return;
  }
  if (a_full && b_full) {
    const int nk_full = klen / BK;
    if (nk_full > 0) pipeline(nk_full, std::true_type{});
    if (klen % BK != 0) { // ragged K: one more, guarded, step
      gload(nk_full, std::false_type{});
      lstore(0);
      block_sync_lds();
      mma_tile(0);
    }
  } else {
    pipeline((klen + BK - 1) / BK, std::false_type{});
  }

  if constexpr (Cfg::KS2) {
    // the second wave group hands its sums over (register r of lane l of wave w
    // at float (w * NREG + r) * 64 + l: consecutive lanes, consecutive banks)
    constexpr int NREG = NACCSET * PT::NACC * TN * TM * NV;
    float *red = reinterpret_cast<float *>(lds) + wave_t * NREG * 64 + lane;
    __syncthreads(); // (every wave is done with the last tile's fragments)
    if (kgrp == 1) {
#pragma unroll
      for (int q = 0; q < NACCSET; q++)
#pragma unroll
        for (int s = 0; s < PT::NACC; s++)
#pragma unroll
          for (int j = 0; j < TN; j++)
#pragma unroll
            for (int i = 0; i < TM; i++)
#pragma unroll
              for (int v = 0; v < NV; v++)
                red[((((q * PT::NACC + s) * TN + j) * TM + i) * NV + v) * 64] = acc[q][s][j][i][v];
    }
    __syncthreads();
    if (kgrp == 1) return;
#pragma unroll
    for (int q = 0; q < NACCSET; q++)
#pragma unroll
      for (int s = 0; s < PT::NACC; s++)
#pragma unroll
        for (int j = 0; j < TN; j++)
#pragma unroll
          for (int i = 0; i < TM; i++)
#pragma unroll
            for (int v = 0; v < NV; v++)
              acc[q][s][j][i][v] += red[((((q * PT::NACC + s) * TN + j) * TM + i) * NV + v) * 64];
  }

  if (ml0 == m0 && nl0 == n0 && rows_a == BM && rows_b == BN) {
    epilogue(c, ml0, nl0, m0, n0, std::true_type{});
  } else {
    epilogue(c, ml0, nl0, m0, n0, std::false_type{});
  }
}

// C (m x n, ldc, batched) *= beta before a split-K accumulation, or = 0
// (beta == 0 stores zeros whatever C held, NaN included).
// Block = 64 lanes along a column x 4 columns; grid = (row chunks, column
// groups, batch).  `vec`: every column starts on a 16-byte boundary, so lanes
// move 16 bytes each.
template <bool CPLX>
__global__ __launch_bounds__(256) void prescale_c_kernel(float *c, uint32_t m, uint32_t n, uint64_t ldc,
                                                         uint64_t stride_c, float beta_re, float beta_im,
                                                         uint32_t vec) {
  constexpr uint32_t ES = CPLX ? 2 : 1;
  const uint64_t mf = (uint64_t)m * ES; // floats per column
  float *cb = c + (uint64_t)blockIdx.z * stride_c * ES;
  const bool zero = beta_re == 0.0f && (!CPLX || beta_im == 0.0f);
  const uint32_t tx = threadIdx.x & 63, ty = threadIdx.x >> 6;
  // one element (a float, or a complex pair of floats)
  auto scale_one = [&](float *p) {
    if constexpr (!CPLX) {
      *p = zero ? 0.0f : beta_re * (*p);
    } else {
      float2 *q = reinterpret_cast<float2 *>(p);
      if (zero) {
        *q = make_float2(0.f, 0.f);
      } else {
        const float2 o = *q;
        *q = make_float2(beta_re * o.x - beta_im * o.y, beta_im * o.x + beta_re * o.y);
      }
    }
  };
  for (uint64_t j = (uint64_t)blockIdx.y * 4 + ty; j < n; j += (uint64_t)gridDim.y * 4) {
    float *col = cb + j * ldc * ES;
    if (vec) {
      for (uint64_t i = ((uint64_t)blockIdx.x * 64 + tx) * 4; i < mf; i += (uint64_t)gridDim.x * 256) {
        if (i + 4 <= mf) {
          float4 *q = reinterpret_cast<float4 *>(col + i);
          if (zero) {
            *q = make_float4(0.f, 0.f, 0.f, 0.f);
          } else {
            const float4 o = *q;
            if constexpr (!CPLX) {
              *q = make_float4(beta_re * o.x, beta_re * o.y, beta_re * o.z, beta_re * o.w);
            } else {
              *q = make_float4(beta_re * o.x - beta_im * o.y, beta_im * o.x + beta_re * o.y,
                               beta_re * o.z - beta_im * o.w, beta_im * o.z + beta_re * o.w);
            }
          }
        } else {
          for (uint64_t t = i; t < mf; t += ES) scale_one(col + t);
        }
      }
    } else {
      for (uint64_t i = ((uint64_t)blockIdx.x * 64 + tx) * ES; i < mf; i += (uint64_t)gridDim.x * 64 * ES)
        scale_one(col + i);
    }
  }
}

template <bool CPLX>
inline void launch_prescale_c(hipStream_t stream, void *c, uint32_t m, uint32_t n, uint64_t ldc,
                              uint64_t stride_c, uint32_t batch, float beta_re, float beta_im) {
  constexpr uint64_t ES = CPLX ? 2 : 1;
  const bool vec = (reinterpret_cast<uintptr_t>(c) % 16 == 0) && (ldc * ES % 4 == 0) &&
                   (batch == 1 || stride_c * ES % 4 == 0);
  const uint64_t per_pass = vec ? 256 : 64; // floats (complex: elements) of a column per block and pass
  const uint64_t chunks = ((uint64_t)m * (vec ? ES : 1) + per_pass - 1) / per_pass;
  const dim3 grid((unsigned)std::min<uint64_t>(chunks, 64), (unsigned)std::min<uint64_t>(((uint64_t)n + 3) / 4, 65535),
                  batch);
  hipLaunchKernelGGL(prescale_c_kernel<CPLX>, grid, dim3(256), 0, stream, static_cast<float *>(c), m, n, ldc,
                     stride_c, beta_re, beta_im, vec ? 1u : 0u);
}

} // namespace cumpsgemm_amd
