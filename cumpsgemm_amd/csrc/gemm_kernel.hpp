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
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace cumpsgemm_amd {

enum class Prec : int { FP16TCEC = 0, FP16TC = 1, BF16X3 = 2, BF16X2 = 3 };

typedef _Float16 h8_t __attribute__((ext_vector_type(8)));
typedef __bf16 b8_t __attribute__((ext_vector_type(8)));
typedef float f8_t __attribute__((ext_vector_type(8)));
typedef float f16v_t __attribute__((ext_vector_type(16)));
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
  uint32_t conj_a, conj_b; // complex only: negate imaginary part on load
  uint32_t tiles_m, tiles_n;
  uint32_t atomic_out; // split-K: C += alpha*acc with float atomics
  // AUTO mode: device flag consulted before doing any work.  The kernel runs
  // only if ((1u << (flag & 31)) & flag_accept_mask) != 0.
  const int *launch_flag;
  uint32_t flag_accept_mask;
};

// ---- split one group of 8 FP32 values into NP packed 16-byte plane chunks ----
template <Prec P> struct splitter;

template <> struct splitter<Prec::FP16TCEC> {
  __device__ static inline void run(const f8_t x, u4_t (&out)[2]) {
    const h8_t hi = __builtin_convertvector(x, h8_t);
    const f8_t r = (x - __builtin_convertvector(hi, f8_t)) * 2048.0f;
    const h8_t lo = __builtin_convertvector(r, h8_t);
    out[0] = __builtin_bit_cast(u4_t, hi);
    out[1] = __builtin_bit_cast(u4_t, lo);
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
__device__ inline f16v_t mfma32(const u4_t a, const u4_t b, const f16v_t c) {
  if constexpr (IS_BF16) {
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(
        __builtin_bit_cast(b8_t, a), __builtin_bit_cast(b8_t, b), c, 0, 0, 0);
  } else {
    return __builtin_amdgcn_mfma_f32_32x32x16_f16(
        __builtin_bit_cast(h8_t, a), __builtin_bit_cast(h8_t, b), c, 0, 0, 0);
  }
}

// Tile configuration.  BK is fixed at 32 (4 chunks of 8 K-values per row).
//   A_KC: op(A) is stored K-contiguous (op T / C); else M-contiguous (op N)
//   B_KC: op(B) is stored K-contiguous (op N);     else N-contiguous (op T / C)
//   OCC : waves per SIMD the register allocator must leave room for
template <Prec P_, bool CPLX_, bool A_KC_, bool B_KC_, int BM_, int BN_, int WM_,
          int WN_, int OCC_ = 1>
struct GemmCfg {
  static constexpr int OCC = OCC_;
  static constexpr Prec P = P_;
  static constexpr bool CPLX = CPLX_;
  static constexpr bool A_KC = A_KC_;
  static constexpr bool B_KC = B_KC_;
  static constexpr int BM = BM_, BN = BN_, BK = 32, WM = WM_, WN = WN_;
  static constexpr int NWAVES = (BM / WM) * (BN / WN);
  static constexpr int NT = NWAVES * 64;
  static constexpr int TM = WM / 32, TN = WN / 32;
  static constexpr int NP = prec_traits<P>::NP;
  static constexpr int NCOMP = CPLX ? 2 : 1;
  // LDS row: 32 K-values * 2 bytes + 16 bytes of padding.  The 80-byte pitch
  // makes both the fragment reads (consecutive rows, same chunk) and the
  // staging writes sweep all banks.
  static constexpr int ROW_BYTES = 80;
  static constexpr int A_PLANE_BYTES = BM * ROW_BYTES;
  static constexpr int B_PLANE_BYTES = BN * ROW_BYTES;
  static constexpr int A_STAGE_BYTES = A_PLANE_BYTES * NP * NCOMP;
  static constexpr int B_STAGE_BYTES = B_PLANE_BYTES * NP * NCOMP;
  static constexpr int STAGE_BYTES = A_STAGE_BYTES + B_STAGE_BYTES;
  static constexpr int LDS_BYTES = 2 * STAGE_BYTES;
  // staging units: one unit = (row, chunk of 8 K-values)
  static constexpr int UA = (BM * 4) / NT;
  static constexpr int UB = (BN * 4) / NT;
  static_assert((BM * 4) % NT == 0 && (BN * 4) % NT == 0, "tile/threads");
  static_assert(BM % WM == 0 && BN % WN == 0 && WM % 32 == 0 && WN % 32 == 0,
                "wave tile");
  static_assert(LDS_BYTES <= 160 * 1024, "LDS budget");
};

// Map a linear workgroup id to a tile so that (a) workgroups that the
// dispatcher places on the same XCD (id mod 8) work on neighbouring tiles and
// share that XCD's L2, (b) tiles are walked in column groups of GROUP tile
// rows so that the A rows / B columns in flight stay small.
__device__ inline void map_tile(uint32_t bid, uint32_t tiles_m, uint32_t tiles_n,
                                uint32_t &tm, uint32_t &tn) {
  const uint32_t total = tiles_m * tiles_n;
  constexpr uint32_t NXCD = 8;
  uint32_t id = bid;
  if (total >= NXCD * 4) {
    const uint32_t q = total / NXCD, r = total % NXCD;
    const uint32_t xcd = bid % NXCD, loc = bid / NXCD;
    // XCD x owns a contiguous range; the first r XCDs own one tile more
    id = xcd * q + (xcd < r ? xcd : r) + loc;
  }
  constexpr uint32_t GROUP = 8;
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
//         lanes; each thread reads 8 consecutive elements (vector loads).
//   !KC:  memory is row-contiguous -> unit = (row, chunk), row fastest over
//         lanes; each thread reads 8 elements `ld` apart, consecutive lanes
//         read consecutive addresses.
// Out-of-range elements read as zero, which contributes nothing to the sums.
// ---------------------------------------------------------------------------
template <bool CPLX, bool KC, int ROWS, int U, int NT>
struct tile_loader {
  // reg[u][comp] holds the 8 K-values of unit u (re or im)
  __device__ static inline void unit_coords(int u, int tid, int &row, int &chunk) {
    const int id = tid + u * NT;
    if constexpr (KC) {
      chunk = id & 3;
      row = id >> 2;
    } else {
      row = id % ROWS;
      chunk = id / ROWS;
    }
  }

  // base points at element (row 0 of the tile, k 0 of the K-step)
  template <bool FAST>
  __device__ static inline void load(f8_t (&reg)[U][CPLX ? 2 : 1],
                                     const float *__restrict__ base, uint64_t ld,
                                     int rows_left, int k_left, int tid,
                                     bool conj) {
#pragma unroll
    for (int u = 0; u < U; u++) {
      int row, chunk;
      unit_coords(u, tid, row, chunk);
      const int k0 = chunk * 8;
      if constexpr (!CPLX) {
        f8_t v;
        if constexpr (KC) {
          const float *p = base + (uint64_t)row * ld + k0;
          if constexpr (FAST) {
            const float4 lo = *reinterpret_cast<const float4 *>(p);
            const float4 hi = *reinterpret_cast<const float4 *>(p + 4);
            v[0] = lo.x; v[1] = lo.y; v[2] = lo.z; v[3] = lo.w;
            v[4] = hi.x; v[5] = hi.y; v[6] = hi.z; v[7] = hi.w;
          } else {
#pragma unroll
            for (int j = 0; j < 8; j++)
              v[j] = (row < rows_left && k0 + j < k_left) ? p[j] : 0.0f;
          }
        } else {
          const float *p = base + (uint64_t)k0 * ld + row;
#pragma unroll
          for (int j = 0; j < 8; j++) {
            if constexpr (FAST)
              v[j] = p[(uint64_t)j * ld];
            else
              v[j] = (row < rows_left && k0 + j < k_left) ? p[(uint64_t)j * ld]
                                                          : 0.0f;
          }
        }
        reg[u][0] = v;
      } else {
        f8_t re, im;
        const float2 *cb = reinterpret_cast<const float2 *>(base);
        if constexpr (KC) {
          const float2 *p = cb + (uint64_t)row * ld + k0;
          if constexpr (FAST) {
#pragma unroll
            for (int j = 0; j < 8; j += 2) {
              const float4 t = *reinterpret_cast<const float4 *>(p + j);
              re[j] = t.x; im[j] = t.y; re[j + 1] = t.z; im[j + 1] = t.w;
            }
          } else {
#pragma unroll
            for (int j = 0; j < 8; j++) {
              float2 t = make_float2(0.f, 0.f);
              if (row < rows_left && k0 + j < k_left) t = p[j];
              re[j] = t.x; im[j] = t.y;
            }
          }
        } else {
          const float2 *p = cb + (uint64_t)k0 * ld + row;
#pragma unroll
          for (int j = 0; j < 8; j++) {
            float2 t = make_float2(0.f, 0.f);
            if (FAST || (row < rows_left && k0 + j < k_left))
              t = p[(uint64_t)j * ld];
            re[j] = t.x; im[j] = t.y;
          }
        }
        if (conj) im = -im;
        reg[u][0] = re;
        reg[u][1] = im;
      }
    }
  }

  // split and write to LDS: planes laid out [comp][plane][row][chunk]
  template <Prec P>
  __device__ static inline void store(const f8_t (&reg)[U][CPLX ? 2 : 1],
                                      char *lds_op, int tid) {
    constexpr int NP = prec_traits<P>::NP;
    constexpr int PLANE = ROWS * 80;
#pragma unroll
    for (int u = 0; u < U; u++) {
      int row, chunk;
      unit_coords(u, tid, row, chunk);
#pragma unroll
      for (int c = 0; c < (CPLX ? 2 : 1); c++) {
        u4_t out[NP];
        splitter<P>::run(reg[u][c], out);
#pragma unroll
        for (int p = 0; p < NP; p++) {
          *reinterpret_cast<u4_t *>(lds_op + (c * NP + p) * PLANE + row * 80 +
                                    chunk * 16) = out[p];
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

  extern __shared__ __attribute__((aligned(16))) char lds[];

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const int wm = wave % (BM / Cfg::WM);
  const int wn = wave / (BM / Cfg::WM);

  uint32_t tile_m, tile_n;
  map_tile(blockIdx.x, args.tiles_m, args.tiles_n, tile_m, tile_n);
  const uint32_t m0 = tile_m * BM, n0 = tile_n * BN;
  const uint32_t kbeg = blockIdx.z * args.k_chunk;
  const uint32_t kend = (kbeg + args.k_chunk < args.k) ? kbeg + args.k_chunk : args.k;
  if (kbeg >= kend) return;

  const float *a = reinterpret_cast<const float *>(args.a) +
                   (uint64_t)blockIdx.y * args.stride_a * ES;
  const float *b = reinterpret_cast<const float *>(args.b) +
                   (uint64_t)blockIdx.y * args.stride_b * ES;
  float *c = reinterpret_cast<float *>(args.c) +
             (uint64_t)blockIdx.y * args.stride_c * ES;

  // operand tile origins at k = kbeg
  const float *a_tile = Cfg::A_KC ? a + ((uint64_t)m0 * args.lda + kbeg) * ES
                                  : a + ((uint64_t)kbeg * args.lda + m0) * ES;
  const float *b_tile = Cfg::B_KC ? b + ((uint64_t)n0 * args.ldb + kbeg) * ES
                                  : b + ((uint64_t)kbeg * args.ldb + n0) * ES;
  const uint64_t a_kstep = Cfg::A_KC ? (uint64_t)BK * ES : (uint64_t)BK * args.lda * ES;
  const uint64_t b_kstep = Cfg::B_KC ? (uint64_t)BK * ES : (uint64_t)BK * args.ldb * ES;

  const int rows_a = (int)((args.m - m0 < (uint32_t)BM) ? args.m - m0 : BM);
  const int rows_b = (int)((args.n - n0 < (uint32_t)BN) ? args.n - n0 : BN);
  // vector loads need 16-byte aligned rows
  const bool a_vec_ok = !Cfg::A_KC || CPLX
                            ? (!Cfg::A_KC || ((args.lda & 1) == 0 && ((uintptr_t)a_tile & 15) == 0))
                            : ((args.lda & 3) == 0 && ((uintptr_t)a_tile & 15) == 0);
  const bool b_vec_ok = !Cfg::B_KC || CPLX
                            ? (!Cfg::B_KC || ((args.ldb & 1) == 0 && ((uintptr_t)b_tile & 15) == 0))
                            : ((args.ldb & 3) == 0 && ((uintptr_t)b_tile & 15) == 0);
  const bool a_full = (rows_a == BM) && a_vec_ok;
  const bool b_full = (rows_b == BN) && b_vec_ok;

  using LA = tile_loader<CPLX, Cfg::A_KC, BM, Cfg::UA, NT>;
  using LB = tile_loader<CPLX, Cfg::B_KC, BN, Cfg::UB, NT>;
  f8_t ra[Cfg::UA][NCOMP];
  f8_t rb[Cfg::UB][NCOMP];

  // accumulators: [component][main/corr][TN][TM]; MFMA rows run along N and
  // MFMA columns along M so that a lane's 64 outputs of one register are 32
  // consecutive M-values -> coalesced column-major stores.
  f16v_t acc[NCOMP][PT::NACC][TN][TM];
#pragma unroll
  for (int q = 0; q < NCOMP; q++)
#pragma unroll
    for (int s = 0; s < PT::NACC; s++)
#pragma unroll
      for (int j = 0; j < TN; j++)
#pragma unroll
        for (int i = 0; i < TM; i++)
#pragma unroll
          for (int v = 0; v < 16; v++) acc[q][s][j][i][v] = 0.0f;

  const int nk = (int)((kend - kbeg + BK - 1) / BK);

  auto gload = [&](int kt) {
    const int k_left = (int)(kend - kbeg) - kt * BK;
    const bool kfull = k_left >= BK;
    if (a_full && kfull)
      LA::template load<true>(ra, a_tile + (uint64_t)kt * a_kstep, args.lda, rows_a, k_left, tid, args.conj_a);
    else
      LA::template load<false>(ra, a_tile + (uint64_t)kt * a_kstep, args.lda, rows_a, k_left, tid, args.conj_a);
    if (b_full && kfull)
      LB::template load<true>(rb, b_tile + (uint64_t)kt * b_kstep, args.ldb, rows_b, k_left, tid, args.conj_b);
    else
      LB::template load<false>(rb, b_tile + (uint64_t)kt * b_kstep, args.ldb, rows_b, k_left, tid, args.conj_b);
  };
  auto lstore = [&](int stage) {
    char *sa = lds + stage * Cfg::STAGE_BYTES;
    char *sb = sa + Cfg::A_STAGE_BYTES;
    LA::template store<P>(ra, sa, tid);
    LB::template store<P>(rb, sb, tid);
  };

  gload(0);
  lstore(0);
  __syncthreads();

  // per-lane fragment offsets: row = lane % 32, chunk = 2*kk + lane / 32
  const int frag_row = lane & 31;
  const int frag_chunk = lane >> 5;
  const int a_frag_off = (wm * Cfg::WM + frag_row) * 80 + frag_chunk * 16;
  const int b_frag_off = (wn * Cfg::WN + frag_row) * 80 + frag_chunk * 16;

  for (int kt = 0; kt < nk; kt++) {
    const int stage = kt & 1;
    if (kt + 1 < nk) gload(kt + 1);

    const char *sa = lds + stage * Cfg::STAGE_BYTES;
    const char *sb = sa + Cfg::A_STAGE_BYTES;
#pragma unroll
    for (int kk = 0; kk < BK / 16; kk++) {
      u4_t fa[NCOMP][NP][TM];
      u4_t fb[NCOMP][NP][TN];
#pragma unroll
      for (int q = 0; q < NCOMP; q++)
#pragma unroll
        for (int p = 0; p < NP; p++) {
#pragma unroll
          for (int i = 0; i < TM; i++)
            fa[q][p][i] = *reinterpret_cast<const u4_t *>(
                sa + (q * NP + p) * Cfg::A_PLANE_BYTES + a_frag_off + i * 32 * 80 + kk * 32);
#pragma unroll
          for (int j = 0; j < TN; j++)
            fb[q][p][j] = *reinterpret_cast<const u4_t *>(
                sb + (q * NP + p) * Cfg::B_PLANE_BYTES + b_frag_off + j * 32 * 80 + kk * 32);
        }
      if constexpr (!CPLX) {
#pragma unroll
        for (int t = 0; t < PT::NPROD; t++)
#pragma unroll
          for (int j = 0; j < TN; j++)
#pragma unroll
            for (int i = 0; i < TM; i++)
              acc[0][PT::ACC[t]][j][i] = mfma32<PT::IS_BF16>(
                  fb[0][PT::PB[t]][j], fa[0][PT::PA[t]][i], acc[0][PT::ACC[t]][j][i]);
      } else {
        // -Im(A) planes for the real part: re = ar*br + (-ai)*bi
        u4_t fan[NP][TM];
#pragma unroll
        for (int p = 0; p < NP; p++)
#pragma unroll
          for (int i = 0; i < TM; i++) fan[p][i] = fa[1][p][i] ^ 0x80008000u;
#pragma unroll
        for (int t = 0; t < PT::NPROD; t++)
#pragma unroll
          for (int j = 0; j < TN; j++)
#pragma unroll
            for (int i = 0; i < TM; i++) {
              const int s = PT::ACC[t], pa = PT::PA[t], pb = PT::PB[t];
              acc[0][s][j][i] = mfma32<PT::IS_BF16>(fb[0][pb][j], fa[0][pa][i], acc[0][s][j][i]);
              acc[1][s][j][i] = mfma32<PT::IS_BF16>(fb[1][pb][j], fa[0][pa][i], acc[1][s][j][i]);
              acc[0][s][j][i] = mfma32<PT::IS_BF16>(fb[1][pb][j], fan[pa][i], acc[0][s][j][i]);
              acc[1][s][j][i] = mfma32<PT::IS_BF16>(fb[0][pb][j], fa[1][pa][i], acc[1][s][j][i]);
            }
      }
    }

    if (kt + 1 < nk) lstore(stage ^ 1);
    __syncthreads();
  }

  // ---- epilogue -----------------------------------------------------------
  // 32x32 accumulator layout: register v of lane l holds
  //   MFMA row (-> n) = 8*(v/4) + 4*(l/32) + v%4,  MFMA column (-> m) = l%32
  const bool beta_zero = (args.beta_re == 0.0f) && (!CPLX || args.beta_im == 0.0f);
#pragma unroll
  for (int j = 0; j < TN; j++)
#pragma unroll
    for (int i = 0; i < TM; i++) {
      const uint32_t mm = m0 + wm * Cfg::WM + i * 32 + (lane & 31);
#pragma unroll
      for (int v = 0; v < 16; v++) {
        const uint32_t nn = n0 + wn * Cfg::WN + j * 32 + 8 * (v / 4) + 4 * (lane >> 5) + (v & 3);
        if (mm < args.m && nn < args.n) {
          float *cp = c + ((uint64_t)nn * args.ldc + mm) * ES;
          if constexpr (!CPLX) {
            float x = acc[0][0][j][i][v];
            if constexpr (PT::NACC == 2) x += acc[0][1][j][i][v] * PT::CORR_SCALE;
            if (args.atomic_out) {
              atomicAdd(cp, x * args.alpha_re);
            } else if (beta_zero) {
              *cp = x * args.alpha_re;
            } else {
              *cp = x * args.alpha_re + args.beta_re * (*cp);
            }
          } else {
            float x = acc[0][0][j][i][v], y = acc[1][0][j][i][v];
            if constexpr (PT::NACC == 2) {
              x += acc[0][1][j][i][v] * PT::CORR_SCALE;
              y += acc[1][1][j][i][v] * PT::CORR_SCALE;
            }
            float rx = x * args.alpha_re - y * args.alpha_im;
            float ry = y * args.alpha_re + x * args.alpha_im;
            if (args.atomic_out) {
              atomicAdd(cp, rx);
              atomicAdd(cp + 1, ry);
            } else {
              if (!beta_zero) {
                const float2 old = *reinterpret_cast<const float2 *>(cp);
                rx = x * args.alpha_re - y * args.alpha_im +
                     (args.beta_re * old.x - args.beta_im * old.y);
                ry = y * args.alpha_re + x * args.alpha_im +
                     (args.beta_im * old.x + args.beta_re * old.y);
              }
              *reinterpret_cast<float2 *>(cp) = make_float2(rx, ry);
            }
          }
        }
      }
    }
}

// C (m x n, ldc, batched) *= beta before a split-K accumulation, or = 0.
template <bool CPLX>
__global__ void prescale_c_kernel(float *c, uint32_t m, uint32_t n, uint64_t ldc,
                                  uint64_t stride_c, float beta_re, float beta_im) {
  const uint64_t total = (uint64_t)m * n;
  float *cb = c + (uint64_t)blockIdx.y * stride_c * (CPLX ? 2 : 1);
  for (uint64_t id = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x; id < total;
       id += (uint64_t)gridDim.x * blockDim.x) {
    const uint64_t i = id % m, j = id / m;
    if constexpr (!CPLX) {
      float *p = cb + j * ldc + i;
      *p = (beta_re == 0.0f) ? 0.0f : beta_re * (*p);
    } else {
      float2 *p = reinterpret_cast<float2 *>(cb) + j * ldc + i;
      if (beta_re == 0.0f && beta_im == 0.0f) {
        *p = make_float2(0.f, 0.f);
      } else {
        const float2 o = *p;
        *p = make_float2(beta_re * o.x - beta_im * o.y, beta_im * o.x + beta_re * o.y);
      }
    }
  }
}

} // namespace cumpsgemm_amd
