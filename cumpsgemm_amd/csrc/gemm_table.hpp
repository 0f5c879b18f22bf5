// gfx950 tile-configuration table: for every (precision, real/complex, layout
// of A, layout of B) a short list of kernel instances ordered from the largest
// tile to the smallest.  The host picks by problem shape (see gemm_host.hip).
// This table is what takes the place of the reference's per-architecture
// instance tables and kernel_module_code keys (src/instance.hpp:33-63,
// src/instance_sm80.cu, src/cumpsgemm.cu:19-89).
#pragma once
#include "gemm_kernel.hpp"
#include <atomic>

namespace cumpsgemm_amd {

struct KernelEntry {
  void (*launch)(const GemmArgs &, dim3 grid, hipStream_t stream);
  // persistent variant (grid.x = CU slots, walks tiles and batches itself), or
  // nullptr; only for shapes made of interior, aligned tiles
  void (*launch_persistent)(const GemmArgs &, dim3 grid, hipStream_t stream);
  // variants with the power-of-two scaling of A, B and C fused in (FP16TCEC
  // tables only, else nullptr)
  void (*launch_scaled)(const GemmArgs &, dim3 grid, hipStream_t stream);
  void (*launch_scaled_persistent)(const GemmArgs &, dim3 grid, hipStream_t stream);
  // variant with twice the waves, each group taking one K-slice of every step
  // (small real tiles only, else nullptr): for problems of no more tiles than CUs
  void (*launch_kslices)(const GemmArgs &, dim3 grid, hipStream_t stream);
  void (*launch_scaled_kslices)(const GemmArgs &, dim3 grid, hipStream_t stream); // (FP16TCEC tables only)
  // the persistent variants on 16x16x32 MFMAs (real FP16TCEC 256x128 and 128x128,
  // real bf16x3 128x128, real FP16TC 256x128; else nullptr): for launches that fill the chip
  void (*launch_persistent_edge16)(const GemmArgs &, dim3 grid, hipStream_t stream);
  void (*launch_scaled_persistent_edge16)(const GemmArgs &, dim3 grid, hipStream_t stream);
  int bm, bn;      // workgroup tile
  int wm, wn;      // wave tile
  int threads;     // workgroup size
  int lds_bytes;   // dynamic LDS per workgroup
  int occ;         // waves per SIMD the kernel was compiled for
  const char *name;
};

constexpr int kNumTileClasses = 5; // 0 = large ... 2 = small, 3 = tall-skinny C, 4 = short-wide C

// layout index = (a_kc ? 1 : 0) + (b_kc ? 2 : 0)
const KernelEntry *lookup_kernel(Prec p, bool cplx, bool a_kc, bool b_kc, int cls);

// Everything a first launch of this kernel would set up behind the caller's
// back -- loading its code object onto the current device (which allocates
// device memory) and lifting the dynamic-LDS limit -- done ahead of time.
template <class Cfg>
void prepare_cfg() {
  hipFuncAttributes attr;
  (void)hipFuncGetAttributes(&attr, reinterpret_cast<const void *>(&gemm_tcec_kernel<Cfg>));
  if (Cfg::LDS_BYTES > 64 * 1024)
    (void)hipFuncSetAttribute(reinterpret_cast<const void *>(&gemm_tcec_kernel<Cfg>),
                              hipFuncAttributeMaxDynamicSharedMemorySize, Cfg::LDS_BYTES);
  (void)hipGetLastError();
}

template <class Cfg>
void launch_cfg(const GemmArgs &args, dim3 grid, hipStream_t stream) {
  if (Cfg::LDS_BYTES > 64 * 1024) {
    // more than 64 KiB of dynamic LDS must be allowed once per kernel and device
    // (setting it twice is harmless, so threads that race here only need the
    // flag itself to be free of a data race)
    static std::atomic<bool> attr_done[64] = {};
    int dev = 0;
    (void)hipGetDevice(&dev);
    if (dev < 0 || dev >= 64 || !attr_done[dev].load(std::memory_order_acquire)) {
      (void)hipFuncSetAttribute(reinterpret_cast<const void *>(&gemm_tcec_kernel<Cfg>),
                                hipFuncAttributeMaxDynamicSharedMemorySize, Cfg::LDS_BYTES);
      if (dev >= 0 && dev < 64) attr_done[dev].store(true, std::memory_order_release);
    }
  }
  hipLaunchKernelGGL(gemm_tcec_kernel<Cfg>, grid, dim3(Cfg::NT), Cfg::LDS_BYTES, stream, args);
}

template <class Cfg> constexpr KernelEntry make_entry(const char *name) {
  KernelEntry e{};
  e.launch = &launch_cfg<Cfg>;
  if constexpr (Cfg::DEEP) e.launch_persistent = &launch_cfg<typename Cfg::persistent_type>;
  if constexpr (Cfg::P == Prec::FP16TCEC) {
    e.launch_scaled = &launch_cfg<typename Cfg::scaled_type>;
    if constexpr (Cfg::DEEP)
      e.launch_scaled_persistent = &launch_cfg<typename Cfg::scaled_type::persistent_type>;
  }
  if constexpr (!Cfg::DEEP && Cfg::MT == 32 && Cfg::BM * 4 + Cfg::BN * 4 == 2 * Cfg::NT) {
    e.launch_kslices = &launch_cfg<GemmCfg<Cfg::P, Cfg::CPLX, Cfg::A_KC, Cfg::B_KC, Cfg::BM, Cfg::BN, Cfg::WM,
                                           Cfg::WN, Cfg::OCC, false, false, false, false, true>>;
    if constexpr (Cfg::P == Prec::FP16TCEC) {
      e.launch_scaled_kslices = &launch_cfg<GemmCfg<Cfg::P, Cfg::CPLX, Cfg::A_KC, Cfg::B_KC, Cfg::BM, Cfg::BN,
                                                    Cfg::WM, Cfg::WN, Cfg::OCC, false, false, true, false, true>>;
    }
  }
  if constexpr (Cfg::HAS_EDGE16_TWIN) {
    e.launch_persistent_edge16 = &launch_cfg<typename Cfg::persistent_type::edge16_type>;
    if constexpr (Cfg::P == Prec::FP16TCEC)
      e.launch_scaled_persistent_edge16 = &launch_cfg<typename Cfg::scaled_type::persistent_type::edge16_type>;
  }
  e.bm = Cfg::BM;
  e.bn = Cfg::BN;
  e.wm = Cfg::WM;
  e.wn = Cfg::WN;
  e.threads = Cfg::NT;
  e.lds_bytes = Cfg::LDS_BYTES;
  e.occ = Cfg::OCC;
  e.name = name;
  return e;
}

// Per-(precision, type) tables, one translation unit each (gemm_inst_*.hip).
// Indexed [layout][class].
#define CUMPSGEMM_DECLARE_TABLE(sym) extern KernelEntry sym[4][kNumTileClasses];
CUMPSGEMM_DECLARE_TABLE(g_tab_fp16tcec_s)
CUMPSGEMM_DECLARE_TABLE(g_tab_fp16tcec_c)
CUMPSGEMM_DECLARE_TABLE(g_tab_fp16tc_s)
CUMPSGEMM_DECLARE_TABLE(g_tab_fp16tc_c)
CUMPSGEMM_DECLARE_TABLE(g_tab_bf16x3_s)
CUMPSGEMM_DECLARE_TABLE(g_tab_bf16x3_c)
CUMPSGEMM_DECLARE_TABLE(g_tab_bf16x2_s)
CUMPSGEMM_DECLARE_TABLE(g_tab_bf16x2_c)
#undef CUMPSGEMM_DECLARE_TABLE

// Real FP16TCEC, 256x128 tile, persistent, operands pre-split by launch_pack_split.
void launch_packed_fp16tcec_s(const GemmArgs &args, dim3 grid, hipStream_t stream, bool walk);
void launch_packed_scaled_fp16tcec_s(const GemmArgs &args, dim3 grid, hipStream_t stream, bool walk);
void launch_packed_bf16x3_s(const GemmArgs &args, dim3 grid, hipStream_t stream, bool walk);
// the uncorrected modes, 256x128 tile: one fp16 plane (FP16TC), two bf16 planes (TF32TC's stand-in)
void launch_packed_fp16tc_s(const GemmArgs &args, dim3 grid, hipStream_t stream, bool walk);
void launch_packed_bf16x2_s(const GemmArgs &args, dim3 grid, hipStream_t stream, bool walk);
void launch_packed_fp16tc_c(const GemmArgs &args, dim3 grid, hipStream_t stream, bool walk);  // complex, 128x64
void launch_packed_bf16x2_c(const GemmArgs &args, dim3 grid, hipStream_t stream, bool walk);
void launch_packed_bf16x3_c(const GemmArgs &args, dim3 grid, hipStream_t stream); // complex, 128x64, two LDS buffers
// load the real pre-split kernels (GEMM and pre-pass) onto the current device
void prepare_packed_fp16tcec_s();
void prepare_packed_bf16x3_s();
void prepare_pack_split_real();
constexpr int kPackedBM = 256, kPackedBN = 128;             // FP16TCEC
constexpr int kPackedBf16BM = 128, kPackedBf16BN = 128;     // bf16x3
void launch_packed_fp16tcec_c(const GemmArgs &args, dim3 grid, hipStream_t stream, bool walk, bool scaled);
constexpr int kPackedCplxBM = 128, kPackedCplxBN = 64;      // complex FP16TCEC

// One table = the same three tile classes for each of the four layout pairs.
// ROW(AKC, BKC) must expand to three make_entry<...>() initialisers.
#define CUMPSGEMM_DEFINE_TABLE(sym, ROW)                                                       \
  KernelEntry sym[4][kNumTileClasses] = {ROW(false, false), ROW(true, false), ROW(false, true), \
                                         ROW(true, true)};
#define CUMPSGEMM_ENTRY(P, CPLX, AKC, BKC, BM, BN, WM, WN, OCC, DEEP, NAME) \
  make_entry<GemmCfg<P, CPLX, AKC, BKC, BM, BN, WM, WN, OCC, DEEP>>(NAME)

} // namespace cumpsgemm_amd
