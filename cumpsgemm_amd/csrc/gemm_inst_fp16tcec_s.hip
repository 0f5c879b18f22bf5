// Kernel instances of the tile table for one (precision, element type) pair:
// three tile classes (large, medium, small) for each layout pair.
#include "gemm_table.hpp"
namespace cumpsgemm_amd {
#define ROW(AKC, BKC) \
  { CUMPSGEMM_ENTRY(Prec::FP16TCEC, false, AKC, BKC, 256, 128, 64, 64, 2, true, "256x128x32_w64x64_deep"), \
    CUMPSGEMM_ENTRY(Prec::FP16TCEC, false, AKC, BKC, 128, 128, 64, 32, 2, true, "128x128x32_w64x32_deep"), \
    CUMPSGEMM_ENTRY(Prec::FP16TCEC, false, AKC, BKC, 64, 64, 32, 32, 2, false, "64x64x32_w32x32"), \
    CUMPSGEMM_ENTRY(Prec::FP16TCEC, false, AKC, BKC, 256, 32, 32, 32, 2, true, "256x32x32_w32x32_deep"), \
    CUMPSGEMM_ENTRY(Prec::FP16TCEC, false, AKC, BKC, 32, 256, 32, 32, 2, true, "32x256x32_w32x32_deep") }
// Both operands M/N-contiguous ("NT": op_A = N, op_B = T): the large class is the
// transposed tile, 128 x 256.  Measured with the split in the K loop, 128x256
// against 256x128: 4096^2 x 1024 315 / 270, 8192^2 x 1024 323 / 292, 16384^2 x 256
// 245 / 236, 8192^3 364 / 366 TFLOP/s; for the three other layouts the two
// tiles are within 2 % of each other at every size.
#define ROW_NT(AKC, BKC) \
  { CUMPSGEMM_ENTRY(Prec::FP16TCEC, false, AKC, BKC, 128, 256, 64, 64, 2, true, "128x256x32_w64x64_deep"), \
    CUMPSGEMM_ENTRY(Prec::FP16TCEC, false, AKC, BKC, 128, 128, 64, 32, 2, true, "128x128x32_w64x32_deep"), \
    CUMPSGEMM_ENTRY(Prec::FP16TCEC, false, AKC, BKC, 64, 64, 32, 32, 2, false, "64x64x32_w32x32"), \
    CUMPSGEMM_ENTRY(Prec::FP16TCEC, false, AKC, BKC, 256, 32, 32, 32, 2, true, "256x32x32_w32x32_deep"), \
    CUMPSGEMM_ENTRY(Prec::FP16TCEC, false, AKC, BKC, 32, 256, 32, 32, 2, true, "32x256x32_w32x32_deep") }
KernelEntry g_tab_fp16tcec_s[4][kNumTileClasses] = {ROW_NT(false, false), ROW(true, false), ROW(false, true),
                                                    ROW(true, true)};
#undef ROW_NT
// the large tile over pre-split operands (one layout: planes are K-contiguous);
// `walk`: persistent form (short tiles) or one tile per workgroup
void launch_packed_fp16tcec_s(const GemmArgs &args, dim3 grid, hipStream_t stream, bool walk) {
  if (walk) {
    launch_cfg<GemmCfg<Prec::FP16TCEC, false, true, true, 256, 128, 64, 64, 2, true, true, false, true>>(
        args, grid, stream);
  } else {
    launch_cfg<GemmCfg<Prec::FP16TCEC, false, true, true, 256, 128, 64, 64, 2, true, false, false, true>>(
        args, grid, stream);
  }
}
void prepare_packed_fp16tcec_s() {
  prepare_cfg<GemmCfg<Prec::FP16TCEC, false, true, true, 256, 128, 64, 64, 2, true, true, false, true>>();
  prepare_cfg<GemmCfg<Prec::FP16TCEC, false, true, true, 256, 128, 64, 64, 2, true, false, false, true>>();
}
void launch_packed_scaled_fp16tcec_s(const GemmArgs &args, dim3 grid, hipStream_t stream, bool walk) {
  if (walk) {
    launch_cfg<GemmCfg<Prec::FP16TCEC, false, true, true, 256, 128, 64, 64, 2, true, true, true, true>>(
        args, grid, stream);
  } else {
    launch_cfg<GemmCfg<Prec::FP16TCEC, false, true, true, 256, 128, 64, 64, 2, true, false, true, true>>(
        args, grid, stream);
  }
}
#undef ROW
} // namespace cumpsgemm_amd
