// Kernel instances of the tile table for one (precision, element type) pair:
// three tile classes (large, medium, small) for each layout pair.
#include "gemm_table.hpp"
namespace cumpsgemm_amd {
#define ROW(AKC, BKC) \
  { CUMPSGEMM_ENTRY(Prec::BF16X3, false, AKC, BKC, 256, 128, 64, 64, 2, false, "256x128x32_w64x64"), \
    CUMPSGEMM_ENTRY(Prec::BF16X3, false, AKC, BKC, 128, 128, 64, 32, 2, true, "128x128x32_w64x32_deep"), \
    CUMPSGEMM_ENTRY(Prec::BF16X3, false, AKC, BKC, 64, 64, 32, 32, 2, false, "64x64x32_w32x32"), \
    CUMPSGEMM_ENTRY(Prec::BF16X3, false, AKC, BKC, 128, 32, 32, 32, 2, true, "128x32x32_w32x32_deep"), \
    CUMPSGEMM_ENTRY(Prec::BF16X3, false, AKC, BKC, 32, 128, 32, 32, 2, true, "32x128x32_w32x32_deep") }
CUMPSGEMM_DEFINE_TABLE(g_tab_bf16x3_s, ROW)
// the large tile over pre-split operands (three bf16 planes, K-contiguous);
// `walk`: persistent form (short tiles) or one tile per workgroup
void launch_packed_bf16x3_s(const GemmArgs &args, dim3 grid, hipStream_t stream, bool walk) {
  if (walk) {
    launch_cfg<GemmCfg<Prec::BF16X3, false, true, true, 128, 128, 64, 32, 2, true, true, false, true>>(
        args, grid, stream);
  } else {
    launch_cfg<GemmCfg<Prec::BF16X3, false, true, true, 128, 128, 64, 32, 2, true, false, false, true>>(
        args, grid, stream);
  }
}
void prepare_packed_bf16x3_s() {
  prepare_cfg<GemmCfg<Prec::BF16X3, false, true, true, 128, 128, 64, 32, 2, true, true, false, true>>();
  prepare_cfg<GemmCfg<Prec::BF16X3, false, true, true, 128, 128, 64, 32, 2, true, false, false, true>>();
}
#undef ROW
} // namespace cumpsgemm_amd
