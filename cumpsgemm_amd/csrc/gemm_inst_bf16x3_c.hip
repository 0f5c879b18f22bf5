// Kernel instances of the tile table for one (precision, element type) pair:
// three tile classes (large, medium, small) for each layout pair.
#include "gemm_table.hpp"
namespace cumpsgemm_amd {
#define ROW(AKC, BKC) \
  { CUMPSGEMM_ENTRY(Prec::BF16X3, true, AKC, BKC, 128, 64, 32, 32, 2, false, "c128x64x32_w32x32"), \
    CUMPSGEMM_ENTRY(Prec::BF16X3, true, AKC, BKC, 64, 64, 32, 32, 2, false, "c64x64x32_w32x32"), \
    CUMPSGEMM_ENTRY(Prec::BF16X3, true, AKC, BKC, 64, 32, 32, 32, 1, false, "c64x32x32_w32x32"), \
    CUMPSGEMM_ENTRY(Prec::BF16X3, true, AKC, BKC, 64, 32, 32, 32, 1, false, "c64x32x32_w32x32"), \
    CUMPSGEMM_ENTRY(Prec::BF16X3, true, AKC, BKC, 64, 32, 32, 32, 1, false, "c64x32x32_w32x32") }
CUMPSGEMM_DEFINE_TABLE(g_tab_bf16x3_c, ROW)
// the large complex tile over pre-split operands (planes re b0, b1, b2, im b0,
// b1, b2; K-contiguous): two LDS buffers, one tile per workgroup
void launch_packed_bf16x3_c(const GemmArgs &args, dim3 grid, hipStream_t stream) {
  launch_cfg<GemmCfg<Prec::BF16X3, true, true, true, 128, 64, 32, 32, 2, false, false, false, true>>(args, grid, stream);
}
#undef ROW
} // namespace cumpsgemm_amd
