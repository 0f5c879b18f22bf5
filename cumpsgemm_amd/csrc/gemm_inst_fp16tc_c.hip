// Kernel instances of the tile table for one (precision, element type) pair:
// three tile classes (large, medium, small) for each layout pair.
#include "gemm_table.hpp"
namespace cumpsgemm_amd {
#define ROW(AKC, BKC) \
  { CUMPSGEMM_ENTRY(Prec::FP16TC, true, AKC, BKC, 128, 64, 32, 32, 2, true, "c128x64x32_w32x32_deep"), \
    CUMPSGEMM_ENTRY(Prec::FP16TC, true, AKC, BKC, 64, 64, 32, 32, 2, false, "c64x64x32_w32x32"), \
    CUMPSGEMM_ENTRY(Prec::FP16TC, true, AKC, BKC, 64, 32, 32, 32, 1, false, "c64x32x32_w32x32"), \
    CUMPSGEMM_ENTRY(Prec::FP16TC, true, AKC, BKC, 64, 32, 32, 32, 1, false, "c64x32x32_w32x32"), \
    CUMPSGEMM_ENTRY(Prec::FP16TC, true, AKC, BKC, 64, 32, 32, 32, 1, false, "c64x32x32_w32x32") }
CUMPSGEMM_DEFINE_TABLE(g_tab_fp16tc_c, ROW)
#undef ROW
// the large complex tile over pre-split operands (planes re, im; K-contiguous);
// `walk`: persistent form or one tile per workgroup (64 accumulator registers:
// built for four waves per SIMD, two workgroups per CU)
void launch_packed_fp16tc_c(const GemmArgs &args, dim3 grid, hipStream_t stream, bool walk) {
  if (walk) launch_cfg<GemmCfg<Prec::FP16TC, true, true, true, 128, 64, 32, 32, 2, true, true, false, true>>(args, grid, stream);
  else launch_cfg<GemmCfg<Prec::FP16TC, true, true, true, 128, 64, 32, 32, 4, true, false, false, true>>(args, grid, stream);
}
} // namespace cumpsgemm_amd
