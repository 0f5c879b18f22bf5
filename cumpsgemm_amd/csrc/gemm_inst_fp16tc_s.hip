// Kernel instances of the tile table for one (precision, element type) pair:
// three tile classes (large, medium, small) for each layout pair.
#include "gemm_table.hpp"
namespace cumpsgemm_amd {
#define ROW(AKC, BKC) \
  { CUMPSGEMM_ENTRY(Prec::FP16TC, false, AKC, BKC, 256, 128, 64, 64, 2, true, "256x128x32_w64x64_deep"), \
    CUMPSGEMM_ENTRY(Prec::FP16TC, false, AKC, BKC, 128, 128, 64, 32, 2, true, "128x128x32_w64x32_deep"), \
    CUMPSGEMM_ENTRY(Prec::FP16TC, false, AKC, BKC, 64, 64, 32, 32, 2, false, "64x64x32_w32x32"), \
    CUMPSGEMM_ENTRY(Prec::FP16TC, false, AKC, BKC, 64, 64, 32, 32, 2, false, "64x64x32_w32x32"), \
    CUMPSGEMM_ENTRY(Prec::FP16TC, false, AKC, BKC, 64, 64, 32, 32, 2, false, "64x64x32_w32x32") }
CUMPSGEMM_DEFINE_TABLE(g_tab_fp16tc_s, ROW)
#undef ROW
// the large tile over pre-split operands (one fp16 plane, K-contiguous);
// `walk`: persistent form (short tiles) or one tile per workgroup.  The one-tile
// form has a single accumulator set and no staging registers: built for four
// waves per SIMD (96 registers), so that two workgroups share a CU and one of
// them multiplies while the other waits at its K-step barrier.
void launch_packed_fp16tc_s(const GemmArgs &args, dim3 grid, hipStream_t stream, bool walk) {
  if (walk) {
    launch_cfg<GemmCfg<Prec::FP16TC, false, true, true, 256, 128, 64, 64, 2, true, true, false, true>>(
        args, grid, stream);
  } else {
    launch_cfg<GemmCfg<Prec::FP16TC, false, true, true, 256, 128, 64, 64, 4, true, false, false, true>>(
        args, grid, stream);
  }
}
} // namespace cumpsgemm_amd
