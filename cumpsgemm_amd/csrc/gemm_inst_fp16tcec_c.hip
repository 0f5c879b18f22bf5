// Kernel instances of the tile table for one (precision, element type) pair:
// three tile classes (large, medium, small) for each layout pair.
#include "gemm_table.hpp"
namespace cumpsgemm_amd {
#define ROW(AKC, BKC) \
  { CUMPSGEMM_ENTRY(Prec::FP16TCEC, true, AKC, BKC, 128, 64, 32, 32, 2, true, "c128x64x32_w32x32_deep"), \
    CUMPSGEMM_ENTRY(Prec::FP16TCEC, true, AKC, BKC, 64, 64, 32, 32, 2, false, "c64x64x32_w32x32"), \
    CUMPSGEMM_ENTRY(Prec::FP16TCEC, true, AKC, BKC, 64, 32, 32, 32, 1, false, "c64x32x32_w32x32"), \
    CUMPSGEMM_ENTRY(Prec::FP16TCEC, true, AKC, BKC, 64, 32, 32, 32, 1, false, "c64x32x32_w32x32"), \
    CUMPSGEMM_ENTRY(Prec::FP16TCEC, true, AKC, BKC, 64, 32, 32, 32, 1, false, "c64x32x32_w32x32") }
CUMPSGEMM_DEFINE_TABLE(g_tab_fp16tcec_c, ROW)
// the large tile over pre-split operands (planes re hi, re lo, im hi, im lo;
// one layout: planes are K-contiguous); `walk`: persistent form or one tile
// per workgroup; `scaled`: the inverse scaling of C folded into alpha
void launch_packed_fp16tcec_c(const GemmArgs &args, dim3 grid, hipStream_t stream, bool walk, bool scaled) {
  if (scaled) {
    if (walk) launch_cfg<GemmCfg<Prec::FP16TCEC, true, true, true, 128, 64, 32, 32, 2, true, true, true, true>>(args, grid, stream);
    else launch_cfg<GemmCfg<Prec::FP16TCEC, true, true, true, 128, 64, 32, 32, 2, true, false, true, true>>(args, grid, stream);
  } else {
    if (walk) launch_cfg<GemmCfg<Prec::FP16TCEC, true, true, true, 128, 64, 32, 32, 2, true, true, false, true>>(args, grid, stream);
    else launch_cfg<GemmCfg<Prec::FP16TCEC, true, true, true, 128, 64, 32, 32, 2, true, false, false, true>>(args, grid, stream);
  }
}
#undef ROW
} // namespace cumpsgemm_amd
