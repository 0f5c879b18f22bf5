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
#undef ROW
} // namespace cumpsgemm_amd
