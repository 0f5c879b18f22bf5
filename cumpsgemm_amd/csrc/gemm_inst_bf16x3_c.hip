// Kernel instances of the tile table for one (precision, element type) pair.
#include "gemm_table.hpp"
namespace cumpsgemm_amd {
CUMPSGEMM_DEFINE_TABLE(g_tab_bf16x3_c, CUMPSGEMM_CPLX_ROW, Prec::BF16X3)
} // namespace cumpsgemm_amd
