// Kernel instances of the tile table for one (precision, element type) pair.
#include "gemm_table.hpp"
namespace cumpsgemm_amd {
CUMPSGEMM_DEFINE_TABLE(g_tab_fp16tcec_c, CUMPSGEMM_CPLX_ROW, Prec::FP16TCEC)
} // namespace cumpsgemm_amd
