// Pre-split of an FP32 operand into fp16 or bf16 planes (see pack_split.hip):
// hi / lo fp16 (FP16TCEC), three or two bf16 terms (bf16x3, bf16x2) or the
// plain fp16 conversion (FP16TC).
#pragma once
#include <hip/hip_runtime.h>
#include <cstdint>

namespace cumpsgemm_amd {
// bytes of the packed form of a (rows x k) operand
inline uint64_t packed_bytes(uint64_t rows_pad, uint64_t k, unsigned planes = 2) {
  return ((k + 31) / 32) * planes * rows_pad * 64;
}
inline uint32_t packed_rows(uint64_t rows) { return (uint32_t)((rows + 255) / 256 * 256); }
enum class PackKind {
  FP16_REAL, FP16_COMPLEX, BF16X3_REAL, FP16TC_REAL, BF16X2_REAL, FP16TC_COMPLEX, BF16X2_COMPLEX, BF16X3_COMPLEX
};
// One pre-pass launch converts both operands of a GEMM (same K).  `ld` in
// elements of the source (complex: complex elements).  scale_max / scale_flag:
// optional power-of-two scaling fused into the split (nullptr: none; A's is
// governed by bit 0x40 of *scale_flag, B's by bit 0x20); launch_flag /
// flag_accept_mask: optional AUTO-mode gate, as in GemmArgs.
struct PackOperand {
  const float *src;
  bool k_contiguous;
  uint64_t ld;
  uint32_t rows;
  void *dst;
  uint32_t rows_pad;
  const uint32_t *scale_max; // nullptr: no scaling
};
void prepare_pack_split_real();
void launch_pack_split_pair(hipStream_t stream, const PackOperand &a, const PackOperand &b, uint32_t k,
                            PackKind kind, const int *scale_flag = nullptr, const int *launch_flag = nullptr,
                            uint32_t flag_accept_mask = 0);
} // namespace cumpsgemm_amd
