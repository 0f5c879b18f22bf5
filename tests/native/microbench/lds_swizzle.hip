// Micro-benchmark: which XOR swizzle of 64-byte LDS rows lets an access pattern
// of the GEMM kernels go without bank conflicts?  Launch i of a pattern
// (0 .. 255) uses the masks m0 = i & 15, m1 = i >> 4:
//   chunk ^= parity(row & m0) | parity(row & m1) << 1.
// Patterns (lane l of a wave; a row holds four 16-byte chunks):
//   0  fragment read of a 16x16x32 MFMA: ds_read_b128, row l % 16, chunk l / 16
//   1  fragment read of a 32x32x16 MFMA: ds_read_b128, row l % 32, chunk l / 32
//   2  staging write, K-contiguous operand: ds_write_b128, row l / 4, chunk l % 4
//   3  staging write, row-contiguous operand: ds_write_b128, row l, one chunk
//   4  half-unit staging write, K-contiguous: ds_write_b64, row l / 8, chunk (l / 2) % 4, half l % 2
//   5  half-unit staging write, row-contiguous: ds_write_b64, row l / 2, one chunk, half l % 2
// Meant to run under
//   rocprofv3 --pmc SQ_LDS_BANK_CONFLICT SQ_INSTS_LDS_LOAD SQ_INSTS_LDS_STORE -- lds_swizzle
// whose per-dispatch counters, in launch order (pattern-major, 256 launches
// each), are the result.
#include <hip/hip_runtime.h>
#include <cstdio>
typedef unsigned u4_t __attribute__((ext_vector_type(4)));
typedef unsigned u2_t __attribute__((ext_vector_type(2)));
__global__ __launch_bounds__(512) void k(int m0, int m1, int pattern, unsigned *sink) {
  __shared__ __attribute__((aligned(16))) char lds[64 * 1024];
  for (int i = threadIdx.x; i < 16 * 1024; i += blockDim.x) reinterpret_cast<unsigned *>(lds)[i] = i;
  __syncthreads();
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  int row, chunk, half = 0;
  switch (pattern) {
  case 0: row = lane & 15; chunk = lane >> 4; break;
  case 1: row = lane & 31; chunk = lane >> 5; break;
  case 2: row = lane >> 2; chunk = lane & 3; break;
  case 3: row = lane; chunk = wave & 3; break;
  case 4: row = lane >> 3; chunk = (lane >> 1) & 3; half = lane & 1; break;
  default: row = lane >> 1; chunk = wave & 3; half = lane & 1; break;
  }
  const int s = (__builtin_popcount(row & m0) & 1) | ((__builtin_popcount(row & m1) & 1) << 1);
  // (each wave works in its own 8 KiB: 64 rows of 64 bytes, twice)
  const int off = wave * 8192 + row * 64 + ((chunk ^ s) << 4) + half * 8;
  u4_t acc = {0, 0, 0, 0};
  for (int it = 0; it < 256; it++) {
    char *p = lds + off + (it & 1) * 4096;
    if (pattern < 2) {
      acc += *reinterpret_cast<const u4_t *>(p);
    } else if (pattern < 4) {
      *reinterpret_cast<u4_t *>(p) = acc;
      acc[0] += it;
    } else {
      u2_t v = {acc[0], acc[1]};
      *reinterpret_cast<u2_t *>(p) = v;
      acc[0] += it;
    }
    asm volatile("" ::: "memory");
  }
  __syncthreads();
  if (acc[0] + acc[1] + acc[2] + acc[3] + lds[off] == 0x12345) sink[0] = 1;
}
int main() {
  unsigned *sink;
  if (hipMalloc(&sink, 64) != hipSuccess) return 1;
  for (int pattern = 0; pattern < 6; pattern++)
    for (int i = 0; i < 256; i++) hipLaunchKernelGGL(k, dim3(8), dim3(512), 0, 0, i & 15, i >> 4, pattern, sink);
  hipError_t e = hipDeviceSynchronize();
  printf("status %s\n", hipGetErrorString(e));
  return e != hipSuccess;
}
