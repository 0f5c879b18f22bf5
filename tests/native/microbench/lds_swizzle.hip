// Micro-benchmark: which XOR swizzle of 64-byte LDS rows lets the fragment read
// of a 16x16x32 MFMA (lane l: row l % 16, 16-byte chunk l / 16) go without
// bank conflicts?  Launch i (0 .. 255) uses the masks m0 = i & 15, m1 = i >> 4:
// chunk ^= parity(row & m0) | parity(row & m1) << 1.  Launch 256 is the
// control: the 32x32x16 pattern (row l % 32, chunk l / 32) with the swizzle of
// the kernels that split in their K loop.  Meant to run under
//   rocprofv3 --pmc SQ_LDS_BANK_CONFLICT SQ_INSTS_LDS_LOAD -- lds_swizzle
// whose per-dispatch counters (in launch order) are the result.
#include <hip/hip_runtime.h>
#include <cstdio>
typedef unsigned u4_t __attribute__((ext_vector_type(4)));
__global__ __launch_bounds__(512) void k(int m0, int m1, int control, unsigned *sink) {
  __shared__ __attribute__((aligned(16))) char lds[64 * 1024];
  for (int i = threadIdx.x; i < 16 * 1024; i += blockDim.x) reinterpret_cast<unsigned *>(lds)[i] = i;
  __syncthreads();
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  int row, chunk, s;
  if (control) {
    row = lane & 31; chunk = lane >> 5;
    s = (((row >> 1) ^ (row >> 3)) & 1) | (((row >> 2) & 1) << 1);
  } else {
    row = lane & 15; chunk = lane >> 4;
    s = (__builtin_popcount(row & m0) & 1) | ((__builtin_popcount(row & m1) & 1) << 1);
  }
  const int off = wave * 4096 + row * 64 + ((chunk ^ s) << 4);
  u4_t acc = {0, 0, 0, 0};
  for (int it = 0; it < 256; it++) {
    const u4_t v = *reinterpret_cast<const u4_t *>(lds + off + (it & 3) * 1024);
    acc += v;
    asm volatile("" ::: "memory");
  }
  if (acc[0] + acc[1] + acc[2] + acc[3] == 0x12345) sink[0] = 1;
}
int main() {
  unsigned *sink;
  if (hipMalloc(&sink, 64) != hipSuccess) return 1;
  for (int i = 0; i <= 256; i++) hipLaunchKernelGGL(k, dim3(8), dim3(512), 0, 0, i & 15, i >> 4, i == 256, sink);
  hipError_t e = hipDeviceSynchronize();
  printf("status %s\n", hipGetErrorString(e));
  return e != hipSuccess;
}
