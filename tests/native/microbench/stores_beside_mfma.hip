// Micro-benchmark: do streaming stores cost MFMA time?  Eight waves per CU
// issue 24 independent 32x32x16 MFMAs per step, then idle (s_sleep) and meet at
// a barrier, like a K-step of a GEMM with gaps; the stores of a step come from
// extra writer waves, from the MFMA waves in a cluster, or from the MFMA waves
// one at a time between their MFMAs.
//   usage: stores_beside_mfma [steps, default 2000] [stores per wave and step: 4 or 8]
#include <hip/hip_runtime.h>
#include <cstdio>
#include <cstdlib>
typedef _Float16 h8_t __attribute__((ext_vector_type(8)));
typedef float f16v_t __attribute__((ext_vector_type(16)));
#define CK(x) do { hipError_t e_ = (x); if (e_ != hipSuccess) { printf("%s: %s\n", #x, hipGetErrorString(e_)); return 1; } } while (0)

// mode bit 0: MFMA waves compute; bit 1: writer waves store; bit 2: MFMA waves store; bit 3: writers at priority 3
template <int SLEEP>
__global__ __launch_bounds__(1024) void k(float *out, int iters, int mode, int spi, float *sink) {
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int nw = blockDim.x >> 6;
  if (wave < 8) {
    f16v_t acc[4];
    for (int q = 0; q < 4; q++) for (int v = 0; v < 16; v++) acc[q][v] = 0.f;
    h8_t a, b;
    for (int v = 0; v < 8; v++) { a[v] = (_Float16)(lane * 0.001f + v); b[v] = (_Float16)(lane * 0.002f - v); }
    float *wp = out + ((size_t)blockIdx.x * 8 + wave) * (size_t)iters * spi * 64 + lane;
    for (int it = 0; it < iters; it++) {
      if (mode & 1) {
#pragma unroll
        for (int r = 0; r < 6; r++)
#pragma unroll
          for (int q = 0; q < 4; q++) acc[q] = __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, acc[q], 0, 0, 0);
      }
      if (mode & 4) {
        for (int s = 0; s < spi; s++) __builtin_nontemporal_store(acc[0][s & 15], wp + ((size_t)it * spi + s) * 64);
      }
      if (SLEEP) __builtin_amdgcn_s_sleep(SLEEP);
      __builtin_amdgcn_s_barrier();
    }
    float x = 0;
    for (int q = 0; q < 4; q++) for (int v = 0; v < 16; v++) x += acc[q][v];
    if (x == 12345.678f) sink[0] = x;
  } else {
    if (mode & 8) __builtin_amdgcn_s_setprio(3);
    const int w = wave - 8, W = nw - 8;
    const int per_step = 8 * spi; // stores of the whole CU per step
    float *wp = out + (size_t)blockIdx.x * iters * per_step * 64 + lane;
    const float v = (float)lane;
    for (int it = 0; it < iters; it++) {
      if (mode & 2)
        for (int s = w; s < per_step; s += W) __builtin_nontemporal_store(v, wp + ((size_t)it * per_step + s) * 64);
      __builtin_amdgcn_s_barrier();
    }
  }
}

// the MFMA waves store themselves, one store after every 24 / SPI MFMAs
template <int SLEEP, int SPI>
__global__ __launch_bounds__(512) void kspread(float *out, int iters, float *sink) {
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  f16v_t acc[4];
  for (int q = 0; q < 4; q++) for (int v = 0; v < 16; v++) acc[q][v] = 0.f;
  h8_t a, b;
  for (int v = 0; v < 8; v++) { a[v] = (_Float16)(lane * 0.001f + v); b[v] = (_Float16)(lane * 0.002f - v); }
  float *wp = out + ((size_t)blockIdx.x * 8 + wave) * (size_t)iters * SPI * 64 + lane;
  for (int it = 0; it < iters; it++) {
#pragma unroll
    for (int idx = 0; idx < 24; idx++) {
      acc[idx & 3] = __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, acc[idx & 3], 0, 0, 0);
      if (idx % (24 / SPI) == (24 / SPI) - 1) {
        __builtin_amdgcn_sched_barrier(0);
        __builtin_nontemporal_store(acc[(idx + 2) & 3][idx & 15], wp + ((size_t)it * SPI + idx / (24 / SPI)) * 64);
        __builtin_amdgcn_sched_barrier(0);
      }
    }
    if (SLEEP) __builtin_amdgcn_s_sleep(SLEEP);
    __builtin_amdgcn_s_barrier();
  }
  float x = 0;
  for (int q = 0; q < 4; q++) for (int v = 0; v < 16; v++) x += acc[q][v];
  if (x == 12345.678f) sink[0] = x;
}

template <int SLEEP>
int run(int iters, int spi, float *out, float *sink) {
  hipEvent_t e0, e1; CK(hipEventCreate(&e0)); CK(hipEventCreate(&e1));
  struct { const char *name; int mode; int threads; } cases[] = {
      {"mfma only", 1, 512}, {"stores only, 4 writer waves", 2, 768}, {"stores only, by the 8 mfma-less waves", 4, 512},
      {"mfma + 4 writer waves", 3, 768}, {"mfma + 4 writer waves, prio 3", 11, 768}, {"mfma + 8 writer waves, prio 3", 11, 1024},
      {"mfma waves store themselves", 5, 512}, {"mfma waves, stores spread between the MFMAs", 21, 512}};
  printf("sleep %d x 64 clocks per step, %d stores per wave and step (%d B per CU and step)\n", SLEEP, spi, spi * 8 * 256);
  for (int rep = 0; rep < 2; rep++)
    for (auto &c : cases) {
      auto go = [&]() {
        if (c.mode == 21) {
          if (spi == 4) hipLaunchKernelGGL((kspread<SLEEP, 4>), dim3(256), dim3(512), 0, 0, out, iters, sink);
          else hipLaunchKernelGGL((kspread<SLEEP, 8>), dim3(256), dim3(512), 0, 0, out, iters, sink);
        } else {
          hipLaunchKernelGGL(k<SLEEP>, dim3(256), dim3(c.threads), 0, 0, out, iters, c.mode, spi, sink);
        }
      };
      for (int w = 0; w < 2; w++) go();
      CK(hipEventRecord(e0));
      for (int w = 0; w < 3; w++) go();
      CK(hipEventRecord(e1)); CK(hipEventSynchronize(e1));
      float ms; CK(hipEventElapsedTime(&ms, e0, e1)); ms /= 3;
      const double flops = 256.0 * 8 * iters * 24 * 32768.0, bytes = 256.0 * 8 * iters * spi * 256.0;
      if (rep == 1)
        printf("  %-40s %8.1f us  mfma %7.1f TFLOP/s  stores %6.2f TB/s\n", c.name, ms * 1e3,
               (c.mode & 1) ? flops / ms / 1e9 : 0.0, (c.mode & 6) ? bytes / ms / 1e9 : 0.0);
      fflush(stdout);
    }
  return 0;
}

int main(int argc, char **argv) {
  const int iters = argc > 1 ? atoi(argv[1]) : 2000;
  const int spi = argc > 2 ? atoi(argv[2]) : 4;
  const size_t floats = (size_t)256 * 8 * iters * spi * 64 + 1024;
  float *out, *sink;
  CK(hipMalloc(&out, floats * 4)); CK(hipMalloc(&sink, 64));
  if (run<8>(iters, spi, out, sink)) return 1;
  if (run<16>(iters, spi, out, sink)) return 1;
  if (run<24>(iters, spi, out, sink)) return 1;
  CK(hipDeviceSynchronize());
  printf("status ok\n");
  return 0;
}
