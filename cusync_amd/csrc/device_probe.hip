// What the matrix pipes of this device sustain on their own.
//
// The published dense fp16 rate (2.5 PFLOP/s) is the MFMA issue rate at the top clock.  Under a
// device-wide MFMA load the clock does not stay there: the power management lowers it, and by how
// much depends on how many bits toggle.  This kernel keeps every SIMD of the device busy with chains
// of v_mfma_f32_32x32x16_f16 on operands that never leave the registers (no LDS, no memory) and
// reports the rate and the clock it ran at (shader cycle counter over the 100 MHz constant counter),
// with all-zero operands or with random ones.  It is the ceiling for any fp16 GEMM on the machine it
// runs on; the GEMM kernels' roofline fractions are to be read against it.
#include <hip/hip_runtime.h>

#include <stdint.h>
#include <vector>

#include "../../include/cusync_amd.h"
#include "rt_internal.h"

namespace {

typedef _Float16 half8 __attribute__((ext_vector_type(8)));
typedef float floatx16 __attribute__((ext_vector_type(16)));

constexpr int kChains = 8;            // independent accumulators per wavefront: a 64x128 wavefront tile
constexpr int kMfmaPerIter = 2 * kChains;

__global__ __launch_bounds__(256, 2) void mfmaBurnKernel(uint32_t iters, uint32_t randomData, float* sink, unsigned long long* ticks) {
  uint32_t seed = (blockIdx.x * 256 + threadIdx.x) * 2654435761u + 12345u;
  half8 a[2], b[4];
  for (int i = 0; i < 6; i++)
    for (int e = 0; e < 8; e++) {
      seed = seed * 1664525u + 1013904223u;
      const _Float16 v = randomData ? (_Float16)((float)(((int)(seed >> 20) & 255) - 128) * (1.0f / 128.0f)) : (_Float16)0.0f;
      if (i < 2) a[i][e] = v; else b[i - 2][e] = v;
    }
  floatx16 acc[kChains];
  for (int i = 0; i < kChains; i++)
    for (int r = 0; r < 16; r++) acc[i][r] = 0.0f;
  const unsigned long long c0 = __builtin_readcyclecounter(), r0 = __builtin_amdgcn_s_memrealtime();
  for (uint32_t it = 0; it < iters; it++) {
#pragma unroll
    for (int kk = 0; kk < 2; kk++)
#pragma unroll
      for (int i = 0; i < 2; i++)
#pragma unroll
        for (int j = 0; j < 4; j++)
          acc[i * 4 + j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(b[j], a[i], acc[i * 4 + j], 0, 0, 0);
  }
  const unsigned long long c1 = __builtin_readcyclecounter(), r1 = __builtin_amdgcn_s_memrealtime();
  float s = 0.0f;
  for (int i = 0; i < kChains; i++)
    for (int r = 0; r < 16; r++) s += acc[i][r];
  if (s == 123.456f) sink[0] = s;                      // keeps the chains alive
  if (threadIdx.x == 0) { ticks[blockIdx.x * 2] = c1 - c0; ticks[blockIdx.x * 2 + 1] = r1 - r0; }
}

}  // namespace

extern "C" {

cusync_error cusync_probe_mfma_rate(int random_data, uint32_t iters, int launches, double* tflops, double* clock_mhz) {
  if (!tflops || !clock_mhz || iters == 0 || launches <= 0) return CUSYNC_ERROR_NOT_INITIALIZED;
  int dev = 0;
  hipDeviceProp_t prop;
  if (CUSYNC_HIP(hipGetDevice(&dev)) || CUSYNC_HIP(hipGetDeviceProperties(&prop, dev))) return CUSYNC_ERROR_DEVICE;
  const uint32_t grid = (uint32_t)prop.multiProcessorCount * 2;      // two wavefronts on every SIMD
  float* sink = nullptr;
  unsigned long long* ticks = nullptr;
  hipEvent_t e0 = nullptr, e1 = nullptr;
  cusync_error result = CUSYNC_SUCCESS;
  if (CUSYNC_HIP(hipMalloc((void**)&sink, 64)) || CUSYNC_HIP(hipMalloc((void**)&ticks, grid * 16)) ||
      CUSYNC_HIP(hipEventCreate(&e0)) || CUSYNC_HIP(hipEventCreate(&e1))) result = CUSYNC_ERROR_DEVICE;
  float ms = 0.0f;
  std::vector<unsigned long long> h(grid * 2);
  if (result == CUSYNC_SUCCESS) {
    // the clock needs a few milliseconds to settle under the load: as many untimed launches first
    for (int i = 0; i < launches; i++) hipLaunchKernelGGL(mfmaBurnKernel, dim3(grid), dim3(256), 0, 0, iters, (uint32_t)(random_data != 0), sink, ticks);
    if (CUSYNC_HIP(hipEventRecord(e0, 0))) result = CUSYNC_ERROR_DEVICE;
    for (int i = 0; i < launches; i++) hipLaunchKernelGGL(mfmaBurnKernel, dim3(grid), dim3(256), 0, 0, iters, (uint32_t)(random_data != 0), sink, ticks);
    if (CUSYNC_HIP(hipEventRecord(e1, 0)) || CUSYNC_HIP(hipEventSynchronize(e1)) || CUSYNC_HIP(hipEventElapsedTime(&ms, e0, e1)) ||
        CUSYNC_HIP(hipMemcpy(h.data(), ticks, grid * 16, hipMemcpyDeviceToHost))) result = CUSYNC_ERROR_DEVICE;
  }
  if (result == CUSYNC_SUCCESS) {
    double cycles = 0.0, real = 0.0;
    for (uint32_t b = 0; b < grid; b++) { cycles += (double)h[b * 2]; real += (double)h[b * 2 + 1]; }
    const double flop = (double)grid * 4.0 * iters * kMfmaPerIter * 32768.0 * launches;   // 32x32x16 MFMA = 32 768 FLOP
    *tflops = flop / ((double)ms * 1e-3) / 1e12;
    *clock_mhz = real > 0.0 ? cycles / real * 100.0 : 0.0;
  }
  if (e0) (void)hipEventDestroy(e0);
  if (e1) (void)hipEventDestroy(e1);
  (void)hipFree(sink); (void)hipFree(ticks);
  return result;
}

}  // extern "C"
