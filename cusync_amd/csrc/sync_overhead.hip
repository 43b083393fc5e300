// Cost of the synchronisation itself, measured two ways.
//
// 1. The reference's sync-overhead example (src/examples/sync-overhead/sync-overhead.cu:40-105): a
//    producer kernel that writes one value per thread and a consumer kernel that adds one to it, run
//    once with post/wait per block and once without, timed from the host.  Twice: with the example's own
//    kernels (a bare flag array, both kernels on one stream: cusync_sync_overhead_bare), and with the
//    public CuStage API (tile/wait/post) on two streams, which is what a chain really pays
//    (cusync_sync_overhead_pair).
// 2. What the example cannot show on a GPU of eight dies: the latency of one post -> wait hand-over
//    between two workgroups, as a ping-pong, for a partner on another XCD (neighbouring workgroup
//    index) and on the same XCD (index + 8; workgroups are dispatched to the XCDs round-robin).
#include <hip/hip_runtime.h>

#include <chrono>
#include <string>
#include <vector>
#include <stdint.h>

#include "../../include/cusync_amd.h"
#include "../../include/cusync/cusync.h"
#include "rt_internal.h"

namespace {

using namespace cusync;

using PairSync = TileSync<IdentityOrder, 1, 1>;
using PairProd = CuStage<IdentityOrder, NoSync, PairSync, NoOptimization>;
using PairCons = CuStage<IdentityOrder, PairSync, NoSync, NoOptimization>;

template<typename Stage>
__global__ void producerKernel(Stage stage, float* data, float value, bool sync) {
  __shared__ int tileSh[3];
  dim3 tile = sync ? stage.tile((dim3*)&tileSh[0]) : dim3(blockIdx.x, 0, 0);
  data[threadIdx.x + tile.x * blockDim.x] = value;
  if (sync) stage.post(tile);
}

template<typename Stage>
__global__ void consumerKernel(Stage stage, float* out, const float* in, bool sync) {
  __shared__ int tileSh[3];
  dim3 tile = sync ? stage.tile((dim3*)&tileSh[0]) : dim3(blockIdx.x, 0, 0);
  if (sync) stage.wait(tile);
  const uint32_t i = threadIdx.x + tile.x * blockDim.x;
  out[i] = in[i] + 1.0f;
}

// The example's own kernels (sync-overhead.cu:40-59): the producer's first thread bumps its block's flag behind a
// barrier, the consumer's first thread spins on flag 0 before the block goes on; no fence and no tile order, and
// the flags are adjacent words as there.  Both kernels run on one stream (:87-88), so every flag is up when the
// consumer starts: what is timed is the cost of touching the flags, not a hand-over.
__global__ void bareProducerKernel(float* data, float value, uint32_t* flags, bool sync) {
  data[threadIdx.x + blockIdx.x * blockDim.x] = value;
  __syncthreads();
  if (sync && threadIdx.x == 0) __hip_atomic_fetch_add(&flags[blockIdx.x], 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

__global__ void bareConsumerKernel(float* out, const float* in, uint32_t* flags, bool sync, uint32_t iter, uint32_t* failed) {
  if (sync && threadIdx.x == 0) {
    uint32_t polls = 0;
    while (__hip_atomic_load(&flags[0], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) < iter + 1)
      if (++polls >= CUSYNC_SPIN_LIMIT) { *failed = 1; break; }      // bounded like every wait of the library
  }
  __syncthreads();
  const uint32_t i = threadIdx.x + blockIdx.x * blockDim.x;
  out[i] = in[i] + 1.0f;
}

// Workgroup 0 posts flag A and waits for flag B; workgroup `partner` does the opposite.  Every wait is
// bounded; a give-up is reported through *failed.  Other workgroups leave at once.
__global__ void pingPongKernel(uint32_t* flags, uint32_t partner, uint32_t rounds, unsigned long long* ticks, uint32_t* failed) {
  if (threadIdx.x != 0) return;
  volatile uint32_t* a = flags;          // 128 bytes apart
  volatile uint32_t* b = flags + 32;
  if (blockIdx.x == 0) {
    const unsigned long long t0 = __builtin_amdgcn_s_memrealtime();
    for (uint32_t i = 1; i <= rounds; i++) {
      dev::releaseAdd(a, 1);
      if (!dev::spinUntilAtLeast(b, i)) { *failed = 1; break; }
    }
    *ticks = __builtin_amdgcn_s_memrealtime() - t0;
  } else if (blockIdx.x == partner) {
    for (uint32_t i = 1; i <= rounds; i++) {
      if (!dev::spinUntilAtLeast(a, i)) { *failed = 1; break; }
      dev::releaseAdd(b, 1);
    }
  }
}

double nowUs() {
  return std::chrono::duration<double, std::micro>(std::chrono::steady_clock::now().time_since_epoch()).count();
}

}  // namespace

extern "C" {

cusync_error cusync_sync_overhead_pair(uint32_t blocks, uint32_t threads, int warmup, int iters,
                                       double* with_sync_us, double* without_sync_us) {
  if (!blocks || !threads || threads > 1024 || iters < 1 || !with_sync_us || !without_sync_us) return CUSYNC_ERROR_NOT_INITIALIZED;
  const size_t n = (size_t)blocks * threads;
  float *in = nullptr, *out = nullptr;
  hipStream_t sp = nullptr, sc = nullptr;
  if (CUSYNC_HIP(hipMalloc((void**)&in, n * 4)) || CUSYNC_HIP(hipMalloc((void**)&out, n * 4)) ||
      CUSYNC_HIP(hipStreamCreateWithFlags(&sp, hipStreamNonBlocking)) ||
      CUSYNC_HIP(hipStreamCreateWithFlags(&sc, hipStreamNonBlocking))) return CUSYNC_ERROR_DEVICE;
  dim3 grid(blocks, 1, 1), block(threads, 1, 1);
  PairSync sync;
  PairProd prod(grid, block, NoSync(), sync);
  PairCons cons(grid, block, sync, NoSync());
  cusync_error result = CUSYNC_SUCCESS;
  if (CuSync::setProducerConsumerPair(prod, cons) != CuSyncSuccess) result = CUSYNC_ERROR_NOT_INITIALIZED;
  double total[2] = {0, 0};
  for (int mode = 0; mode < 2 && result == CUSYNC_SUCCESS; mode++) {     // 0: post/wait on two streams, 1: stream order
    for (int i = 0; i < warmup + iters; i++) {
      const double t0 = nowUs();
      if (mode == 0) {
        hipLaunchKernelGGL(producerKernel<PairProd>, grid, block, 0, sp, prod, in, (float)i, true);
        prod.invokeWaitKernel(sc);
        hipLaunchKernelGGL(consumerKernel<PairCons>, grid, block, 0, sc, cons, out, in, true);
      } else {
        hipLaunchKernelGGL(producerKernel<PairProd>, grid, block, 0, sp, prod, in, (float)i, false);
        hipLaunchKernelGGL(consumerKernel<PairCons>, grid, block, 0, sp, cons, out, in, false);
      }
      if (CUSYNC_HIP(hipDeviceSynchronize())) { result = CUSYNC_ERROR_DEVICE; break; }
      if (i >= warmup) total[mode] += nowUs() - t0;
      if (mode == 0) { prod.incrementIter(); cons.incrementIter(); }
    }
    // The pair's result (sync-overhead.cu checks nothing; tests/simple-test.cu checks a synced pair this way):
    // every element is what the producer of the LAST run wrote, plus one.  A consumer block that read before
    // its producer block had posted would have found the value of the run before.
    if (result == CUSYNC_SUCCESS) {
      std::vector<float> host(n);
      if (CUSYNC_HIP(hipMemcpy(host.data(), out, n * 4, hipMemcpyDeviceToHost))) { result = CUSYNC_ERROR_DEVICE; break; }
      const float want = (float)(warmup + iters - 1) + 1.0f;
      size_t bad = 0;
      for (size_t k = 0; k < n; k++) bad += host[k] != want;
      if (bad) {
        cusync::rt::setError(std::string("sync overhead pair: ") + std::to_string(bad) + " of " + std::to_string(n) +
                             " elements are not the producer's value plus one (" + (mode == 0 ? "post/wait on two streams" : "stream order") + ")");
        result = CUSYNC_ERROR_DEVICE;
      }
    }
  }
  if (result == CUSYNC_SUCCESS) {
    const cusync_stage_desc cd = cons.desc();
    uint32_t gaveUp = 0;
    if (cusync_stage_read_state(&cd, nullptr, nullptr, nullptr, nullptr, nullptr, &gaveUp) != CUSYNC_SUCCESS) result = CUSYNC_ERROR_DEVICE;
    else if (gaveUp) { cusync::rt::setError("sync overhead pair: a wait gave up"); result = CUSYNC_ERROR_DEVICE; }
  }
  *with_sync_us = total[0] / iters;
  *without_sync_us = total[1] / iters;
  prod.destroy(); cons.destroy();
  (void)hipStreamDestroy(sp); (void)hipStreamDestroy(sc);
  (void)hipFree(in); (void)hipFree(out);
  return result;
}

cusync_error cusync_sync_overhead_bare(uint32_t blocks, uint32_t threads, int warmup, int iters,
                                       double* with_flags_us, double* without_flags_us) {
  if (!blocks || !threads || threads > 1024 || iters < 1 || !with_flags_us || !without_flags_us) return CUSYNC_ERROR_NOT_INITIALIZED;
  const size_t n = (size_t)blocks * threads;
  float *in = nullptr, *out = nullptr;
  uint32_t* flags = nullptr;
  hipStream_t st = nullptr;
  if (CUSYNC_HIP(hipMalloc((void**)&in, n * 4)) || CUSYNC_HIP(hipMalloc((void**)&out, n * 4)) ||
      CUSYNC_HIP(hipMalloc((void**)&flags, ((size_t)blocks + 1) * 4)) || CUSYNC_HIP(hipMemset(flags, 0, ((size_t)blocks + 1) * 4)) ||
      CUSYNC_HIP(hipStreamCreateWithFlags(&st, hipStreamNonBlocking))) return CUSYNC_ERROR_DEVICE;
  uint32_t* failed = flags + blocks;
  dim3 grid(blocks, 1, 1), block(threads, 1, 1);
  cusync_error result = CUSYNC_SUCCESS;
  double total[2] = {0, 0};
  uint32_t run = 0;      // runs of the flagged leg so far: flag 0 stands at `run` when one begins
  for (int mode = 0; mode < 2 && result == CUSYNC_SUCCESS; mode++) {     // 0: with the flags, 1: without
    for (int i = 0; i < warmup + iters; i++) {
      const double t0 = nowUs();
      hipLaunchKernelGGL(bareProducerKernel, grid, block, 0, st, in, (float)i, flags, mode == 0);
      hipLaunchKernelGGL(bareConsumerKernel, grid, block, 0, st, out, in, flags, mode == 0, run, failed);
      if (CUSYNC_HIP(hipDeviceSynchronize())) { result = CUSYNC_ERROR_DEVICE; break; }
      if (i >= warmup) total[mode] += nowUs() - t0;
      if (mode == 0) run++;
    }
    if (result != CUSYNC_SUCCESS) break;
    std::vector<float> host(n);
    uint32_t gaveUp = 0;
    if (CUSYNC_HIP(hipMemcpy(host.data(), out, n * 4, hipMemcpyDeviceToHost)) ||
        CUSYNC_HIP(hipMemcpy(&gaveUp, failed, 4, hipMemcpyDeviceToHost))) { result = CUSYNC_ERROR_DEVICE; break; }
    const float want = (float)(warmup + iters - 1) + 1.0f;
    size_t bad = 0;
    for (size_t k = 0; k < n; k++) bad += host[k] != want;
    if (bad || gaveUp) {
      cusync::rt::setError(std::string("sync overhead, bare flags: ") + std::to_string(bad) + " of " + std::to_string(n) +
                           " elements are not the producer's value plus one" + (gaveUp ? "; a poll gave up" : ""));
      result = CUSYNC_ERROR_DEVICE;
    }
  }
  *with_flags_us = total[0] / iters;
  *without_flags_us = total[1] / iters;
  (void)hipStreamDestroy(st);
  (void)hipFree(in); (void)hipFree(out); (void)hipFree(flags);
  return result;
}

cusync_error cusync_sync_overhead_pingpong(uint32_t partner, uint32_t rounds, double* ns_per_round_trip) {
  if (partner == 0 || partner >= 64 || rounds == 0 || !ns_per_round_trip) return CUSYNC_ERROR_NOT_INITIALIZED;
  uint32_t* flags = nullptr;
  unsigned long long* ticks = nullptr;
  if (CUSYNC_HIP(hipMalloc((void**)&flags, 1024)) || CUSYNC_HIP(hipMemset(flags, 0, 1024)) ||
      CUSYNC_HIP(hipMalloc((void**)&ticks, 8))) return CUSYNC_ERROR_DEVICE;
  uint32_t* failed = flags + 64;
  // 64 workgroups of one wave always fit the device at once, so both partners are running
  hipLaunchKernelGGL(pingPongKernel, dim3(64), dim3(64), 0, 0, flags, partner, rounds, ticks, failed);
  unsigned long long t = 0;
  uint32_t bad = 0;
  cusync_error result = CUSYNC_SUCCESS;
  if (CUSYNC_HIP(hipDeviceSynchronize()) || CUSYNC_HIP(hipMemcpy(&t, ticks, 8, hipMemcpyDeviceToHost)) ||
      CUSYNC_HIP(hipMemcpy(&bad, failed, 4, hipMemcpyDeviceToHost))) result = CUSYNC_ERROR_DEVICE;
  if (bad) { cusync::rt::setError("ping-pong: a wait gave up"); result = CUSYNC_ERROR_DEVICE; }
  *ns_per_round_trip = (double)t * 10.0 / rounds;      // the constant-rate counter ticks at 100 MHz
  (void)hipFree(flags); (void)hipFree(ticks);
  return result;
}

}  // extern "C"
