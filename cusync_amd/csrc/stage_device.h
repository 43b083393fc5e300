// Device-side stage for the prebuilt kernels.
//
// DynStage wraps a cusync_stage_desc and offers the same three hooks a kernel
// uses on a cusync::CuStage — next tile, wait, post — with the policy evaluated
// at run time.  It adds what a persistent kernel needs: a launch may hold fewer
// workgroups than the stage has tiles, each workgroup then draws tickets until
// the tiles run out.
//
// Forward progress.  A consumer workgroup spins while it holds a slot on a CU.
// The wait-kernel flag is therefore raised only when EVERY workgroup of the
// producer launch has started: from then on no producer workgroup can be kept
// off the device, and since a producer of the first stage never waits, every
// semaphore a consumer spins on is eventually posted.  The launcher keeps a
// producer launch within what the device holds at once, so the flag goes up as
// soon as the launch has been dispatched.
#pragma once

#include <hip/hip_runtime.h>
#include "../../include/cusync/device-functions.h"
#include "policy_eval.h"

namespace cusync {

struct DynStage {
  cusync_stage_desc d;
  // True when every producer tile starts and ends on a 128-byte line of the
  // buffer the consumer reads (set by the launcher).  Then a line of that buffer
  // can only enter this XCD's caches after the semaphore guarding it was seen,
  // because the kernel began with clean caches and never touches a tile before
  // its wait; the wait can skip the cache invalidation that would also throw
  // away the weights the XCD's workgroups share.
  bool lineAligned;

  __device__ __forceinline__ bool isProducer() const { return d.out.kind != CUSYNC_POLICY_NOSYNC; }
  __device__ __forceinline__ bool isConsumer() const { return d.in.kind != CUSYNC_POLICY_NOSYNC; }
  __device__ __forceinline__ uint32_t numTiles() const { return d.grid.x * d.grid.y * d.grid.z; }
  __device__ __forceinline__ bool customOrder() const { return !(d.opts & CUSYNC_OPT_AVOID_CUSTOM_ORDER); }

  // Called once per workgroup by its first thread, before the first tile.
  // `launched` = number of workgroups in this launch.
  __device__ __forceinline__ void announceStart(uint32_t launched) const {
    if (!isProducer() || (d.opts & CUSYNC_OPT_AVOID_WAIT_KERNEL)) return;
    const uint32_t arrived = dev::ticketAdd(d.startCounter, 1);
    if (arrived == launched - 1) {
      dev::storeRelaxed(d.startCounter, 0);
      dev::releaseStore(d.kernelExecuted, (uint32_t)d.iter);
    }
  }

  // Draws the next ticket for this workgroup (first thread only).  `round` is
  // how many tickets this workgroup has already drawn.  Returns numTiles() or
  // more when the tiles have run out.
  __device__ __forceinline__ uint32_t drawTicket(uint32_t launched, uint32_t round) const {
    if (!customOrder()) {
      const uint32_t wg = blockIdx.x + gridDim.x * (blockIdx.y + gridDim.y * blockIdx.z);
      return wg + round * launched;
    }
    const uint32_t t = dev::ticketAdd(d.tileCounter, 1);
    // Every workgroup draws exactly one ticket past the end; the last of those
    // re-arms the dispenser for the next run.
    if (t == numTiles() + launched - 1) dev::storeRelaxed(d.tileCounter, 0);
    return t;
  }

  __device__ __forceinline__ cusync_dim3 ticketToTile(uint32_t ticket) const {
    if (customOrder()) return d.tileOrder[ticket];
    cusync_dim3 t;
    t.x = ticket % d.grid.x;
    t.y = (ticket / d.grid.x) % d.grid.y;
    t.z = ticket / (d.grid.x * d.grid.y);
    return t;
  }

  __device__ __forceinline__ bool needsWait(const cusync_dim3& tile) const {
    return isConsumer() && dyn::isSync(d.in, tile);
  }

  // Per-run count a semaphore of the input policy must reach.
  __device__ __forceinline__ uint32_t waitTarget() const { return (uint32_t)d.iter * dyn::waitValue(d.in); }

  // Current value of the semaphore guarding `tile`, without waiting and without
  // ordering: the caller compares it with waitTarget() later, after other work.
  __device__ __forceinline__ uint32_t peek(const cusync_dim3& tile) const {
    return dev::pollOnce(&d.tileStatusRead[dyn::tileIndex(d.in, tile, d.prodGrid)]);
  }

  // Wave-uniform wait: every lane of the calling wave passes the same tile.
  // No barrier; each wave that is going to read the tile calls this itself.
  __device__ __forceinline__ void waitWave(const cusync_dim3& tile) const {
    if (!needsWait(tile)) return;
    const uint32_t idx = dyn::tileIndex(d.in, tile, d.prodGrid);
    const bool ok = lineAligned ? dev::spinUntilAtLeastNoInvalidate(&d.tileStatusRead[idx], waitTarget())
                                : dev::spinUntilAtLeast(&d.tileStatusRead[idx], waitTarget());
    if (!ok && __builtin_amdgcn_mbcnt_hi(~0u, __builtin_amdgcn_mbcnt_lo(~0u, 0u)) == 0)
      dev::ticketAdd(d.spinTimeouts, 1);
  }

  // Workgroup-wide post; contains a barrier, call from all threads.
  __device__ __forceinline__ void post(const cusync_dim3& tile) const {
    if (!isProducer()) return;
    __syncthreads();
    if (threadIdx.x == 0 && threadIdx.y == 0 && threadIdx.z == 0) {
      const uint32_t idx = dyn::tileIndex(d.out, tile, d.grid);
      const uint32_t v = dyn::postValue(d.out);
      if (d.opts & CUSYNC_OPT_NO_ATOMIC_ADD) dev::releaseStore(&d.tileStatusWrite[idx], v * (uint32_t)d.iter);
      else dev::releaseAdd(&d.tileStatusWrite[idx], v);
    }
  }
};

}  // namespace cusync
