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

  // Id of the XCD (accelerator die) this wave runs on, 0..7.
  static __device__ __forceinline__ uint32_t xcdId() {
    uint32_t x;
    asm volatile("s_getreg_b32 %0, hwreg(HW_REG_XCC_ID)" : "=s"(x));
    return x & 7u;
  }

  // Draws the next ticket for this workgroup (first thread only).  `round` is
  // how many tickets this workgroup has already drawn, `dry` a bit mask the
  // caller keeps across rounds (start it at 0).  Returns numTiles() or more
  // when the tiles have run out.
  //
  // Each of the eight XCDs has its own L2, so which workgroup gets which tile
  // decides how much of the operands is re-fetched from memory.  The tiles are
  // therefore dealt per XCD: XCD x owns the column tiles [x*gx/8, (x+1)*gx/8) of
  // every row, in row-major order, and a workgroup draws from the dispenser of
  // the XCD it runs on.  The workgroups of one XCD thus share the same few B
  // column panels (and, row by row, the same A panels) in their L2.  A
  // workgroup whose own dispenser is empty helps the next XCD, so the end of the
  // launch stays balanced.  The ticket returned is the tile's position in the
  // row-major schedule; it still goes through the stage's ticket -> tile table.
  __device__ __forceinline__ uint32_t drawTicket(uint32_t launched, uint32_t round, uint32_t& dry) const {
    if (!customOrder()) {
      const uint32_t wg = blockIdx.x + gridDim.x * (blockIdx.y + gridDim.y * blockIdx.z);
      return wg + round * launched;
    }
    constexpr uint32_t kLine = 32;          // counters are 128 bytes apart
    const uint32_t mine = xcdId();
    for (uint32_t s = 0; s < 8; s++) {
      const uint32_t x = (mine + s) & 7u;
      if (dry & (1u << x)) continue;
      const uint32_t lo = x * d.grid.x / 8, cols = (x + 1) * d.grid.x / 8 - lo;
      const uint32_t count = cols * d.grid.y * d.grid.z;
      if (count != 0) {
        const uint32_t l = dev::ticketAdd(&d.xcdTickets[x * kLine], 1);
        if (l < count) return lo + l % cols + (l / cols) * d.grid.x;
      }
      dry |= 1u << x;
    }
    // Nothing left anywhere.  The last workgroup to find that out re-arms the
    // dispensers for the next run.
    const uint32_t finished = dev::ticketAdd(&d.xcdTickets[8 * kLine], 1);
    if (finished == launched - 1) {
      for (uint32_t x = 0; x < 9; x++) dev::storeRelaxed(&d.xcdTickets[x * kLine], 0);
    }
    return 0xffffffffu;
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

  // Starts a read of the semaphore guarding `tile` without waiting for it and
  // without ordering; dev::pollFinish() on the result, after other work, gives
  // the value to compare with waitTarget().
  __device__ __forceinline__ uint32_t peekBegin(const cusync_dim3& tile) const {
    return dev::pollBegin(&d.tileStatusRead[dyn::tileIndex(d.in, tile, d.prodGrid)]);
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
