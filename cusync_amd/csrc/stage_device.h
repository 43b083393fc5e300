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
  // allStatic(launched) of the launch this object goes to, worked out by the launcher (set by prepare()): in the
  // kernel it is a loop of eight rounds of integer divisions that every wavefront would run before its first load.
  bool noDraws;
  // Diagnosis (set by the launcher from CUSYNC_FORCE_RELEASE): every post, and every count the k-slices and key-range
  // splits hand partial results over with, is a release at device scope (and the counts' readers acquire), as the
  // plain protocol has it, also where the stores were written through and acknowledged and the library normally
  // raises them relaxed.  Results must not change; only the write-backs and invalidations come back.
  bool releaseAll;

  __device__ __forceinline__ bool isProducer() const { return d.out.kind != CUSYNC_POLICY_NOSYNC; }
  // Whether this stage's kernels write their output through to memory as they store it (sc1): a producer's do, so
  // that the post finds nothing to write back.  The epilogues take their store policy from here and hand the same
  // answer to post(): one flag decides both.
  __device__ __forceinline__ bool storesThrough() const { return isProducer(); }
  // A count that hands over data written through and acknowledged (k-slices, key-range splits): relaxed, or a
  // release under releaseAll.
  __device__ __forceinline__ uint32_t countIn(uint32_t* counter) const {
    return releaseAll ? __hip_atomic_fetch_add(counter, 1u, __ATOMIC_RELEASE, __HIP_MEMORY_SCOPE_AGENT)
                      : __hip_atomic_fetch_add(counter, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  }
  // ... and what its reader does before it touches the data (nothing: it reads with device-coherent loads).
  __device__ __forceinline__ void countSeen() const { if (releaseAll) dev::acquireFence(); }
  __device__ __forceinline__ bool isConsumer() const { return d.in.kind != CUSYNC_POLICY_NOSYNC; }
  __device__ __forceinline__ uint32_t numTiles() const { return d.grid.x * d.grid.y * d.grid.z; }
  __host__ __device__ __forceinline__ bool customOrder() const { return !(d.opts & CUSYNC_OPT_AVOID_CUSTOM_ORDER); }

  // ---- tickets -------------------------------------------------------------
  // A launch may hold fewer workgroups than the stage has tiles; each workgroup
  // then takes tickets until the tiles run out.  All of the following are
  // called by the first thread of a workgroup only.
  //
  // Each of the eight XCDs has its own L2, so which workgroup gets which tile
  // decides how much of the operands is re-fetched from memory.  The tiles are
  // therefore dealt per XCD.  With at least eight column tiles XCD x owns the
  // column tiles [x*gx/8, (x+1)*gx/8) of every row, in row-major order: its
  // workgroups share the same few B column panels (and, row by row, the same
  // A panels) in their L2.  With fewer column tiles (a convolution with 64
  // output channels has one) XCD x owns the row tiles [x*gy/8, (x+1)*gy/8)
  // instead, so that the rows of A it reads — for a convolution each input
  // pixel is read by up to R*S neighbouring rows — stay in its L2.  The
  // ticket is the tile's position in the row-major schedule; it still goes
  // through the stage's ticket -> tile table.
  //
  // A device-wide atomic takes the better part of a microsecond, several when
  // hundreds of workgroups hit one address at kernel start, and a kernel of a
  // few tens of microseconds cannot afford a chain of them:
  //  * Workgroups are dispatched to the XCDs round-robin: the workgroups
  //    with the same index modulo 8 share an XCD (which one varies from launch
  //    to launch, so the hardware XCD id is of no use here).  Workgroup b
  //    therefore works on list b%8.  Where it really runs only matters for
  //    locality: every position is taken exactly once either way.
  //  * The first tile of a workgroup needs no atomic: it is position b/8 of
  //    its list.
  //  * Later tiles come from a dispenser per list that starts behind those
  //    static positions.  The draw is split in two so that a kernel can issue
  //    it before the epilogue of a tile and pick the result up afterwards.
  //    (Not earlier: a workgroup that reserved its next tile at the start of
  //    the current one would take work from workgroups that have none.)
  //  * A workgroup whose own list is used up looks at all dispensers at once
  //    (plain loads, one round trip): a counter seen at or above its list's
  //    length is dry for good, the others are tried in turn, so the end of the
  //    launch stays balanced.  The last workgroup to find everything dry
  //    re-arms the dispensers for the next run.
  __host__ __device__ __forceinline__ bool dealtByRows() const { return d.grid.x < 8; }
  __host__ __device__ __forceinline__ uint32_t xcdTiles(uint32_t x) const {
    const uint32_t span = dealtByRows() ? d.grid.y : d.grid.x;
    return ((x + 1) * span / 8 - x * span / 8) * (dealtByRows() ? d.grid.x : d.grid.y) * d.grid.z;
  }
  // Positions of XCD x's list that are handed out statically to the first tiles of the workgroups.
  __host__ __device__ __forceinline__ uint32_t xcdStatic(uint32_t x, uint32_t launched) const {
    const uint32_t wgs = launched > x ? (launched - x + 7) / 8 : 0;
    const uint32_t tiles = xcdTiles(x);
    return wgs < tiles ? wgs : tiles;
  }
  __device__ __forceinline__ uint32_t xcdTicket(uint32_t x, uint32_t l) const {
    const uint32_t span = dealtByRows() ? d.grid.y : d.grid.x;
    const uint32_t lo = x * span / 8, width = (x + 1) * span / 8 - lo;
    if (!dealtByRows()) return lo + l % width + (l / width) * d.grid.x;
    const uint32_t perSlice = width * d.grid.x;          // this XCD's tiles in one k-slice
    return (l / perSlice) * d.grid.x * d.grid.y + lo * d.grid.x + l % perSlice;
  }
  // True when the static first tiles already are all tiles (a launch of one round whose workgroups spread
  // evenly over the lists): nobody then needs a dispenser, a look at the others or the count of workgroups
  // that ran dry, and a workgroup leaves after its tile without a single atomic.
  __host__ __device__ __forceinline__ bool allStatic(uint32_t launched) const {
    if (!customOrder()) return false;
    bool all = true;
    for (uint32_t x = 0; x < 8; x++) all = all && xcdStatic(x, launched) == xcdTiles(x);
    return all;
  }
  // Host side, once the descriptor and lineAligned are in place: what the kernel would otherwise work out per wavefront.
  __host__ void prepare(uint32_t launched) { noDraws = allStatic(launched); }
  static __device__ __forceinline__ uint32_t workgroupIndex() {
    return blockIdx.x + gridDim.x * (blockIdx.y + gridDim.y * blockIdx.z);
  }
  static __device__ __forceinline__ uint32_t homeList() { return workgroupIndex() & 7u; }

  // Counts this workgroup as started; give the result to finishStart() later
  // (after other work has been issued, so that the round trip is hidden).
  __device__ __forceinline__ uint32_t beginStart() const {
    if (!isProducer() || (d.opts & CUSYNC_OPT_AVOID_WAIT_KERNEL)) return 0;
    return dev::ticketAdd(d.startCounter, 1);
  }
  // The workgroup that started last raises the wait-kernel flag.
  __device__ __forceinline__ void finishStart(uint32_t token, uint32_t launched) const {
    if (!isProducer() || (d.opts & CUSYNC_OPT_AVOID_WAIT_KERNEL)) return;
    if (token == launched - 1) {
      dev::storeRelaxed(d.startCounter, 0);
      // The flag says that every producer workgroup is on the device and publishes no data (a consumer reads the
      // producer's output behind the tiles' semaphores): relaxed stores.  As releases they wrote this XCD's L2 back,
      // the second one as far as the host, on the critical path of the one workgroup that raises them.
      dev::storeRelaxed(d.kernelExecuted, (uint32_t)d.iter);
      __hip_atomic_store(d.spinTimeouts + CUSYNC_HOST_FLAG_OFFSET, (uint32_t)d.iter, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);     // mirror for a host that holds the consumer back itself
    }
  }

  // Issues the draw of the next ticket; `dry` is the mask drawFinish() keeps.
  __device__ __forceinline__ uint32_t drawBegin(uint32_t dry, bool noDraws = false) const {
    if (!customOrder() || noDraws) return 0;
    const uint32_t mine = homeList();
    if (dry & (1u << mine)) return 0xffffffffu;
    return dev::ticketAdd(&d.xcdTickets[mine * 32], 1);
  }
  // Turns the result of drawBegin() into a ticket; numTiles() or more when the
  // tiles have run out.  `round` = tickets this workgroup has drawn before.
  __device__ __forceinline__ uint32_t drawFinish(uint32_t raw, uint32_t launched, uint32_t round, uint32_t& dry,
                                                 bool noDraws = false) const {
    if (!customOrder()) return workgroupIndex() + round * launched;
    if (noDraws) return 0xffffffffu;
    constexpr uint32_t kLine = 32;          // counters are 128 bytes apart
    const uint32_t mine = homeList();
    if (raw != 0xffffffffu) {
      const uint32_t l = raw + xcdStatic(mine, launched);
      if (l < xcdTiles(mine)) return xcdTicket(mine, l);
    }
    dry |= 1u << mine;
    uint32_t seen[8];
#pragma unroll
    for (uint32_t x = 0; x < 8; x++) seen[x] = dev::loadRelaxed(&d.xcdTickets[x * kLine]);
#pragma unroll
    for (uint32_t x = 0; x < 8; x++)
      if (seen[x] + xcdStatic(x, launched) >= xcdTiles(x)) dry |= 1u << x;
    for (uint32_t s = 1; s < 8; s++) {
      const uint32_t x = (mine + s) & 7u;
      if (dry & (1u << x)) continue;
      const uint32_t l = dev::ticketAdd(&d.xcdTickets[x * kLine], 1) + xcdStatic(x, launched);
      if (l < xcdTiles(x)) return xcdTicket(x, l);
      dry |= 1u << x;
    }
    const uint32_t finished = dev::ticketAdd(&d.xcdTickets[8 * kLine], 1);
    if (finished == launched - 1) {
      for (uint32_t x = 0; x < 9; x++) dev::storeRelaxed(&d.xcdTickets[x * kLine], 0);
    }
    return 0xffffffffu;
  }
  // First ticket of a workgroup: its static position if its XCD's list is long enough.
  __device__ __forceinline__ uint32_t firstTicket(uint32_t launched, uint32_t& dry, bool noDraws = false) const {
    if (!customOrder()) return workgroupIndex();
    const uint32_t b = workgroupIndex(), x = b & 7u, pos = b >> 3;
    if (pos < xcdTiles(x)) return xcdTicket(x, pos);
    return drawFinish(drawBegin(dry, noDraws), launched, 0, dry, noDraws);
  }

  __device__ __forceinline__ cusync_dim3 ticketToTile(uint32_t ticket) const {
    if (customOrder() && !(d.flags & CUSYNC_STAGE_IDENTITY_ORDER)) return d.tileOrder[ticket];
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
    return dev::pollBegin(&d.tileStatusRead[dyn::tileIndex(d.in, tile, d.prodGrid) * CUSYNC_SEM_STRIDE]);
  }

  // Wave-uniform wait: every lane of the calling wave passes the same tile.
  // No barrier; each wave that is going to read the tile calls this itself.
  __device__ __forceinline__ void waitWave(const cusync_dim3& tile) const {
    if (!needsWait(tile)) return;
    const uint32_t idx = dyn::tileIndex(d.in, tile, d.prodGrid) * CUSYNC_SEM_STRIDE;
    const bool ok = lineAligned ? dev::spinUntilAtLeastNoInvalidate(&d.tileStatusRead[idx], waitTarget())
                                : dev::spinUntilAtLeast(&d.tileStatusRead[idx], waitTarget());
    if (!ok && __builtin_amdgcn_mbcnt_hi(~0u, __builtin_amdgcn_mbcnt_lo(~0u, 0u)) == 0)
      dev::countGiveUp(d.spinTimeouts);
  }

  // Wave-uniform wait for every tile {r, col, z} whose rows meet rowLo..rowHi (row blocks of tileM rows):
  // one lane per row block, so that all their semaphores are read in the same round trips instead of one
  // after the other.  A lane stops polling once its tile is posted.
  __device__ __forceinline__ void waitWaveRows(uint32_t rowLo, uint32_t rowHi, uint32_t tileM, uint32_t col, uint32_t z) const {
    if (!isConsumer()) return;
    const uint32_t lane = __builtin_amdgcn_mbcnt_hi(~0u, __builtin_amdgcn_mbcnt_lo(~0u, 0u));
    const uint32_t b0 = rowLo / tileM, blocks = rowHi / tileM - b0 + 1;
    const uint32_t target = waitTarget();
    bool timedOut = false;
    for (uint32_t base = 0; base < blocks; base += 64) {
      const uint32_t i = base + lane;
      const cusync_dim3 mine = {(b0 + (i < blocks ? i : 0u)) * tileM, col, z};
      bool pending = i < blocks && needsWait(mine);
      const uint32_t* sem = &d.tileStatusRead[dyn::tileIndex(d.in, mine, d.prodGrid) * CUSYNC_SEM_STRIDE];
      uint32_t polls = 0, naps = 1;
      for (;;) {
        if (pending && dev::loadRelaxed(sem) >= target) pending = false;
        if (__ballot(pending) == 0) break;
        if (++polls >= CUSYNC_SPIN_LIMIT) { timedOut = true; break; }
        for (uint32_t n = 0; n < naps; n++) __builtin_amdgcn_s_sleep(16);
        if (naps < CUSYNC_MAX_NAPS) naps <<= 1;
      }
    }
    if (lineAligned) __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    else dev::acquireFence();
    if (timedOut && lane == 0) dev::countGiveUp(d.spinTimeouts);
  }

  // Wave-uniform look, without spinning, at the tiles {r, col, z} of the row blocks that meet rowLo..rowHi (at most
  // 64 of them, one per lane, one round trip): how many of them, counted from the first, are posted.
  __device__ __forceinline__ uint32_t peekWaveRows(uint32_t rowLo, uint32_t rowHi, uint32_t tileM, uint32_t col, uint32_t z) const {
    if (!isConsumer()) return 64;
    const uint32_t lane = __builtin_amdgcn_mbcnt_hi(~0u, __builtin_amdgcn_mbcnt_lo(~0u, 0u));
    const uint32_t b0 = rowLo / tileM;
    uint32_t blocks = rowHi / tileM - b0 + 1;
    if (blocks > 64) blocks = 64;
    const cusync_dim3 mine = {(b0 + (lane < blocks ? lane : 0u)) * tileM, col, z};
    const bool polls = lane < blocks && needsWait(mine);
    uint32_t v = 0xffffffffu;
    if (polls) v = dev::loadRelaxed(&d.tileStatusRead[dyn::tileIndex(d.in, mine, d.prodGrid) * CUSYNC_SEM_STRIDE]);
    const uint64_t pending = __ballot(lane < blocks && v < waitTarget());
    const uint32_t ready = pending ? (uint32_t)__builtin_ctzll(pending) : blocks;
    if (ready) {
      if (lineAligned) __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
      else dev::acquireFence();
    }
    return ready;
  }

  // Wave-uniform wait for tile {row, col, 0} that looks ahead: the first poll reads, one per lane, the
  // semaphores of up to `count` (at most 64) tiles {row, col + i * colStep, 0} in one round trip and
  // returns how many of them, counted from the first, are posted.  If the first is not, the wave spins on
  // that one alone (all lanes polling for as long as the producer needs would be that many times the
  // traffic on the semaphores) and returns 1.  A consumer that is several tiles behind its producer
  // then polls once per sixty-four tiles instead of once per tile; every poll is a round trip to memory
  // that the loads already in flight have to drain behind.
  __device__ __forceinline__ uint32_t waitWaveAhead(uint32_t row, uint32_t col, uint32_t colStep, uint32_t count) const {
    const uint32_t lane = __builtin_amdgcn_mbcnt_hi(~0u, __builtin_amdgcn_mbcnt_lo(~0u, 0u));
    const uint32_t n = count < 64u ? count : 64u;
    const cusync_dim3 mine = {row, col + (lane < n ? lane : 0u) * colStep, 0};
    const bool polls = lane < n && needsWait(mine);
    const uint32_t target = waitTarget();
    uint32_t v = 0xffffffffu;
    if (polls) v = dev::loadRelaxed(&d.tileStatusRead[dyn::tileIndex(d.in, mine, d.prodGrid) * CUSYNC_SEM_STRIDE]);
    const uint64_t pending = __ballot(v < target);
    uint32_t ready = pending ? (uint32_t)__builtin_ctzll(pending) : n;
    if (ready > n) ready = n;
    if (ready == 0) {
      const cusync_dim3 first = {row, col, 0};
      waitWave(first);           // spins, fences, counts a time-out
      return 1;
    }
    if (lineAligned) __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    else dev::acquireFence();
    return ready;
  }

  // The same look-ahead for a consumer tile that meets several row blocks of its producer (rowLo..rowHi, blocks of
  // tileM rows): one lane per (row block, column tile), as many column tiles as fit into the wave, in one round
  // trip.  Returns how many column tiles, counted from the first, have all their row blocks posted; if the first
  // has not, the wave waits for that one (all its row blocks) and returns 1.
  __device__ __forceinline__ uint32_t waitWaveAheadRows(uint32_t rowLo, uint32_t rowHi, uint32_t tileM, uint32_t col,
                                                        uint32_t colStep, uint32_t count) const {
    const uint32_t lane = __builtin_amdgcn_mbcnt_hi(~0u, __builtin_amdgcn_mbcnt_lo(~0u, 0u));
    const uint32_t b0 = rowLo / tileM, blocks = rowHi / tileM - b0 + 1;
    if (blocks > 32) { waitWaveRows(rowLo, rowHi, tileM, col, 0); return 1; }
    uint32_t n = 64 / blocks;
    if (n > count) n = count;
    const uint32_t myCol = lane / blocks, myBlock = lane % blocks;
    const bool inRange = myCol < n;
    const cusync_dim3 mine = {(b0 + (inRange ? myBlock : 0u)) * tileM, col + (inRange ? myCol : 0u) * colStep, 0};
    const bool polls = inRange && needsWait(mine);
    const uint32_t target = waitTarget();
    uint32_t v = 0xffffffffu;
    if (polls) v = dev::loadRelaxed(&d.tileStatusRead[dyn::tileIndex(d.in, mine, d.prodGrid) * CUSYNC_SEM_STRIDE]);
    const uint64_t pending = __ballot(inRange && v < target);
    uint32_t ready = pending ? (uint32_t)__builtin_ctzll(pending) / blocks : n;      // lanes are ordered by column tile
    if (ready > n) ready = n;
    if (ready == 0) {
      waitWaveRows(rowLo, rowHi, tileM, col, 0);          // spins, fences, counts a time-out
      return 1;
    }
    if (lineAligned) __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    else dev::acquireFence();
    return ready;
  }

  // Workgroup-wide post; contains a barrier, call from all threads.  `times`: how many posts of the policy this
  // one stands for (a workgroup that finished several logical tiles guarded by one semaphore adds them at once).
  // `writtenThrough`: every store of the tile went through to memory as it was made (sc1), so once the wavefronts
  // have seen their stores acknowledged there is nothing left for a release to write back, and the semaphore is
  // raised without one (a release at device scope starts a write-back of this XCD's L2 whatever it holds).
  __device__ __forceinline__ void post(const cusync_dim3& tile, uint32_t times = 1, bool writtenThrough = false) const {
    if (!isProducer()) return;
    // The release is the first thread's and waits for its own wavefront's stores; a workgroup barrier does not wait
    // for stores to memory.  Every wavefront sees its own stores of the tile through before it reaches the barrier.
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();
    if (threadIdx.x == 0 && threadIdx.y == 0 && threadIdx.z == 0) {
      const uint32_t idx = dyn::tileIndex(d.out, tile, d.grid) * CUSYNC_SEM_STRIDE;
      const uint32_t v = dyn::postValue(d.out) * times;
      if (writtenThrough && !releaseAll) {
        if (d.opts & CUSYNC_OPT_NO_ATOMIC_ADD) dev::storeRelaxed(&d.tileStatusWrite[idx], v * (uint32_t)d.iter);
        else __hip_atomic_fetch_add((uint32_t*)&d.tileStatusWrite[idx], v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      } else {
        if (d.opts & CUSYNC_OPT_NO_ATOMIC_ADD) dev::releaseStore(&d.tileStatusWrite[idx], v * (uint32_t)d.iter);
        else dev::releaseAdd(&d.tileStatusWrite[idx], v);
      }
    }
  }
};

}  // namespace cusync
