// Global-memory semaphore primitives for gfx950.
//
// An MI355X has eight XCDs, each with a private L2, so a value written by a
// workgroup on one XCD is only guaranteed visible to a workgroup on another
// after an agent-scope release on the writer side and an agent-scope acquire on
// the reader side.  These helpers are the only places in the library that touch
// a semaphore.  They replace the PTX of the reference
// (src/include/cusync/device-functions.h:14-32: ld.acquire.gpu / ld.global.cg,
// and st.release.gpu / atomicAdd after __threadfence_system in
// src/include/cusync/cusync_device_defs.h:57-67).
#pragma once

#include "cusync_defines.h"
#include <stdint.h>

#if CUSYNC_HAS_DEVICE
namespace cusync {
namespace dev {

// Coherent (agent-scope) load that is not an acquire: cheap enough to spin on.
CUSYNC_DEVICE uint32_t loadRelaxed(const volatile uint32_t* addr) {
  return __hip_atomic_load((const uint32_t*)addr, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

// Same role as globalVolatileLoad of the reference: acquire at agent scope.
CUSYNC_DEVICE uint32_t loadAcquire(const volatile uint32_t* addr) {
  return __hip_atomic_load((const uint32_t*)addr, __ATOMIC_ACQUIRE, __HIP_MEMORY_SCOPE_AGENT);
}

// Orders every later load of the calling wave after the loads before it and
// drops stale lines of this XCD's caches.
CUSYNC_DEVICE void acquireFence() { __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "agent"); }

// Upper bound on polls of one wait.  A wait that is never satisfied (a lost
// post, a stage wired to the wrong producer) must not hold the GPU forever:
// after this many polls the wait gives up and reports failure.  One poll is a
// trip to the coherent level of the memory system plus a sleep that grows to
// about one microsecond, so the default allows a second or two.
#ifndef CUSYNC_SPIN_LIMIT
#define CUSYNC_SPIN_LIMIT (1u << 20)
#endif
// Longest sleep between two polls, in units of 1024 clocks (about 0.43 us).  Eight (3.5 us) cost the
// chains 2-3 us per handover against two; one brought nothing more.
#ifndef CUSYNC_MAX_NAPS
#define CUSYNC_MAX_NAPS 2
#endif

// First half of a poll by a whole wave: only the first active lane touches
// memory (sixty-four lanes loading the same coherent address are sixty-four
// requests to one memory channel).  The result stays in that lane's register so
// the wave need not wait for it yet; pollFinish() broadcasts it.
CUSYNC_DEVICE uint32_t pollBegin(const volatile uint32_t* addr) {
  uint32_t v = 0;
  const uint64_t exec = __builtin_amdgcn_read_exec();
  const uint32_t before = __builtin_amdgcn_mbcnt_hi((uint32_t)(exec >> 32), __builtin_amdgcn_mbcnt_lo((uint32_t)exec, 0u));
  if (before == 0) v = loadRelaxed(addr);
  return v;
}
CUSYNC_DEVICE uint32_t pollFinish(uint32_t begun) { return __builtin_amdgcn_readfirstlane(begun); }
CUSYNC_DEVICE uint32_t pollOnce(const volatile uint32_t* addr) { return pollFinish(pollBegin(addr)); }

// Polls *addr until it is >= want; returns false if the poll budget ran out.
// Sleeps between polls and doubles the sleep up to about a microsecond: a
// semaphore is one address, and hundreds of waves polling it back to back would
// saturate the memory channel it lives on and slow the very producer they are
// waiting for.
CUSYNC_DEVICE bool pollUntilAtLeast(const volatile uint32_t* addr, uint32_t want) {
  uint32_t polls = 0, naps = 1;
  while (pollOnce(addr) < want) {
    if (++polls >= CUSYNC_SPIN_LIMIT) return false;
    for (uint32_t i = 0; i < naps; i++) __builtin_amdgcn_s_sleep(16);   // 16 * 64 clocks
    if (naps < CUSYNC_MAX_NAPS) naps <<= 1;
  }
  return true;
}

// Spin until *addr >= want, then acquire at agent scope.  Meant to be executed
// by every lane of a wave with the same arguments (the loads coalesce into one
// request, the branch is uniform), or by a single lane.
CUSYNC_DEVICE bool spinUntilAtLeast(const volatile uint32_t* addr, uint32_t want) {
  const bool ok = pollUntilAtLeast(addr, want);
  acquireFence();
  return ok;
}

// Same without the cache invalidation of the acquire.  Only valid when no line
// of the guarded data can already sit in this XCD's caches (see DynStage).
// Program order is still kept: the loads that follow are issued after the poll
// returned.
CUSYNC_DEVICE bool spinUntilAtLeastNoInvalidate(const volatile uint32_t* addr, uint32_t want) {
  const bool ok = pollUntilAtLeast(addr, want);
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
  return ok;
}

// Release-add: everything the workgroup wrote before its last barrier becomes
// visible device-wide before the new count does.
CUSYNC_DEVICE void releaseAdd(volatile uint32_t* addr, uint32_t value) {
  __hip_atomic_fetch_add((uint32_t*)addr, value, __ATOMIC_RELEASE, __HIP_MEMORY_SCOPE_AGENT);
}

CUSYNC_DEVICE void releaseStore(volatile uint32_t* addr, uint32_t value) {
  __hip_atomic_store((uint32_t*)addr, value, __ATOMIC_RELEASE, __HIP_MEMORY_SCOPE_AGENT);
}

// The wait-kernel flag and the count of waits that gave up live in host memory that the device can reach, so that
// the host reads them without a copy: they are written at system scope.
CUSYNC_DEVICE void releaseStoreSystem(volatile uint32_t* addr, uint32_t value) {
  __hip_atomic_store((uint32_t*)addr, value, __ATOMIC_RELEASE, __HIP_MEMORY_SCOPE_SYSTEM);
}
CUSYNC_DEVICE void countGiveUp(uint32_t* addr) {
  __hip_atomic_fetch_add(addr, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
}

CUSYNC_DEVICE uint32_t ticketAdd(uint32_t* addr, uint32_t value) {
  return __hip_atomic_fetch_add(addr, value, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

CUSYNC_DEVICE void storeRelaxed(uint32_t* addr, uint32_t value) {
  __hip_atomic_store(addr, value, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

}  // namespace dev
}  // namespace cusync
#endif
