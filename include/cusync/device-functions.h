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
// trip to the coherent level of the memory system plus a short sleep, i.e. of
// the order of a microsecond, so the default allows a few seconds.
#ifndef CUSYNC_SPIN_LIMIT
#define CUSYNC_SPIN_LIMIT (1u << 22)
#endif

// Spin until *addr >= want; returns false if the poll budget ran out first.
// Meant to be executed by every lane of a wave with the same arguments (the
// loads coalesce into one request, the branch is uniform), or by a single lane.
// s_sleep yields issue slots to the waves that do the producer's work on the
// same CU.
CUSYNC_DEVICE bool spinUntilAtLeast(const volatile uint32_t* addr, uint32_t want) {
  uint32_t polls = 0;
  bool ok = true;
  while (loadRelaxed(addr) < want) {
    if (++polls >= CUSYNC_SPIN_LIMIT) { ok = false; break; }
    __builtin_amdgcn_s_sleep(2);
  }
  acquireFence();
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

CUSYNC_DEVICE uint32_t ticketAdd(uint32_t* addr, uint32_t value) {
  return __hip_atomic_fetch_add(addr, value, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

CUSYNC_DEVICE void storeRelaxed(uint32_t* addr, uint32_t value) {
  __hip_atomic_store(addr, value, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

}  // namespace dev
}  // namespace cusync
#endif
