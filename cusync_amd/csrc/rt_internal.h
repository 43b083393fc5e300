// Shared between the translation units of libcusync_amd.so; not installed.
#pragma once

#include <hip/hip_runtime.h>
#include <string>

#include "../../include/cusync_amd.h"

namespace cusync {
namespace rt {
// Records `msg` as the text cusync_rt_last_error() returns (per host thread).
void setError(const std::string& msg);
// Returns 0 on hipSuccess; otherwise records a message and returns the code.
int check(hipError_t e, const char* what, const char* file, int line);
// True when the environment variable CUSYNC_FORCE_ACQUIRE is set to something other than 0: every consumer
// wait then ends with the agent-scope acquire (cache invalidation), also where the launcher found that the
// producer's tiles are whole cache lines of the consumer's operand and the invalidation can be skipped.
bool forceAcquire();
// True when CUSYNC_FORCE_RELEASE is set to something other than 0: every post of the library's kernels and every
// count their k-slices and key-range splits hand partial results over with is a device-scope release (the counts'
// readers acquire), also where the data was written through and acknowledged and the count is normally relaxed.
// With CUSYNC_FORCE_ACQUIRE this is the plain release/acquire protocol end to end; results must be the same.
bool forceRelease();
// True when CUSYNC_WAIT_KERNEL is set to something other than 0: the chain handles then hold every consumer back
// with the wait kernel, also behind a producer whose launch takes every workgroup slot (where they would wait on
// the host).  For measuring what the host-side hold is there to prevent.
bool forceWaitKernel();
// Called by a kernel launcher right after it launched a run of `stage`: records, in the stage's block of host memory,
// whether that launch took every workgroup slot of the device.  cusync_hold_back reads it.  No-op for a stage that
// posts nothing.
void noteLaunch(const cusync_stage_desc& stage, bool fillsDevice);
// Adds up the counters of waits that gave up (cusync_stage_desc::spinTimeouts) of the stages given; null
// entries and stages without a counter are skipped.  Returns false if a copy from the device failed.
bool spinTimeoutsOf(const cusync_stage_desc* const* stages, int count, uint32_t* sum);
// For the chain handles, after the host has synchronised with a run: CUSYNC_SUCCESS if the sum above still
// equals *seen, else records a message naming `what`, brings *seen up to date and returns CUSYNC_ERROR_DEVICE
// (the chain went on with data its producer had not posted: the outputs of that run are not valid).
// The diagnosis buffer set with cusync_rt_set_timeline (null when off) and the records it holds.
void timeline(unsigned long long** buffer, uint32_t* capacity);
void setTimeline(unsigned long long* buffer, uint32_t capacity);
cusync_error checkSpinTimeouts(const cusync_stage_desc* const* stages, int count, uint32_t* seen, const char* what);
}  // namespace rt
}  // namespace cusync

#define CUSYNC_HIP(call) ::cusync::rt::check((call), #call, __FILE__, __LINE__)
