// Thin runtime layer of libcusync_amd.so: the only translation unit besides the
// kernel launchers that calls the HIP runtime.  Implements the cusync_rt_*,
// cusync_stage_* and wait-kernel entry points declared in include/cusync_amd.h.
#include <hip/hip_runtime.h>

#include <stdio.h>
#include <stdlib.h>
#include <string.h>
#include <algorithm>
#include <chrono>
#include <string>
#include <vector>

#include "../../include/cusync_amd.h"
#include "../../include/cusync/device-functions.h"
#include "policy_eval.h"
#include "rt_internal.h"

namespace cusync {
namespace rt {

static thread_local std::string g_last_error;

void setError(const std::string& msg) { g_last_error = msg; }

int check(hipError_t e, const char* what, const char* file, int line) {
  if (e == hipSuccess) return 0;
  char buf[512];
  snprintf(buf, sizeof buf, "%s failed at %s:%d: %s", what, file, line, hipGetErrorString(e));
  g_last_error = buf;
  return (int)e;
}

static unsigned long long* g_timeline = nullptr;
static uint32_t g_timelineCap = 0;
void timeline(unsigned long long** buffer, uint32_t* capacity) { *buffer = g_timeline; *capacity = g_timelineCap; }
void setTimeline(unsigned long long* buffer, uint32_t capacity) { g_timeline = buffer; g_timelineCap = capacity; }

bool forceAcquire() {
  static const bool on = [] {
    const char* v = getenv("CUSYNC_FORCE_ACQUIRE");
    return v && *v && strcmp(v, "0") != 0;
  }();
  return on;
}

bool forceRelease() {
  static const bool on = [] {
    const char* v = getenv("CUSYNC_FORCE_RELEASE");
    return v && *v && strcmp(v, "0") != 0;
  }();
  return on;
}

bool forceWaitKernel() {
  static const bool on = [] {
    const char* v = getenv("CUSYNC_WAIT_KERNEL");
    return v && *v && strcmp(v, "0") != 0;
  }();
  return on;
}

bool spinTimeoutsOf(const cusync_stage_desc* const* stages, int count, uint32_t* sum) {
  uint32_t total = 0;
  for (int i = 0; i < count; i++) {
    if (!stages[i] || !stages[i]->spinTimeouts) continue;
    total += __atomic_load_n(stages[i]->spinTimeouts, __ATOMIC_ACQUIRE);     // host memory: no copy
  }
  *sum = total;
  return true;
}

cusync_error checkSpinTimeouts(const cusync_stage_desc* const* stages, int count, uint32_t* seen, const char* what) {
  uint32_t now = 0;
  if (!spinTimeoutsOf(stages, count, &now)) return CUSYNC_ERROR_DEVICE;
  if (now == *seen) return CUSYNC_SUCCESS;
  char buf[256];
  snprintf(buf, sizeof buf, "%s: %u wait(s) gave up after CUSYNC_SPIN_LIMIT polls and went on with data that was not "
                            "posted; the outputs of this call are not valid", what, now - *seen);
  *seen = now;
  setError(buf);
  return CUSYNC_ERROR_DEVICE;
}

}  // namespace rt
}  // namespace cusync

#define RT(call) CUSYNC_HIP(call)

// One wave; lane 0 polls.  Same contract as waitKernel of the reference
// (src/cusync.cu:11-19) with a bounded spin.
// A wait that gives up is counted in *timeouts (may be null), as the waits inside the kernels are.
__global__ void cusync_wait_kernel_impl(const uint32_t* semaphore, uint32_t value, uint32_t* timeouts) {
  if (threadIdx.x == 0 && !cusync::dev::spinUntilAtLeast(semaphore, value) && timeouts) cusync::dev::countGiveUp(timeouts);
}

extern "C" {

const char* cusync_rt_last_error(void) { return cusync::rt::g_last_error.c_str(); }

cusync_error cusync_rt_set_timeline(void* device_buffer, size_t bytes) {
  if (!device_buffer || bytes < 72) { cusync::rt::setTimeline(nullptr, 0); return CUSYNC_SUCCESS; }
  if ((uintptr_t)device_buffer % 8) { cusync::rt::setError("timeline: the buffer must be 8-byte aligned"); return CUSYNC_ERROR_NOT_INITIALIZED; }
  cusync::rt::setTimeline((unsigned long long*)device_buffer, (uint32_t)std::min<size_t>((bytes - 8) / 64, 0xffffffffu));
  return CUSYNC_SUCCESS;
}

int cusync_rt_device_count(void) {
  int n = 0;
  if (hipGetDeviceCount(&n) != hipSuccess) return 0;
  return n;
}

int cusync_rt_device_info(int* num_cus, int* clock_khz, size_t* lds_per_cu, size_t* hbm_bytes,
                          char* name, size_t name_len) {
  hipDeviceProp_t p;
  int dev = 0;
  if (RT(hipGetDevice(&dev))) return 1;
  if (RT(hipGetDeviceProperties(&p, dev))) return 1;
  if (num_cus) *num_cus = p.multiProcessorCount;
  if (clock_khz) *clock_khz = p.clockRate;
  if (lds_per_cu) *lds_per_cu = p.maxSharedMemoryPerMultiProcessor;
  if (hbm_bytes) *hbm_bytes = p.totalGlobalMem;
  if (name && name_len) { strncpy(name, p.gcnArchName, name_len - 1); name[name_len - 1] = 0; }
  return 0;
}

int cusync_rt_malloc(void** ptr, size_t bytes) { return RT(hipMalloc(ptr, bytes)); }
int cusync_rt_free(void* ptr) { return RT(hipFree(ptr)); }
int cusync_rt_memset(void* ptr, int value, size_t bytes) { return RT(hipMemset(ptr, value, bytes)); }
int cusync_rt_memcpy_h2d(void* dst, const void* src, size_t bytes) { return RT(hipMemcpy(dst, src, bytes, hipMemcpyHostToDevice)); }
int cusync_rt_memcpy_d2h(void* dst, const void* src, size_t bytes) { return RT(hipMemcpy(dst, src, bytes, hipMemcpyDeviceToHost)); }
int cusync_rt_memcpy_d2d(void* dst, const void* src, size_t bytes) { return RT(hipMemcpy(dst, src, bytes, hipMemcpyDeviceToDevice)); }
// Default priority on purpose: the chain's forward progress does not depend on
// queue priorities (see stage_device.h).
int cusync_rt_stream_create(void** stream) { return RT(hipStreamCreateWithFlags((hipStream_t*)stream, hipStreamNonBlocking)); }
int cusync_rt_stream_destroy(void* stream) { return RT(hipStreamDestroy((hipStream_t)stream)); }
int cusync_rt_stream_sync(void* stream) { return RT(hipStreamSynchronize((hipStream_t)stream)); }
int cusync_rt_device_sync(void) { return RT(hipDeviceSynchronize()); }
int cusync_rt_event_create(void** event) { return RT(hipEventCreate((hipEvent_t*)event)); }
int cusync_rt_event_destroy(void* event) { return RT(hipEventDestroy((hipEvent_t)event)); }
int cusync_rt_event_record(void* event, void* stream) { return RT(hipEventRecord((hipEvent_t)event, (hipStream_t)stream)); }
int cusync_rt_event_sync(void* event) { return RT(hipEventSynchronize((hipEvent_t)event)); }
int cusync_rt_event_elapsed_us(void* start, void* end, double* us) {
  float ms = 0;
  int rc = RT(hipEventElapsedTime(&ms, (hipEvent_t)start, (hipEvent_t)end));
  if (us) *us = (double)ms * 1000.0;
  return rc;
}
int cusync_rt_stream_wait_event(void* stream, void* event) { return RT(hipStreamWaitEvent((hipStream_t)stream, (hipEvent_t)event, 0)); }

/* ---- stages --------------------------------------------------------------- */

static uint32_t numTiles(const cusync_stage_desc* d) { return d->grid.x * d->grid.y * d->grid.z; }

cusync_error cusync_stage_alloc(cusync_stage_desc* d, const cusync_dim3* host_tile_order) {
  if (!d || !host_tile_order) return CUSYNC_ERROR_NOT_INITIALIZED;
  const uint32_t n = numTiles(d);
  if (n == 0) { cusync::rt::setError("cusync_stage_alloc: empty grid"); return CUSYNC_ERROR_NOT_INITIALIZED; }
  d->tileOrder = nullptr; d->tileCounter = nullptr; d->startCounter = nullptr; d->xcdTickets = nullptr;
  d->kernelExecuted = nullptr; d->spinTimeouts = nullptr; d->tileStatusWrite = nullptr;
  // The small device counters share one allocation: [tileCounter, startCounter, -, kernelExecuted, xcdTickets[9]], each on its
  // own 128-byte line so that polling one does not disturb the others.
  const size_t line = 128;
  char* counters = nullptr;
  if (RT(hipMalloc((void**)&counters, 13 * line))) return CUSYNC_ERROR_DEVICE;
  d->tileCounter = (uint32_t*)(counters);         // base of the block: what cusync_stage_free releases
  // a failure from here on gives back what was allocated so far; the text of the failed call is kept
  auto fail = [&]() {
    const std::string why = cusync_rt_last_error();
    cusync_stage_free(d);
    cusync::rt::setError(why);
    return CUSYNC_ERROR_DEVICE;
  };
  if (RT(hipMemset(counters, 0, 13 * line))) return fail();
  d->startCounter = (uint32_t*)(counters + line);
  d->xcdTickets = (uint32_t*)(counters + 4 * line);
  // The two words the host wants to look at while kernels run, or without a copy after them, live in pinned host
  // memory the device reaches over the bus: the count of waits that gave up (first line: the base of the block)
  // and a mirror of the wait-kernel flag (second line, CUSYNC_HOST_FLAG_OFFSET words on).  Each is written at most
  // once per kernel; the flag the wait kernel polls stays in device memory.
  char* shared = nullptr;
  if (RT(hipHostMalloc((void**)&shared, 2 * line, hipHostMallocDefault))) return fail();
  memset(shared, 0, 2 * line);
  d->spinTimeouts = (uint32_t*)shared;
  const bool producer = d->out.kind != CUSYNC_POLICY_NOSYNC;
  if (producer && !(d->opts & CUSYNC_OPT_AVOID_WAIT_KERNEL)) d->kernelExecuted = (uint32_t*)(counters + 3 * line);
  bool identity = true;
  for (uint32_t i = 0; i < n && identity; i++) {
    const cusync_dim3& t = host_tile_order[i];
    identity = t.x == i % d->grid.x && t.y == (i / d->grid.x) % d->grid.y && t.z == i / (d->grid.x * d->grid.y);
  }
  d->flags = identity ? CUSYNC_STAGE_IDENTITY_ORDER : 0;
  if (RT(hipMalloc((void**)&d->tileOrder, sizeof(cusync_dim3) * n))) return fail();
  if (RT(hipMemcpy(d->tileOrder, host_tile_order, sizeof(cusync_dim3) * n, hipMemcpyHostToDevice))) return fail();
  if (producer) {
    if (RT(hipMalloc((void**)&d->tileStatusWrite, sizeof(uint32_t) * n * CUSYNC_SEM_STRIDE))) return fail();
    if (RT(hipMemset(d->tileStatusWrite, 0, sizeof(uint32_t) * n * CUSYNC_SEM_STRIDE))) return fail();
  }
  return CUSYNC_SUCCESS;
}

cusync_error cusync_stage_free(cusync_stage_desc* d) {
  if (!d) return CUSYNC_ERROR_NOT_INITIALIZED;
  int bad = 0;
  if (d->tileCounter) bad |= RT(hipFree(d->tileCounter));       // base of the counters block
  if (d->spinTimeouts) bad |= RT(hipHostFree(d->spinTimeouts));  // base of the block in host memory
  if (d->tileOrder) bad |= RT(hipFree(d->tileOrder));
  if (d->tileStatusWrite) bad |= RT(hipFree(d->tileStatusWrite));
  d->tileOrder = nullptr; d->tileCounter = nullptr; d->startCounter = nullptr; d->xcdTickets = nullptr;
  d->kernelExecuted = nullptr; d->spinTimeouts = nullptr; d->tileStatusWrite = nullptr;
  return bad ? CUSYNC_ERROR_DEVICE : CUSYNC_SUCCESS;
}

cusync_error cusync_stage_create(cusync_stage_desc* d, int order) {
  if (!d) return CUSYNC_ERROR_NOT_INITIALIZED;
  const uint32_t n = numTiles(d);
  if (n == 0) { cusync::rt::setError("cusync_stage_create: empty grid"); return CUSYNC_ERROR_NOT_INITIALIZED; }
  std::vector<cusync_dim3> host(n);
  std::vector<char> taken(n, 0);
  bool bad = false;
  for (uint32_t z = 0; z < d->grid.z; z++)
    for (uint32_t y = 0; y < d->grid.y; y++)
      for (uint32_t x = 0; x < d->grid.x; x++) {
        cusync_dim3 b = {x, y, z};
        const uint32_t id = cusync::dyn::blockIndex(order, d->grid, b);
        if (id >= n || taken[id]) { bad = true; continue; }
        taken[id] = 1;
        host[id] = b;
      }
  d->iter = d->iter > 0 ? d->iter : 1;
  cusync_error e = cusync_stage_alloc(d, host.data());
  if (e != CUSYNC_SUCCESS) return e;
  return bad ? CUSYNC_ERROR_INVALID_LINEAR_BLOCK_INDEX : CUSYNC_SUCCESS;
}

cusync_error cusync_set_producer_consumer_pair(const cusync_stage_desc* prod, cusync_stage_desc* cons) {
  if (!prod || !cons) return CUSYNC_ERROR_NOT_INITIALIZED;
  if (prod->out.kind == CUSYNC_POLICY_NOSYNC) return CUSYNC_ERROR_NOT_PRODUCER;
  if (cons->in.kind == CUSYNC_POLICY_NOSYNC) return CUSYNC_ERROR_NOT_CONSUMER;
  if (prod->tileStatusWrite == nullptr) return CUSYNC_ERROR_NOT_INITIALIZED;
  cons->prodGrid = prod->grid;
  cons->tileStatusRead = prod->tileStatusWrite;
  return CUSYNC_SUCCESS;
}

static cusync_error launchWaitKernel(uint32_t* semaphore, uint32_t value, uint32_t* timeouts, void* stream) {
  if (!semaphore) return CUSYNC_ERROR_NOT_INITIALIZED;
  hipLaunchKernelGGL(cusync_wait_kernel_impl, dim3(1), dim3(64), 0, (hipStream_t)stream, semaphore, value, timeouts);
  if (RT(hipGetLastError())) return CUSYNC_ERROR_DEVICE;
  return CUSYNC_SUCCESS;
}

cusync_error cusync_wait_kernel(uint32_t* semaphore, uint32_t value, void* stream) {
  return launchWaitKernel(semaphore, value, nullptr, stream);
}

cusync_error cusync_invoke_wait_kernel(const cusync_stage_desc* prod, void* stream) {
  if (!prod) return CUSYNC_ERROR_NOT_INITIALIZED;
  if (prod->out.kind == CUSYNC_POLICY_NOSYNC) return CUSYNC_ERROR_NOT_PRODUCER;
  if (prod->opts & CUSYNC_OPT_AVOID_WAIT_KERNEL) return CUSYNC_SUCCESS;
  return launchWaitKernel(prod->kernelExecuted, (uint32_t)prod->iter, prod->spinTimeouts, stream);
}

cusync_error cusync_invoke_wait_kernel_after(const cusync_stage_desc* prod, void* stream, void* launch_event) {
  if (!prod) return CUSYNC_ERROR_NOT_INITIALIZED;
  if (prod->out.kind == CUSYNC_POLICY_NOSYNC) return CUSYNC_ERROR_NOT_PRODUCER;
  if (prod->opts & CUSYNC_OPT_AVOID_WAIT_KERNEL) return CUSYNC_SUCCESS;
  if (launch_event && RT(hipStreamWaitEvent((hipStream_t)stream, (hipEvent_t)launch_event, 0))) return CUSYNC_ERROR_DEVICE;
  return launchWaitKernel(prod->kernelExecuted, (uint32_t)prod->iter, prod->spinTimeouts, stream);
}

// Polls the host-memory mirror of the producer's flag.  *timedOut says whether a failure was the time limit.
static cusync_error waitStartedOnHost(const cusync_stage_desc* prod, uint32_t timeout_ms, bool* timedOut) {
  *timedOut = false;
  if (!prod) return CUSYNC_ERROR_NOT_INITIALIZED;
  if (prod->out.kind == CUSYNC_POLICY_NOSYNC) return CUSYNC_ERROR_NOT_PRODUCER;
  if (prod->opts & CUSYNC_OPT_AVOID_WAIT_KERNEL) return CUSYNC_SUCCESS;
  if (!prod->kernelExecuted) return CUSYNC_ERROR_NOT_INITIALIZED;
  const auto t0 = std::chrono::steady_clock::now();
  const uint32_t want = (uint32_t)prod->iter;
  for (uint32_t spins = 0;; spins++) {
    if (__atomic_load_n(prod->spinTimeouts + CUSYNC_HOST_FLAG_OFFSET, __ATOMIC_ACQUIRE) >= want) return CUSYNC_SUCCESS;
    __builtin_ia32_pause();      // the flag arrives over the bus: leave the core's other thread and the memory pipeline alone meanwhile
    if ((spins & 1023u) == 1023u &&
        std::chrono::steady_clock::now() - t0 > std::chrono::milliseconds(timeout_ms ? timeout_ms : 2000)) {
      cusync::rt::setError("cusync_wait_producer_started: the producer's workgroups did not all start in time");
      *timedOut = true;
      return CUSYNC_ERROR_DEVICE;
    }
  }
}

cusync_error cusync_wait_producer_started(const cusync_stage_desc* prod, uint32_t timeout_ms) {
  bool timedOut;
  return waitStartedOnHost(prod, timeout_ms, &timedOut);
}

extern "C++" { namespace cusync { namespace rt {
void noteLaunch(const cusync_stage_desc& stage, bool fillsDevice) {
  if (stage.out.kind == CUSYNC_POLICY_NOSYNC || !stage.spinTimeouts) return;
  __atomic_store_n(stage.spinTimeouts + CUSYNC_HOST_FLAG_OFFSET + 1, fillsDevice ? (uint32_t)stage.iter : 0u, __ATOMIC_RELAXED);
}
}} }

cusync_error cusync_hold_back(const cusync_stage_desc* prod, void* stream) {
  if (!prod) return CUSYNC_ERROR_NOT_INITIALIZED;
  if (prod->out.kind == CUSYNC_POLICY_NOSYNC) return CUSYNC_ERROR_NOT_PRODUCER;
  if (prod->opts & CUSYNC_OPT_AVOID_WAIT_KERNEL) return CUSYNC_SUCCESS;
  if (!prod->kernelExecuted || !prod->spinTimeouts) return CUSYNC_ERROR_NOT_INITIALIZED;
  const bool filled = __atomic_load_n(prod->spinTimeouts + CUSYNC_HOST_FLAG_OFFSET + 1, __ATOMIC_RELAXED) == (uint32_t)prod->iter;
  if (filled && !cusync::rt::forceWaitKernel()) {
    // a stream that is being captured has launched nothing yet: the flag would never rise while this thread waits
    hipStreamCaptureStatus capturing = hipStreamCaptureStatusNone;
    if (RT(hipStreamIsCapturing((hipStream_t)stream, &capturing))) return CUSYNC_ERROR_DEVICE;
    if (capturing == hipStreamCaptureStatusNone) {
      bool timedOut = false;
      const cusync_error e = waitStartedOnHost(prod, 0, &timedOut);
      if (e == CUSYNC_SUCCESS || !timedOut) return e;
      // The producer is queued behind other work of the device, or its launch was refused: the wait kernel holds
      // the consumer's stream back from here on, with its own bounded wait and its own count of waits that gave up.
    }
  }
  return launchWaitKernel(prod->kernelExecuted, (uint32_t)prod->iter, prod->spinTimeouts, stream);
}

cusync_error cusync_stage_read_state(const cusync_stage_desc* d, uint32_t* sems, cusync_dim3* tile_order,
                                     uint32_t* tile_counter, uint32_t* start_counter,
                                     uint32_t* kernel_executed, uint32_t* spin_timeouts) {
  if (!d) return CUSYNC_ERROR_NOT_INITIALIZED;
  const uint32_t n = numTiles(d);
  int bad = 0;
  if (sems) {
    if (!d->tileStatusWrite) return CUSYNC_ERROR_NOT_PRODUCER;
    bad |= RT(hipMemcpy2D(sems, sizeof(uint32_t), d->tileStatusWrite, sizeof(uint32_t) * CUSYNC_SEM_STRIDE, sizeof(uint32_t), n,
                          hipMemcpyDeviceToHost));      // one semaphore per 128-byte line on the device, packed for the caller
  }
  if (tile_order) bad |= RT(hipMemcpy(tile_order, d->tileOrder, sizeof(cusync_dim3) * n, hipMemcpyDeviceToHost));
  if (tile_counter) {
    // the plain dispenser plus the nine per-XCD counters: all must be back at 0 between runs
    uint32_t block[13 * 32];
    bad |= RT(hipMemcpy(block, d->tileCounter, sizeof block, hipMemcpyDeviceToHost));
    uint32_t sum = block[0];
    for (int i = 0; i < 9; i++) sum += block[(4 + i) * 32];
    *tile_counter = sum;
  }
  if (start_counter) bad |= RT(hipMemcpy(start_counter, d->startCounter, 4, hipMemcpyDeviceToHost));
  if (spin_timeouts) *spin_timeouts = d->spinTimeouts ? __atomic_load_n(d->spinTimeouts, __ATOMIC_ACQUIRE) : 0;
  if (kernel_executed) {       // the flag's mirror in host memory, which the producer writes right after the flag
    *kernel_executed = 0;
    if (d->kernelExecuted) {
      uint32_t dev = 0;
      bad |= RT(hipMemcpy(&dev, d->kernelExecuted, 4, hipMemcpyDeviceToHost));
      const uint32_t host = __atomic_load_n(d->spinTimeouts + CUSYNC_HOST_FLAG_OFFSET, __ATOMIC_ACQUIRE);
      *kernel_executed = dev == host ? dev : 0xffffffffu;     // the two must agree once the device is idle
    }
  }
  return bad ? CUSYNC_ERROR_DEVICE : CUSYNC_SUCCESS;
}

/* ---- host evaluation of policies -------------------------------------------- */

uint32_t cusync_policy_tile_index(const cusync_policy_desc* p, cusync_dim3 tile, cusync_dim3 grid) {
  return cusync::dyn::tileIndex(*p, tile, grid);
}
uint32_t cusync_policy_wait_value(const cusync_policy_desc* p, cusync_dim3 tile, cusync_dim3 grid) {
  (void)tile; (void)grid;
  return cusync::dyn::waitValue(*p);
}
uint32_t cusync_policy_post_value(const cusync_policy_desc* p, cusync_dim3 tile, cusync_dim3 grid) {
  (void)tile; (void)grid;
  return cusync::dyn::postValue(*p);
}
int cusync_policy_is_sync(const cusync_policy_desc* p, cusync_dim3 tile, cusync_dim3 grid) {
  (void)grid;
  return cusync::dyn::isSync(*p, tile) ? 1 : 0;
}
uint32_t cusync_order_block_index(int order, cusync_dim3 grid, cusync_dim3 block) {
  return cusync::dyn::blockIndex(order, grid, block);
}
cusync_dim3 cusync_order_tile_to_block(int order, cusync_dim3 tile) {
  return cusync::dyn::tileToBlock(order, tile);
}

}  // extern "C"
