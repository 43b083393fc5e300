// CuSync for MI355X: tile-level synchronisation between dependent kernels that
// run concurrently on two HIP streams of one GPU.
//
// Public C++ API.  Type, member and enumerator names are those of the
// reference's src/include/cusync/cusync.h so that code written against it
// (stage construction, setProducerConsumerPair, invokeWaitKernel,
// incrementIter, and tile()/wait()/post() inside kernels) compiles unchanged.
// The host half compiles with any C++14 compiler and reaches the GPU only
// through the C ABI in cusync_amd.h; the device half is visible under hipcc.
#pragma once

#include <assert.h>
#include <stdint.h>
#include <stdio.h>
#include <stdlib.h>
#include <type_traits>
#include <vector>

#include "cusync_defines.h"
#include "../cusync_amd.h"
#include "device-functions.h"
#include "tile-orders.h"
#include "policies.h"

// Aborts on a failed runtime call, like CUDA_CHECK of the reference
// (src/include/cusync/cusync.h:16-23).  `cmd` is a cusync_rt_* call (0 = ok).
#define CUSYNC_RT_CHECK(cmd) do {                                     \
  int cusync_rt_status_ = (cmd);                                      \
  if (cusync_rt_status_ != 0) {                                       \
    printf("Failed: HIP error %s:%d '%s'\n", __FILE__, __LINE__,      \
           cusync_rt_last_error());                                   \
    exit(EXIT_FAILURE);                                               \
  }                                                                   \
} while (0)

#ifndef DIVUP
#define DIVUP(x, y) (((x) + (y) - 1) / (y))
#endif

namespace cusync {

class CuSyncTest;
struct CuSync;

// Same enumerators, same order, as src/include/cusync/cusync.h:46-53.
enum CuSyncError {
  CuSyncErrorNotProducer = CUSYNC_ERROR_NOT_PRODUCER,
  CuSyncErrorNotConsumer = CUSYNC_ERROR_NOT_CONSUMER,
  CuSyncErrorNotInitialized = CUSYNC_ERROR_NOT_INITIALIZED,
  CuSyncErrorInvalidLinearBlockIndex = CUSYNC_ERROR_INVALID_LINEAR_BLOCK_INDEX,
  CuSyncErrorCUDAError = CUSYNC_ERROR_DEVICE,
  CuSyncSuccess = CUSYNC_SUCCESS
};

// src/include/cusync/cusync.h:69-75.
enum Optimizations {
  NoOptimization   = CUSYNC_OPT_NONE,
  NoAtomicAdd      = CUSYNC_OPT_NO_ATOMIC_ADD,       // post stores postValue*iter instead of adding
  AvoidWaitKernel  = CUSYNC_OPT_AVOID_WAIT_KERNEL,   // all stages fit on the device at once
  AvoidCustomOrder = CUSYNC_OPT_AVOID_CUSTOM_ORDER,  // tiles follow the hardware's block order
  ReorderTileLoads = CUSYNC_OPT_REORDER_TILE_LOADS   // load the unsynchronised operand before waiting
};

// A CuStage describes one kernel of a chain: its grid, the grid of the kernel
// that feeds it, and how it synchronises on its input and its output.  It is a
// small trivially-copyable object; kernels take it by value.  Copies share the
// device buffers of the original.
template<typename TileOrder, typename InputSyncPolicy, typename OutputSyncPolicy, int Opts = NoOptimization>
class CuStage {
private:
  dim3 grid_;
  dim3 prodGrid_;
  dim3 tileSize_;
  int iter;                         // run counter, starts at 1
  InputSyncPolicy inputPolicy_;
  OutputSyncPolicy outputPolicy_;

  dim3* tileOrder;                  // device: ticket -> tile
  uint32_t* tileCounter;            // device: ticket dispenser
  uint32_t* startCounter_;          // device: used by the prebuilt persistent kernels
  uint32_t* xcdTickets_;            // device: per-XCD ticket dispensers of the prebuilt kernels
  uint32_t* kernelExecuted_;        // device: wait-kernel flag
  uint32_t* spinTimeouts_;          // device: waits that gave up
  volatile uint32_t* tileStatusWrite_;
  volatile uint32_t* tileStatusRead_;
  int status_;                      // outcome of the constructor
  uint32_t flags_;                  // CUSYNC_STAGE_* bits reported by cusync_stage_alloc

  friend class CuSyncTest;
  friend struct CuSync;

  // Fills the ticket -> tile table from TileOrder::blockIndex and uploads it
  // (src/include/cusync/cusync.h:125-157).  Unlike the reference an index outside
  // the table is rejected instead of written.
  CuSyncError buildScheduleBuffer() {
    const uint32_t n = numTiles();
    std::vector<cusync_dim3> order(n);
    std::vector<char> taken(n, 0);
    bool bad = false;
    for (uint32_t z = 0; z < grid_.z; z++)
      for (uint32_t y = 0; y < grid_.y; y++)
        for (uint32_t x = 0; x < grid_.x; x++) {
          const uint32_t id = TileOrder().blockIndex(grid_, dim3(x, y, z));
          if (id >= n || taken[id]) { bad = true; continue; }
          taken[id] = 1;
          order[id].x = x; order[id].y = y; order[id].z = z;
        }
    cusync_stage_desc d = desc();
    cusync_error e = cusync_stage_alloc(&d, order.data());
    if (e != CUSYNC_SUCCESS) {
      printf("Failed: HIP error %s:%d '%s'\n", __FILE__, __LINE__, cusync_rt_last_error());
      exit(EXIT_FAILURE);
    }
    tileOrder = (dim3*)d.tileOrder;
    tileCounter = d.tileCounter;
    startCounter_ = d.startCounter;
    xcdTickets_ = d.xcdTickets;
    flags_ = d.flags;
    kernelExecuted_ = d.kernelExecuted;
    spinTimeouts_ = d.spinTimeouts;
    tileStatusWrite_ = d.tileStatusWrite;
    return bad ? CuSyncErrorInvalidLinearBlockIndex : CuSyncSuccess;
  }

  template<typename ProdCuStage>
  void setProdGrid(ProdCuStage& prod) { prodGrid_ = prod.grid(); }

  CUSYNC_DEVICE_HOST volatile uint32_t* getTileStatusToPost() { return tileStatusWrite_; }
  CUSYNC_DEVICE_HOST volatile uint32_t* getTileStatusToWait() { return tileStatusRead_; }
  void setTileStatusToPost(volatile uint32_t* ptr) { tileStatusWrite_ = ptr; }
  void setTileStatusToWait(volatile uint32_t* ptr) { tileStatusRead_ = ptr; }

public:
  // tileSize is stored and never read, as in the reference (drivers pass {1,1,1}).
  CuStage(dim3 grid, dim3 tileSize, InputSyncPolicy inputPolicy, OutputSyncPolicy outputPolicy)
      : grid_(grid), prodGrid_(0, 0, 0), tileSize_(tileSize), iter(1),
        inputPolicy_(inputPolicy), outputPolicy_(outputPolicy),
        tileOrder(nullptr), tileCounter(nullptr), startCounter_(nullptr), xcdTickets_(nullptr), kernelExecuted_(nullptr), spinTimeouts_(nullptr),
        tileStatusWrite_(nullptr), tileStatusRead_(nullptr), status_(CuSyncSuccess), flags_(0) {
    static_assert(!((Opts & NoAtomicAdd) && std::is_same<OutputSyncPolicy, NoSync>::value &&
                    std::is_same<InputSyncPolicy, NoSync>::value), "NoAtomicAdd on a stage that never syncs");
    status_ = buildScheduleBuffer();
  }

  CUSYNC_DEVICE_HOST CuStage()
      : grid_(0, 0, 0), prodGrid_(0, 0, 0), tileSize_(0, 0, 0), iter(1),
        tileOrder(nullptr), tileCounter(nullptr), startCounter_(nullptr), xcdTickets_(nullptr), kernelExecuted_(nullptr), spinTimeouts_(nullptr),
        tileStatusWrite_(nullptr), tileStatusRead_(nullptr), status_(CuSyncErrorNotInitialized), flags_(0) {}

  // Outcome of construction: CuSyncSuccess, or CuSyncErrorInvalidLinearBlockIndex
  // when TileOrder::blockIndex is not a bijection onto [0, numTiles).
  CuSyncError status() const { return (CuSyncError)status_; }

  dim3 grid() { return grid_; }

  // Holds `stream` back until the producer kernel of the current run is on the
  // device (src/include/cusync/cusync.h:203-209).  For a run launched by one of
  // the library's launchers (CuSyncGemm::run, ...) the library picks the way
  // that suits that launch (cusync_hold_back): the reference's wait kernel, or,
  // where the launch took every workgroup slot of the device and a wait kernel's
  // wave would keep the producer's last workgroup off it, a wait on the calling
  // thread.  A kernel of the caller's own always gets the wait kernel.
  // `launchEvent` (optional, not in the reference): a hipEvent_t recorded on the
  // producer's stream right before the producer's launch.  `stream` then waits
  // for it first, so that the wait kernel's wave cannot reach the device ahead of
  // the producer's workgroups and hold a CU one of them needs.
  CuSyncError invokeWaitKernel(void* stream, void* launchEvent = nullptr) {
    if (!isProducer()) return CuSyncErrorNotProducer;
    if (getAvoidWaitKernel()) return CuSyncSuccess;
    if (kernelExecuted_ == nullptr) return CuSyncErrorNotInitialized;
    const cusync_stage_desc d = desc();
    if (launchEvent != nullptr) return (CuSyncError)cusync_invoke_wait_kernel_after(&d, stream, launchEvent);
    return (CuSyncError)cusync_hold_back(&d, stream);
  }

  void incrementIter() { iter += 1; }
  int iteration() const { return iter; }

  // Releases the device buffers.  Call once, on the object that was constructed
  // (not on a copy), after the last kernel using any copy has finished.
  void destroy() {
    cusync_stage_desc d = desc();
    cusync_stage_free(&d);
    tileOrder = nullptr; tileCounter = nullptr; startCounter_ = nullptr; xcdTickets_ = nullptr;
    kernelExecuted_ = nullptr; spinTimeouts_ = nullptr; tileStatusWrite_ = nullptr;
  }

  CUSYNC_DEVICE_HOST bool getNoAtomicAdd()      const { return (Opts & NoAtomicAdd) != 0; }
  CUSYNC_DEVICE_HOST bool getAvoidWaitKernel()  const { return (Opts & AvoidWaitKernel) != 0; }
  CUSYNC_DEVICE_HOST bool getReorderTileLoads() const { return (Opts & ReorderTileLoads) != 0; }
  CUSYNC_DEVICE_HOST bool getAvoidCustomOrder() const { return (Opts & AvoidCustomOrder) != 0; }

  CUSYNC_DEVICE_HOST bool isProducer() const { return !std::is_same<OutputSyncPolicy, NoSync>::value; }
  CUSYNC_DEVICE_HOST bool isConsumer() const { return !std::is_same<InputSyncPolicy, NoSync>::value; }

  CUSYNC_DEVICE_HOST uint32_t numTiles() const { return grid_.x * grid_.y * grid_.z; }

  // Run-time image of this stage for the prebuilt kernels (cusync_gemm_run, ...).
  cusync_stage_desc desc() const {
    cusync_stage_desc d = {};
    d.grid = {grid_.x, grid_.y, grid_.z};
    d.prodGrid = {prodGrid_.x, prodGrid_.y, prodGrid_.z};
    d.tileSize = {tileSize_.x, tileSize_.y, tileSize_.z};
    d.iter = iter;
    d.opts = Opts;
    d.flags = flags_;
    d.in = inputPolicy_.desc();
    d.out = outputPolicy_.desc();
    d.tileOrder = (cusync_dim3*)tileOrder;
    d.tileCounter = tileCounter;
    d.startCounter = startCounter_;
    d.xcdTickets = xcdTickets_;
    d.kernelExecuted = kernelExecuted_;
    d.spinTimeouts = spinTimeouts_;
    d.tileStatusWrite = (uint32_t*)tileStatusWrite_;
    d.tileStatusRead = (uint32_t*)tileStatusRead_;
    return d;
  }

  // Semaphore index this stage waits on for `tile`.
  CUSYNC_DEVICE_HOST uint32_t waitTileIndex(dim3 tile) { return inputPolicy_.tileIndex(tile, prodGrid_); }
  // Per-run count that semaphore must reach.
  CUSYNC_DEVICE_HOST uint32_t expectedWaitValue(dim3 tile) { return inputPolicy_.waitValue(tile, prodGrid_); }

#if CUSYNC_HAS_DEVICE
  // Current value of the semaphore guarding `tile`.
  CUSYNC_DEVICE uint32_t waitSemValue(dim3 tile) {
    return dev::loadAcquire(&tileStatusRead_[waitTileIndex(tile) * CUSYNC_SEM_STRIDE]);
  }

  // Blocks the workgroup until the producer has delivered `tile`.  Thread
  // `waitingThread` of the workgroup spins; with callSync the others are held
  // at a barrier, without it the caller must synchronise before touching the data.
  CUSYNC_DEVICE CuSyncError wait(dim3& tile, uint32_t waitingThread = 0, bool callSync = true);

  // Declares `tile` complete.  Contains a workgroup barrier, so every thread of
  // the workgroup must call it after its last store to the tile.
  CUSYNC_DEVICE CuSyncError post(const dim3& tile, uint32_t postThread = 0);
  // The wait-kernel flag and, for a host that holds the consumer back itself, its mirror in host memory.
  CUSYNC_DEVICE void raiseFlag() {
    dev::releaseStore(kernelExecuted_, (uint32_t)iter);
    dev::releaseStoreSystem(spinTimeouts_ + CUSYNC_HOST_FLAG_OFFSET, (uint32_t)iter);
  }

  // First statement of a sync-aware kernel: returns the tile this workgroup
  // processes (a ticket through the tile order, or blockIdx with
  // AvoidCustomOrder / a null shared_storage) and raises the wait-kernel flag.
  // The ticket is the workgroup's linear index when the launch has one workgroup
  // per tile, otherwise the next value of the stage's dispenser
  // (src/include/cusync/cusync_device_defs.h:77-103).
  CUSYNC_DEVICE dim3 tile(dim3* shared_storage);
#endif
};

struct CuSync {
  // Connects a producer to its consumer: the consumer learns the producer's grid
  // and waits on the producer's semaphores (src/include/cusync/cusync.h:289-298).
  template<typename Stage1, typename Stage2>
  static CuSyncError setProducerConsumerPair(Stage1& prod, Stage2& cons) {
    if (!prod.isProducer()) return CuSyncErrorNotProducer;
    if (!cons.isConsumer()) return CuSyncErrorNotConsumer;
    if (prod.getTileStatusToPost() == nullptr) return CuSyncErrorNotInitialized;
    cons.setProdGrid(prod);
    cons.setTileStatusToWait(prod.getTileStatusToPost());
    return CuSyncSuccess;
  }
};

#if CUSYNC_HAS_DEVICE

#define CUSTAGE_METHOD(RET) \
  template<typename TileOrder, typename InputSyncPolicy, typename OutputSyncPolicy, int Opts> \
  CUSYNC_DEVICE RET CuStage<TileOrder, InputSyncPolicy, OutputSyncPolicy, Opts>::

CUSTAGE_METHOD(CuSyncError) wait(dim3& tile, uint32_t waitingThread, bool callSync) {
  if (!isConsumer()) return CuSyncErrorNotConsumer;
  if (!inputPolicy_.isSync(tile, prodGrid_)) return CuSyncSuccess;
  const uint32_t flat = threadIdx.x + blockDim.x * (threadIdx.y + blockDim.y * threadIdx.z);
  if (flat == waitingThread) {
    const uint32_t need = (uint32_t)iter * inputPolicy_.waitValue(tile, prodGrid_);
    const uint32_t idx = inputPolicy_.tileIndex(tile, prodGrid_);
    if (!dev::spinUntilAtLeast(&tileStatusRead_[idx * CUSYNC_SEM_STRIDE], need)) dev::countGiveUp(spinTimeouts_);
  }
  if (callSync) __syncthreads();
  return CuSyncSuccess;
}

CUSTAGE_METHOD(CuSyncError) post(const dim3& tile, uint32_t postThread) {
  if (!isProducer()) return CuSyncErrorNotProducer;
  // Every wavefront sees its own stores through to memory first: a workgroup barrier does not wait for them, and
  // the release below, issued by one thread, waits for the stores of that thread's wavefront only.
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  __syncthreads();
  const uint32_t flat = threadIdx.x + blockDim.x * (threadIdx.y + blockDim.y * threadIdx.z);
  if (flat == postThread) {
    const uint32_t idx = outputPolicy_.tileIndex(tile, grid_);
    const uint32_t value = outputPolicy_.postValue(tile, grid_);
    if (getNoAtomicAdd()) dev::releaseStore(&tileStatusWrite_[idx * CUSYNC_SEM_STRIDE], value * (uint32_t)iter);
    else dev::releaseAdd(&tileStatusWrite_[idx * CUSYNC_SEM_STRIDE], value);
  }
  return CuSyncSuccess;
}

CUSTAGE_METHOD(dim3) tile(dim3* shared_storage) {
  const bool leader = threadIdx.x == 0 && threadIdx.y == 0 && threadIdx.z == 0;
  const bool raisesFlag = !getAvoidWaitKernel() && isProducer();
  if (getAvoidCustomOrder() || shared_storage == nullptr) {
    // Hardware order.  Only the first block can speak for the kernel being on
    // the device; the caller vouches that the rest fits beside its consumer.
    if (raisesFlag && leader && blockIdx.x == 0 && blockIdx.y == 0 && blockIdx.z == 0)
      raiseFlag();
    return dim3(blockIdx.x, blockIdx.y, blockIdx.z);
  }
  if (leader) {
    const uint32_t launched = gridDim.x * gridDim.y * gridDim.z;
    uint32_t ticket;
    if (launched == numTiles()) {
      // One workgroup per tile, the usual launch: the ticket is the workgroup's linear index, which the hardware
      // hands out in increasing order, and nobody touches the dispenser (a device-wide atomic that every workgroup
      // of a launch hits at kernel start costs the launch about 11 ns per workgroup, one after the other).
      ticket = blockIdx.x + gridDim.x * (blockIdx.y + gridDim.y * blockIdx.z);
      if (raisesFlag) {
        // Every workgroup of this run has started once all have been counted.  They are counted in eight lists by
        // index modulo 8 (the workgroups of a list share an XCD, and the eight counters eight memory channels); the
        // last of a list reports for it, the last list to report raises the flag.  Whoever closes a count re-arms it.
        const uint32_t list = ticket & 7u, members = (launched - list + 7u) / 8u, lists = launched < 8u ? launched : 8u;
        if (dev::ticketAdd(&xcdTickets_[list * 32], 1) == members - 1) {
          dev::storeRelaxed(&xcdTickets_[list * 32], 0);
          if (dev::ticketAdd(&xcdTickets_[8 * 32], 1) == lists - 1) {
            dev::storeRelaxed(&xcdTickets_[8 * 32], 0);
            raiseFlag();
          }
        }
      }
    } else {
      ticket = dev::ticketAdd(tileCounter, 1);
      if (ticket == numTiles() - 1) {
        // Last ticket: every workgroup of this run has started, so none of them
        // can be kept off the device by a spinning consumer.  Re-arm the
        // dispenser and let the consumer's stream go.
        dev::storeRelaxed(tileCounter, 0);
        if (raisesFlag) raiseFlag();
      }
    }
    *shared_storage = tileOrder[ticket];
  }
  __syncthreads();
  return *shared_storage;
}

#undef CUSTAGE_METHOD
#endif  // CUSYNC_HAS_DEVICE

}  // namespace cusync
