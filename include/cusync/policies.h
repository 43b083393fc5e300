// Synchronisation policies.
//
// A policy decides, for a tile given as {row offset, column offset, z} in
// ELEMENTS of the producer's output, which semaphore guards it (tileIndex), what
// count that semaphore must reach per run (waitValue), what a producer adds when
// it finishes a tile (postValue) and whether a wait on that tile is needed at
// all (isSync).  Concept and names follow src/include/cusync/policies.h:7-13 of
// the reference; StridedSync and ConsecutiveSync live in the reference's drivers
// (src/ml-bench/transformer/mlp.cu:76-101, attention.cu:51-70) and are part of
// the library here.
//
// Every policy also reports a cusync_policy_desc so that the prebuilt kernels,
// which evaluate policies at run time, can be driven from these types.
#pragma once

#include "cusync_defines.h"
#include "tile-orders.h"
#include "../cusync_amd.h"

namespace cusync {

namespace detail {
inline cusync_policy_desc makePolicyDesc(int kind, int order, uint32_t tileM, uint32_t tileN,
                                         uint32_t waitValue, uint32_t postValue) {
  cusync_policy_desc d = {};
  d.kind = kind; d.order = order;
  d.tileM = tileM; d.tileN = tileN;
  d.waitValue = waitValue; d.postValue = postValue;
  d.R = 1; d.S = 1;
  return d;
}
}  // namespace detail

// Marks the side of a stage that does not synchronise.  A stage is a producer
// iff its output policy is not NoSync and a consumer iff its input policy is not.
struct NoSync {
  CUSYNC_DEVICE_HOST NoSync() {}
  CUSYNC_DEVICE_HOST uint32_t waitValue(const dim3&, const dim3&) const { return 0; }
  CUSYNC_DEVICE_HOST uint32_t tileIndex(const dim3&, const dim3&) const { return 0; }
  CUSYNC_DEVICE_HOST bool isSync(const dim3&, const dim3&) const { return false; }
  CUSYNC_DEVICE_HOST uint32_t postValue(const dim3&, const dim3&) const { return 0; }
  cusync_policy_desc desc() const { return detail::makePolicyDesc(CUSYNC_POLICY_NOSYNC, 0, 1, 1, 0, 0); }
};

// One semaphore per row of tiles.  A consumer waits once, before its main loop
// (the wait is requested with tile.z == 1), for all tiles of that row.
template<uint32_t TileM>
struct RowSync {
  uint32_t waitValue_;
  uint32_t postValue_;

  CUSYNC_DEVICE_HOST RowSync() : waitValue_(0), postValue_(0) {}
  // waitValue = number of producer tiles per row; each adds 1.
  RowSync(uint32_t waitValue) : waitValue_(waitValue), postValue_(1) {}
  RowSync(uint32_t waitValue, uint32_t postValue) : waitValue_(waitValue), postValue_(postValue) {}

  CUSYNC_DEVICE_HOST uint32_t waitValue(const dim3&, const dim3&) const { return waitValue_; }
  CUSYNC_DEVICE_HOST uint32_t postValue(const dim3&, const dim3&) const { return postValue_; }
  CUSYNC_DEVICE_HOST uint32_t tileIndex(const dim3& tile, const dim3&) const { return tile.x / TileM; }
  CUSYNC_DEVICE_HOST bool isSync(const dim3& tile, const dim3&) const { return tile.z == 1; }
  cusync_policy_desc desc() const {
    return detail::makePolicyDesc(CUSYNC_POLICY_ROWSYNC, CUSYNC_ORDER_TRANSPOSE_XY, TileM, 1, waitValue_, postValue_);
  }
};

// One semaphore per producer tile.  A wait is only needed when the column
// offset enters a new producer tile.
template<typename TileOrder, uint32_t TileM, uint32_t TileN>
struct TileSync {
  uint32_t waitValue_;
  uint32_t postValue_;

  CUSYNC_DEVICE_HOST TileSync() : waitValue_(1), postValue_(1) {}
  TileSync(uint32_t waitValue, uint32_t postValue) : waitValue_(waitValue), postValue_(postValue) {}

  CUSYNC_DEVICE_HOST uint32_t waitValue(const dim3&, const dim3&) const { return waitValue_; }
  CUSYNC_DEVICE_HOST uint32_t postValue(const dim3&, const dim3&) const { return postValue_; }
  CUSYNC_DEVICE_HOST uint32_t tileIndex(const dim3& tile, const dim3& grid) const {
    return TileOrder().tileIndex(dim3(tile.x / TileM, tile.y / TileN, 0), grid);
  }
  CUSYNC_DEVICE_HOST bool isSync(const dim3& tile, const dim3&) const { return tile.y % TileN == 0; }
  cusync_policy_desc desc() const {
    return detail::makePolicyDesc(CUSYNC_POLICY_TILESYNC, TileOrder::kOrderId, TileM, TileN, waitValue_, postValue_);
  }
};

// The producer's N extent holds `stride` groups of GridN columns (LLaMA: gate
// and up projections side by side); column tile ty of every group shares one
// semaphore, so the consumer proceeds when all `stride` groups have delivered it.
template<typename TileOrder, uint32_t GridN, uint32_t TileM, uint32_t TileN, uint32_t stride>
struct StridedSync {
  uint32_t waitValue_;
  uint32_t postValue_;

  CUSYNC_DEVICE_HOST StridedSync() : waitValue_(stride), postValue_(1) {}

  CUSYNC_DEVICE_HOST uint32_t waitValue(const dim3&, const dim3&) const { return stride; }
  CUSYNC_DEVICE_HOST uint32_t postValue(const dim3&, const dim3&) const { return 1; }
  CUSYNC_DEVICE_HOST uint32_t tileIndex(const dim3& tile, const dim3& grid) const {
    const uint32_t tilesPerGroup = GridN / TileN;
    uint32_t ty = tile.y / TileN;
    if (ty >= tilesPerGroup) ty -= tilesPerGroup;
    return TileOrder().tileIndex(dim3(tile.x / TileM, ty, 0), grid);
  }
  CUSYNC_DEVICE_HOST bool isSync(const dim3& tile, const dim3&) const { return tile.y % TileN == 0; }
  cusync_policy_desc desc() const {
    cusync_policy_desc d = detail::makePolicyDesc(CUSYNC_POLICY_STRIDEDSYNC, TileOrder::kOrderId, TileM, TileN, stride, 1);
    d.gridN = GridN; d.stride = stride;
    return d;
  }
};

// Consumer side of an implicit-GEMM convolution with an R x S filter fed by
// another convolution: the consumer's K extent is R*S*C, so K tile y maps to
// channel tile y/(R*S) of the producer, and only the first of each R*S run waits.
template<typename TileOrder, uint32_t R, uint32_t S, uint32_t TileM, uint32_t TileN>
struct Conv2DTileSync {
  uint32_t waitValue_;
  uint32_t postValue_;

  CUSYNC_DEVICE_HOST Conv2DTileSync() : waitValue_(1), postValue_(1) {}
  Conv2DTileSync(uint32_t waitValue, uint32_t postValue) : waitValue_(waitValue), postValue_(postValue) {}

  CUSYNC_DEVICE_HOST uint32_t waitValue(const dim3&, const dim3&) const { return waitValue_; }
  CUSYNC_DEVICE_HOST uint32_t postValue(const dim3&, const dim3&) const { return postValue_; }
  CUSYNC_DEVICE_HOST uint32_t tileIndex(const dim3& tile, const dim3& grid) const {
    return TileOrder().tileIndex(dim3(tile.x / TileM, (tile.y / TileN) / (R * S), 0), grid);
  }
  CUSYNC_DEVICE_HOST bool isSync(const dim3& tile, const dim3&) const { return (tile.y / TileN) % (R * S) == 0; }
  cusync_policy_desc desc() const {
    cusync_policy_desc d = detail::makePolicyDesc(CUSYNC_POLICY_CONV2DTILESYNC, TileOrder::kOrderId, TileM, TileN, waitValue_, postValue_);
    d.R = R; d.S = S;
    return d;
  }
};

// Groups the (H/8)/TileN consecutive column tiles of each of the Q, K and V
// projections under one semaphore per row of tiles; waited once before the
// main loop (tile.z == 1).
template<typename TileOrder, uint32_t H, uint32_t TileM, uint32_t TileN>
struct ConsecutiveSync {
  CUSYNC_DEVICE_HOST ConsecutiveSync() {}

  CUSYNC_DEVICE_HOST uint32_t waitValue(const dim3&, const dim3&) const { return (H / 8) / TileN; }
  CUSYNC_DEVICE_HOST uint32_t postValue(const dim3&, const dim3&) const { return 1; }
  CUSYNC_DEVICE_HOST uint32_t tileIndex(const dim3& tile, const dim3& grid) const {
    const uint32_t g = (H / 8) / TileN;
    return TileOrder().tileIndex(dim3(tile.x / TileM, (tile.y / TileN) / g, 0), dim3(grid.x / g, grid.y, grid.z));
  }
  CUSYNC_DEVICE_HOST bool isSync(const dim3& tile, const dim3&) const { return tile.z == 1; }
  cusync_policy_desc desc() const {
    cusync_policy_desc d = detail::makePolicyDesc(CUSYNC_POLICY_CONSECUTIVESYNC, TileOrder::kOrderId, TileM, TileN, (H / 8) / TileN, 1);
    d.H = H;
    return d;
  }
};

}  // namespace cusync
