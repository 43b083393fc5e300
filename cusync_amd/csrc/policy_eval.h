// Run-time evaluation of tile orders and sync policies described by
// cusync_policy_desc.  One definition serves the host entry points
// (cusync_policy_*) and the prebuilt kernels, so both always agree.
// Arithmetic follows the policy classes in include/cusync/policies.h, which in
// turn follow the reference (src/include/cusync/policies.h:18-210,
// src/ml-bench/transformer/mlp.cu:76-101, attention.cu:51-70).
#pragma once

#include <stdint.h>
#include "../../include/cusync_amd.h"

#if defined(__HIPCC__)
#define CUSYNC_HD __host__ __device__ __forceinline__
#else
#define CUSYNC_HD inline
#endif

namespace cusync {
namespace dyn {

CUSYNC_HD uint32_t blockIndex(int order, const cusync_dim3& grid, const cusync_dim3& block) {
  (void)order;  // both built-in orders linearise x fastest, then y, then z
  return block.x + grid.x * (block.y + grid.y * block.z);
}

CUSYNC_HD cusync_dim3 tileToBlock(int order, const cusync_dim3& tile) {
  cusync_dim3 b;
  if (order == CUSYNC_ORDER_TRANSPOSE_XY) { b.x = tile.y; b.y = tile.x; b.z = tile.z; }
  else { b = tile; }
  return b;
}

CUSYNC_HD uint32_t orderTileIndex(int order, uint32_t tx, uint32_t ty, const cusync_dim3& grid) {
  cusync_dim3 t = {tx, ty, 0};
  return blockIndex(order, grid, tileToBlock(order, t));
}

CUSYNC_HD uint32_t waitValue(const cusync_policy_desc& p) {
  switch (p.kind) {
    case CUSYNC_POLICY_ROWSYNC:
    case CUSYNC_POLICY_TILESYNC:
    case CUSYNC_POLICY_CONV2DTILESYNC:  return p.waitValue;
    case CUSYNC_POLICY_STRIDEDSYNC:     return p.stride;
    case CUSYNC_POLICY_CONSECUTIVESYNC: return (p.H / 8) / p.tileN;
    default:                            return 0;
  }
}

CUSYNC_HD uint32_t postValue(const cusync_policy_desc& p) {
  switch (p.kind) {
    case CUSYNC_POLICY_ROWSYNC:
    case CUSYNC_POLICY_TILESYNC:
    case CUSYNC_POLICY_CONV2DTILESYNC:  return p.postValue;
    case CUSYNC_POLICY_STRIDEDSYNC:
    case CUSYNC_POLICY_CONSECUTIVESYNC: return 1;
    default:                            return 0;
  }
}

CUSYNC_HD uint32_t tileIndex(const cusync_policy_desc& p, const cusync_dim3& tile, const cusync_dim3& grid) {
  switch (p.kind) {
    case CUSYNC_POLICY_ROWSYNC:
      return tile.x / p.tileM;
    case CUSYNC_POLICY_TILESYNC:
      return orderTileIndex(p.order, tile.x / p.tileM, tile.y / p.tileN, grid);
    case CUSYNC_POLICY_CONV2DTILESYNC:
      return orderTileIndex(p.order, tile.x / p.tileM, (tile.y / p.tileN) / (p.R * p.S), grid);
    case CUSYNC_POLICY_STRIDEDSYNC: {
      const uint32_t perGroup = p.gridN / p.tileN;
      uint32_t ty = tile.y / p.tileN;
      if (ty >= perGroup) ty -= perGroup;
      return orderTileIndex(p.order, tile.x / p.tileM, ty, grid);
    }
    case CUSYNC_POLICY_CONSECUTIVESYNC: {
      const uint32_t g = (p.H / 8) / p.tileN;
      cusync_dim3 gg = {grid.x / g, grid.y, grid.z};
      return orderTileIndex(p.order, tile.x / p.tileM, (tile.y / p.tileN) / g, gg);
    }
    default:
      return 0;
  }
}

CUSYNC_HD bool isSync(const cusync_policy_desc& p, const cusync_dim3& tile) {
  switch (p.kind) {
    case CUSYNC_POLICY_ROWSYNC:
    case CUSYNC_POLICY_CONSECUTIVESYNC: return tile.z == 1;
    case CUSYNC_POLICY_TILESYNC:
    case CUSYNC_POLICY_STRIDEDSYNC:     return tile.y % p.tileN == 0;
    case CUSYNC_POLICY_CONV2DTILESYNC:  return (tile.y / p.tileN) % (p.R * p.S) == 0;
    default:                            return false;
  }
}

}  // namespace dyn
}  // namespace cusync
