// Tile processing orders.
//
// A tile order answers two questions: (1) in which position of the schedule
// does a workgroup (block) of the grid run — blockIndex(), used once on the
// host to build the ticket -> tile table — and (2) which block of the producer
// grid computed a given logical tile — tileToBlock(), used on the device to find
// the semaphore of that tile.  Same concept and class names as
// src/include/cusync/tile-orders.h:19-76 of the reference.
//
// Orders are stateless; a policy default-constructs one where it needs it.
#pragma once

#include "cusync_defines.h"
#include "../cusync_amd.h"
#include <stdint.h>

namespace cusync {

template<typename Derived>
struct GenericTileOrder {
  // Linear schedule position of `block` within `grid`.
  CUSYNC_DEVICE_HOST uint32_t blockIndex(const dim3& grid, const dim3& block) const {
    (void)grid; (void)block;
    return 0;
  }
  // Block that owns logical tile `tile`.
  CUSYNC_DEVICE_HOST dim3 tileToBlock(const dim3& tile) const {
    (void)tile;
    return dim3(0, 0, 0);
  }
  // Linear index of a logical tile: position of the block that owns it.
  CUSYNC_DEVICE_HOST uint32_t tileIndex(const dim3& tile, const dim3& grid) const {
    const Derived d{};
    return d.blockIndex(grid, d.tileToBlock(tile));
  }
  // CUSYNC_ORDER_* id understood by the prebuilt kernels, -1 for a user order.
  static constexpr int kOrderId = -1;
};

namespace detail {
CUSYNC_DEVICE_HOST uint32_t rowMajorBlockIndex(const dim3& grid, const dim3& block) {
  return block.x + grid.x * (block.y + grid.y * block.z);
}
}  // namespace detail

// Tiles are named (row-tile, column-tile) while the grid is laid out
// (column-tiles, row-tiles): the block of tile {x,y,z} is {y,x,z}.
struct TransposeXYOrder : public GenericTileOrder<TransposeXYOrder> {
  CUSYNC_DEVICE_HOST uint32_t blockIndex(const dim3& grid, const dim3& block) const {
    return detail::rowMajorBlockIndex(grid, block);
  }
  CUSYNC_DEVICE_HOST dim3 tileToBlock(const dim3& tile) const { return dim3(tile.y, tile.x, tile.z); }
  static constexpr int kOrderId = CUSYNC_ORDER_TRANSPOSE_XY;
};

// Tile {x,y,z} is block {x,y,z}.
struct IdentityOrder : public GenericTileOrder<IdentityOrder> {
  CUSYNC_DEVICE_HOST uint32_t blockIndex(const dim3& grid, const dim3& block) const {
    return detail::rowMajorBlockIndex(grid, block);
  }
  CUSYNC_DEVICE_HOST dim3 tileToBlock(const dim3& tile) const { return dim3(tile.x, tile.y, tile.z); }
  static constexpr int kOrderId = CUSYNC_ORDER_IDENTITY;
};

}  // namespace cusync
