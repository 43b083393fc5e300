// Instantiates part of the GEMM tile table (see gemm_tiles.h).
#include "gemm_tiles.h"
#include "gemm_kernel_staged.h"

namespace cusync {
namespace gemm {

void fillStagedTiles(TileInfo* t) {
  t[CUSYNC_TILE_256x128x64] = CUSYNC_TILE(256, 128, 64, 2, 2);
  t[CUSYNC_TILE_128x128x64] = CUSYNC_TILE(128, 128, 64, 2, 2);
  t[CUSYNC_TILE_64x128x64] = CUSYNC_TILE(64, 128, 64, 1, 4);
  t[CUSYNC_TILE_32x128x64] = CUSYNC_TILE(32, 128, 64, 1, 4);
  t[CUSYNC_TILE_128x256x64] = CUSYNC_TILE(128, 256, 64, 2, 2);
  t[CUSYNC_TILE_256x64x64] = CUSYNC_TILE(256, 64, 64, 4, 1);
  t[CUSYNC_TILE_128x64x64] = CUSYNC_TILE(128, 64, 64, 2, 2);
}

}  // namespace gemm
}  // namespace cusync
