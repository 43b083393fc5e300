// Instantiates part of the GEMM tile table (see gemm_tiles.h).
#include "gemm_tiles.h"
#include "gemm_kernel_dma.h"

namespace cusync {
namespace gemm {

void fillDmaTilesFew(TileInfo* t) {
  t[CUSYNC_TILE_D32x128x64] = CUSYNC_TILE_DMA_FEW(32, 128, 64, 1, 4, 4, 2);     // 60 KB of loads in flight per workgroup
  t[CUSYNC_TILE_D64x128x64] = CUSYNC_TILE_DMA_FEW(64, 128, 64, 1, 4, 3, 2);
  t[CUSYNC_TILE_D64x192x64] = CUSYNC_TILE_DMA_FEW(64, 192, 64, 2, 2, 4, 1);     // 96 KB of loads in flight per CU
}

}  // namespace gemm
}  // namespace cusync
