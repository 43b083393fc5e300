// Instantiates part of the GEMM tile table (see gemm_tiles.h).
#include "gemm_tiles.h"
#include "gemm_kernel_dma.h"

namespace cusync {
namespace gemm {

void fillDmaTilesWide(TileInfo* t) {
  // eight wavefronts of 128x64: an A fragment costs one LDS read, a B fragment two transposing ones, so the tall
  // wavefront tile is the cheaper one (measured against 64x128: 641 -> 630 us per B=2048 step)
  t[CUSYNC_TILE_256x256x32] = CUSYNC_TILE_DMA(256, 256, 32, 2, 4, 4, 2, false, true);   // 4 stages, one workgroup per CU
  t[CUSYNC_TILE_256x192x32] = CUSYNC_TILE_DMA(256, 192, 32, 4, 2, 4, 2, false, true);   // eight wavefronts of 64x96
}

}  // namespace gemm
}  // namespace cusync
