// Instantiates part of the GEMM tile table (see gemm_tiles.h).
#include "gemm_tiles.h"
#include "gemm_kernel_dma.h"

namespace cusync {
namespace gemm {

void fillDmaTilesXWide(TileInfo* t) {
  // eight wavefronts of 128x96 (192 accumulator registers per lane), 3 stages of 40 KB, alternating order
  t[CUSYNC_TILE_256x384x32] = CUSYNC_TILE_DMA(256, 384, 32, 2, 4, 3, 2, false, false, true);
  // eight wavefronts of 64x96, K in slots of 64 columns (two of A, three of B)
  t[CUSYNC_TILE_256x192x64] = CUSYNC_TILE_DMA(256, 192, 64, 4, 2, 2, 2, false, false, true);
}

}  // namespace gemm
}  // namespace cusync
