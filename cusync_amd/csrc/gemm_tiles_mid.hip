// Instantiates part of the GEMM tile table (see gemm_tiles.h).
#include "gemm_tiles.h"
#include "gemm_kernel_dma.h"

namespace cusync {
namespace gemm {

void fillDmaTilesMid(TileInfo* t) {
  t[CUSYNC_TILE_256x128x32] = CUSYNC_TILE_DMA(256, 128, 32, 2, 2, 3, 2);   // 3 stages, two workgroups per CU
  t[CUSYNC_TILE_128x256x32] = CUSYNC_TILE_DMA(128, 256, 32, 2, 2, 3, 2);
  t[CUSYNC_TILE_128x128x32] = CUSYNC_TILE_DMA(128, 128, 32, 2, 2, 3, 3);   // three workgroups per CU
  t[CUSYNC_TILE_128x192x32] = CUSYNC_TILE_DMA(128, 192, 32, 2, 2, 3, 2);   // 6144 and 12288 columns are 32 and 64 tiles
  t[CUSYNC_TILE_128x192x32_ALONE] = CUSYNC_TILE_DMA(128, 192, 32, 2, 2, 4, 2, false, true);   // 80 KB of LDS, so one workgroup per CU
  t[CUSYNC_TILE_D128x192x64] = CUSYNC_TILE_DMA(128, 192, 64, 2, 2, 3, 1);   // 120 KB of LDS; A rows arrive as whole 128-byte lines
}

}  // namespace gemm
}  // namespace cusync
