// Table of the GEMM tile shapes the library is built with.  The kernels are instantiated in several
// translation units (gemm_tiles_*.hip) so that they compile side by side; each unit fills in its entries.
#pragma once

#include "gemm_common.h"

namespace cusync {
namespace gemm {

constexpr int kMaxChainedGemms = 4;
struct GemmChainParams {
  GemmParams gemm[kMaxChainedGemms];
  uint32_t count;
};

struct TileInfo {
  uint32_t bm, bn, bk;
  uint32_t threads;
  size_t lds;
  void (*kernel[2])(GemmParams);   // [plain A, SwiGLU A]
  int residentPerCU;     // filled lazily
  void (*chainKernel)(GemmChainParams);   // several dependent GEMMs in one launch; direct-to-LDS tiles only
  // kernel[0] compiled without the per-chunk waits of the tile policies, for stages that wait for whole rows or
  // for nothing (the few-row direct-to-LDS tiles only, see CUSYNC_TILE_DMA_FEW)
  void (*kernelNoChunkWaits)(GemmParams);
};

void fillStagedTiles(TileInfo* tiles);     // register-staged tiles (the only ones with a SwiGLU A operand)
void fillDmaTilesWide(TileInfo* tiles);    // direct-to-LDS, 256 rows, eight wavefronts
void fillDmaTilesMid(TileInfo* tiles);     // direct-to-LDS, 128 to 256 rows, four wavefronts
void fillDmaTilesFew(TileInfo* tiles);     // direct-to-LDS, 32 and 64 rows
void fillDmaTilesXWide(TileInfo* tiles);   // direct-to-LDS, 256x384, eight wavefronts in two alternating groups

// Entry of a register-staged tile.
#define CUSYNC_TILE(BM, BN, BK, WM, WN) \
  TileInfo{ BM, BN, BK, kThreads, (size_t)TileCfg<BM, BN, BK, WM, WN>::LDS_BYTES, \
    { gemmKernel<TileCfg<BM, BN, BK, WM, WN>, false>, gemmKernel<TileCfg<BM, BN, BK, WM, WN>, true> }, -1, nullptr, nullptr }

// Entry of a direct-to-LDS tile: no SwiGLU variant (that operand needs arithmetic on its way into LDS).
#define CUSYNC_TILE_DMA(...) \
  TileInfo{ DmaCfg<__VA_ARGS__>::BM, DmaCfg<__VA_ARGS__>::BN, DmaCfg<__VA_ARGS__>::BK, DmaCfg<__VA_ARGS__>::THREADS, \
    (size_t)DmaCfg<__VA_ARGS__>::LDS_BYTES, { gemmDmaKernel<DmaCfg<__VA_ARGS__>>, nullptr }, -1, gemmDmaChainKernel<DmaCfg<__VA_ARGS__>>, nullptr }

// Entry of a few-row direct-to-LDS tile: also the kernel compiled without the per-chunk waits.  A launch of these
// tiles is short (40 us), and the wait code a kernel carries without running it (stream order, RowSync) costs it
// 1.5-2 us: 84.1 -> 82.4 us for the stream-ordered 1-row MLP, 85.5 -> 83.6 at 16 rows.  For the big tiles the two
// kernels measure the same (2048 rows: 594 us either way), so those are built once.
#define CUSYNC_TILE_DMA_FEW(...) \
  TileInfo{ DmaCfg<__VA_ARGS__>::BM, DmaCfg<__VA_ARGS__>::BN, DmaCfg<__VA_ARGS__>::BK, DmaCfg<__VA_ARGS__>::THREADS, \
    (size_t)DmaCfg<__VA_ARGS__>::LDS_BYTES, { gemmDmaKernel<DmaCfg<__VA_ARGS__>>, nullptr }, -1, gemmDmaChainKernel<DmaCfg<__VA_ARGS__>>, \
    gemmDmaKernel<DmaCfg<__VA_ARGS__>, kAPlain, false> }

}  // namespace gemm
}  // namespace cusync
