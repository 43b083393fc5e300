// Choice of the number of k-slices for a GEMM of a chain, shared by the chains that make it.
#pragma once

#include <stdint.h>
#include <algorithm>

namespace cusync {
namespace gemm {

// k-slices for a GEMM of `tiles` output tiles: double while the launch stays
// within one workgroup per CU (256 of them) and every slice keeps at least eight
// K chunks.  Small batches are bound by streaming the weights, and without
// slices a 32-row problem occupies 48 workgroups on 256 CUs; a launch of more
// than one round of workgroups pays more for adding the slices' partial sums than
// the extra loads in flight gain (M=16, N=6144, K=12288 on 32x128 tiles, 48 of them: 51 / 36 / 41 / 46 us
// with 2 / 4 / 8 / 16 slices; M=64, N=5504, K=8192 on 64x128 tiles, 43 of them: 34 / 29 / 34 / 41 us).
// Every slice takes ceil(chunks / slices) chunks of K, so a count that does not divide the chunks can leave the
// last slices without any (44 chunks in 16 slices: three each, and the sixteenth would begin past the end).
inline bool everySliceHasAChunk(uint32_t K, uint32_t bk, uint32_t slices) {
  const uint32_t chunks = (K + bk - 1) / bk;
  return slices >= 1 && slices <= chunks && (slices - 1) * ((chunks + slices - 1) / slices) < chunks;
}

inline int pickSplit(int requested, uint32_t tiles, uint32_t K, uint32_t bk, int resident) {
  if (requested > 0) return requested;
  const uint32_t target = (uint32_t)std::min(resident, 256);
  int s = 1;
  while (tiles * (uint32_t)s * 2 <= target && K / ((uint32_t)s * 2) >= 8 * bk && everySliceHasAChunk(K, bk, (uint32_t)s * 2)) s *= 2;
  return s;
}

// Whether the k-slices of a tile add it up together (each waits for its siblings, then sums and stores a share of
// the tile) instead of leaving all of it to the slice that arrives last.  The waiting slices hold their CUs, so
// every slice of the launch must have a workgroup of its own from the start (one round, all of them dealt a
// static first tile) and nothing may keep a sibling off the device: under AvoidWaitKernel the consumer's launch
// can reach the device before its producer's and take the slots the siblings need, the resident slices would
// spin until their bound runs out, so there the last-arriver form is kept, whose workgroups retire and free
// their slots.  Tiles of 128 rows and more whose 32-row pieces divide among the slices only.
inline bool slicesShareReduction(int splitK, bool requested, bool directToLdsTile, bool everyTileStatic, uint32_t launched,
                                 uint32_t tiles, uint32_t tileM, bool avoidWaitKernel) {
  return splitK > 1 && requested && directToLdsTile && everyTileStatic && launched == tiles && tileM >= 128 &&
         (tileM / 32) % (uint32_t)splitK == 0 && !avoidWaitKernel;
}

}  // namespace gemm
}  // namespace cusync
