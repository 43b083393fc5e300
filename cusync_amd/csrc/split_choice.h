// Choice of the number of k-slices for a GEMM of a chain, shared by the chains that make it.
#pragma once

#include <stdint.h>
#include <algorithm>

namespace cusync {
namespace gemm {

// k-slices for a GEMM of `tiles` output tiles: double while the launch stays
// within one and a half workgroups per CU and every slice keeps at least eight
// K chunks.  Small batches are bound by streaming the weights, and without
// slices a 32-row problem occupies 48 workgroups on 256 CUs; beyond about 384
// workgroups the cost of adding the slices' partial sums outweighs the gain
// (measured: M=16, N=6144, K=12288 takes 121 / 49 / 52 / 72 us with 1 / 4 / 8 / 16 slices).
// Every slice takes ceil(chunks / slices) chunks of K, so a count that does not divide the chunks can leave the
// last slices without any (44 chunks in 16 slices: three each, and the sixteenth would begin past the end).
inline bool everySliceHasAChunk(uint32_t K, uint32_t bk, uint32_t slices) {
  const uint32_t chunks = (K + bk - 1) / bk;
  return slices >= 1 && slices <= chunks && (slices - 1) * ((chunks + slices - 1) / slices) < chunks;
}

inline int pickSplit(int requested, uint32_t tiles, uint32_t K, uint32_t bk, int resident) {
  if (requested > 0) return requested;
  const uint32_t target = (uint32_t)std::min(resident, 384);
  int s = 1;
  while (tiles * (uint32_t)s * 2 <= target && K / ((uint32_t)s * 2) >= 8 * bk && everySliceHasAChunk(K, bk, (uint32_t)s * 2)) s *= 2;
  return s;
}

}  // namespace gemm
}  // namespace cusync
