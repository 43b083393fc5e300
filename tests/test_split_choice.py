"""The k-slice rule of the GEMM launcher and of the chains (cusync_amd/csrc/split_choice.h), host code only.

The kernel gives slice z the K chunks [z * per, (z + 1) * per) with per = ceil(chunks / slices): a slice count is
usable only if the last slice still begins inside K.  The closed form the library uses is checked against that
definition by brute force, and the automatic choice against the cases the design was measured on."""
import os
import subprocess

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))

SRC = r"""
#include <cstdio>
#include "split_choice.h"
using namespace cusync::gemm;
int main() {
  // every (chunks, slices) pair of a small range: 1 if the library accepts it
  for (uint32_t chunks = 1; chunks <= 96; chunks++)
    for (uint32_t slices = 1; slices <= 40; slices++)
      std::printf("E %u %u %d\n", chunks, slices, everySliceHasAChunk(chunks * 64 - 8, 64, slices) ? 1 : 0);
  const uint32_t cases[][4] = {
    {48, 12288, 64, 256}, {96, 6144, 64, 256}, {32, 12288, 64, 256}, {64, 6144, 64, 256},     // GPT-3 shard, few rows
    {43, 8192, 64, 512}, {64, 2752, 64, 256}, {64, 2816, 64, 256},                               // LLaMA shard
    {64, 12288, 32, 256}, {128, 6144, 32, 256}, {256, 12288, 32, 256}, {512, 6144, 32, 256},    // 512 and 2048 rows on 256x192
    {1, 8256, 64, 256}, {1, 64, 64, 256}};
  for (auto& c : cases) std::printf("P %u %u %u %u %d\n", c[0], c[1], c[2], c[3], pickSplit(0, c[0], c[1], c[2], (int)c[3]));
  std::printf("R %d\n", pickSplit(7, 48, 12288, 64, 256));
  // shared reduction: (slices, requested, direct tile, all static, launched, tiles, tileM, AvoidWaitKernel)
  std::printf("S %d\n", slicesShareReduction(4, true, true, true, 256, 256, 256, false) ? 1 : 0);
  std::printf("S %d\n", slicesShareReduction(4, true, true, true, 256, 256, 256, true) ? 1 : 0);     // consumer may arrive first
  std::printf("S %d\n", slicesShareReduction(4, false, true, true, 256, 256, 256, false) ? 1 : 0);   // not asked for
  std::printf("S %d\n", slicesShareReduction(4, true, true, true, 200, 256, 256, false) ? 1 : 0);    // a second round
  std::printf("S %d\n", slicesShareReduction(4, true, true, true, 256, 256, 64, false) ? 1 : 0);     // few-row tile
  std::printf("S %d\n", slicesShareReduction(3, true, true, true, 192, 192, 256, false) ? 1 : 0);    // 8 pieces, 3 slices
  std::printf("S %d\n", slicesShareReduction(1, true, true, true, 256, 256, 256, false) ? 1 : 0);    // no slices
  std::printf("S %d\n", slicesShareReduction(2, true, false, true, 256, 256, 256, false) ? 1 : 0);   // register-staged tile
  std::printf("S %d\n", slicesShareReduction(2, true, true, false, 256, 256, 256, false) ? 1 : 0);   // tiles drawn from a dispenser
  return 0;
}
"""


def test_split_choice(tmp_path):
    src = tmp_path / "split_choice_test.cpp"
    src.write_text(SRC)
    exe = tmp_path / "split_choice_test"
    subprocess.check_call(["g++", "-std=c++17", "-Wall", "-I", os.path.join(ROOT, "cusync_amd", "csrc"), str(src), "-o", str(exe)])
    out = subprocess.check_output([str(exe)], text=True).split("\n")
    picks = {}
    shares = []
    for line in out:
        f = line.split()
        if not f:
            continue
        if f[0] == "E":
            chunks, slices, got = int(f[1]), int(f[2]), int(f[3])
            per = -(-chunks // slices)
            # the definition: every slice z < slices begins before the end of K (K = chunks * 64 - 8: a ragged last chunk)
            want = all(z * per * 64 < chunks * 64 - 8 for z in range(slices))
            assert got == int(want), (chunks, slices)
        elif f[0] == "P":
            picks[tuple(int(v) for v in f[1:5])] = int(f[5])
        elif f[0] == "S":
            shares.append(int(f[1]))
        elif f[0] == "R":
            assert int(f[1]) == 7                     # a requested count is passed through (and validated by the GEMM)
    # one workgroup per CU at most, and at least eight chunks per slice
    assert picks[(48, 12288, 64, 256)] == 4 and picks[(96, 6144, 64, 256)] == 2
    assert picks[(32, 12288, 64, 256)] == 8 and picks[(64, 6144, 64, 256)] == 4
    assert picks[(43, 8192, 64, 512)] == 4            # 344 workgroups would be a second round
    assert picks[(64, 2752, 64, 256)] == 4 and picks[(64, 2816, 64, 256)] == 4
    assert picks[(64, 12288, 32, 256)] == 4 and picks[(128, 6144, 32, 256)] == 2
    assert picks[(256, 12288, 32, 256)] == 1 and picks[(512, 6144, 32, 256)] == 1
    # 129 chunks: sixteen slices of nine would leave the last one empty, and the doubling stops at eight
    assert picks[(1, 8256, 64, 256)] == 8
    assert picks[(1, 64, 64, 256)] == 1
    # the slices of a tile wait for each other only where nothing can keep a sibling off the device: never for a stage
    # under AvoidWaitKernel, whose consumer may be dispatched ahead of its producer
    assert shares == [1, 0, 0, 0, 0, 0, 0, 0, 0]
