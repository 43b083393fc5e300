"""CPU checks of the drop-in boundary: the library loads, exports every symbol the
C header declares, and its host-side policy arithmetic agrees with the oracle.
No GPU call is made here."""
import ctypes as C
import itertools
import os
import re

import numpy as np
import pytest

import oracle as orc
from cusync_amd import _lib, api

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def declared_symbols():
    text = open(os.path.join(ROOT, "include", "cusync_amd.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(cusync_[a-z0-9_]+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    L = _lib.load()
    names = declared_symbols()
    assert len(names) >= 40
    for n in names:
        assert hasattr(L, n), "libcusync_amd.so does not export " + n
    # and the ctypes table covers exactly the header
    assert sorted(_lib.SIGNATURES) == names


def test_error_and_option_values_match_reference_enum():
    assert (api.ERR.NOT_PRODUCER, api.ERR.NOT_CONSUMER, api.ERR.NOT_INITIALIZED,
            api.ERR.INVALID_LINEAR_BLOCK_INDEX, api.ERR.DEVICE, api.ERR.SUCCESS) == (0, 1, 2, 3, 4, 5)
    hdr = open(os.path.join(ROOT, "include", "cusync_amd.h")).read()
    assert "CUSYNC_SUCCESS = 5" in hdr and "CUSYNC_ERROR_NOT_PRODUCER = 0" in hdr


def _orc_policy(p):
    return orc.Policy(p.kind, p.order, p.tileM, p.tileN, p.waitValue, p.postValue, p.gridN, p.stride, p.R, p.S, p.H)


POLICIES = [
    api.row_sync(256, 24),
    api.tile_sync(api.ORDER.TRANSPOSE_XY, 256, 128),
    api.tile_sync(api.ORDER.IDENTITY, 32, 32),
    api.strided_sync(api.ORDER.TRANSPOSE_XY, 2816, 256, 128, 2),
    api.strided_sync(api.ORDER.TRANSPOSE_XY, 2752, 128, 64, 2),
    api.conv2d_tile_sync(api.ORDER.TRANSPOSE_XY, 3, 3, 64, 64),
    api.consecutive_sync(api.ORDER.TRANSPOSE_XY, 12288, 128, 128),
    api.no_sync(),
]


@pytest.mark.parametrize("p", POLICIES, ids=lambda p: "kind%d" % p.kind)
def test_host_policy_eval_matches_oracle(p):
    rng = np.random.default_rng(p.kind)
    grid = (48, 8, 1)
    op = _orc_policy(p)
    for _ in range(300):
        tile = (int(rng.integers(0, 8 * 256)), int(rng.integers(0, 48 * 128)), int(rng.integers(0, 2)))
        assert api.policy_tile_index(p, tile, grid) == orc.policy_tile_index(op, tile, grid)
        assert api.policy_is_sync(p, tile, grid) == orc.policy_is_sync(op, tile, grid)
    assert api.policy_wait_value(p) == orc.policy_wait_value(op, (0, 0, 0), grid)
    assert api.policy_post_value(p) == orc.policy_post_value(op, (0, 0, 0), grid)


def test_order_eval_matches_oracle():
    L = _lib.load()
    for order in (0, 1):
        for grid in [(3, 4, 2), (48, 8, 1)]:
            for b in itertools.product(range(grid[0]), range(min(grid[1], 3)), range(grid[2])):
                assert L.cusync_order_block_index(order, api.d3(grid), api.d3(b)) == orc.block_index(order, grid, b)
        assert L.cusync_order_tile_to_block(order, api.d3((3, 5, 7))).tup() == orc.tile_to_block(order, (3, 5, 7))


def test_gemm_grid_convention():
    # grid = (n-tiles, m-tiles, k-slices)
    assert api.gemm_grid(api.TILE.T256x128x64, 2048, 6144) == (48, 8, 1)
    assert api.gemm_grid(api.TILE.T256x128x64, 1, 12288) == (96, 1, 1)
    assert api.gemm_grid(api.TILE.T256x256x32, 1000, 5504) == (22, 4, 1)
    assert api.tile_shape(api.TILE.T256x64x64) == (256, 64, 64)
    with pytest.raises(ValueError):
        api.tile_shape(99)


def test_host_headers_compile_without_hipcc(tmp_path):
    """The C++ API's host half must build with a plain C++ compiler."""
    import subprocess
    src = tmp_path / "host_only.cpp"
    src.write_text(r'''
#include <cusync/cusync.h>
#include <cusync/wait-kernel.h>
#include <cusync/gemm.h>
using namespace cusync;
using Sync = TileSync<TransposeXYOrder, 256, 128>;
using Prod = CuStage<TransposeXYOrder, NoSync, Sync, NoAtomicAdd | ReorderTileLoads>;
using Cons = CuStage<TransposeXYOrder, Sync, NoSync>;
static_assert(std::is_trivially_copyable<Prod>::value, "stages are passed to kernels by value");
int main() {
  Sync s;
  if (s.tileIndex(dim3(256, 384, 0), dim3(48, 8, 1)) != 51) return 1;
  RowSync<256> r(24);
  if (r.waitValue(dim3(0,0,0), dim3(1,1,1)) != 24 || r.postValue(dim3(0,0,0), dim3(1,1,1)) != 1) return 2;
  StridedSync<TransposeXYOrder, 2816, 256, 128, 2> st;
  if (st.tileIndex(dim3(256, 30 * 128, 0), dim3(44, 4, 1)) != 8 + 44) return 3;
  if (CuSyncSuccess != 5 || CuSyncErrorNotProducer != 0) return 4;
  Cons* c = nullptr; (void)c;
  // the launcher objects are host code over the C ABI: they compile without hipcc, and the parts that need no GPU work
  typedef CuSyncGemm<Prod, CUSYNC_TILE_256x128x32, CUSYNC_EPILOGUE_GELU> Gemm1;
  const dim3 g = Gemm1::get_grid_shape(GemmCoord(2048, 6144, 12288), 2);
  if (g.x != 48 || g.y != 8 || g.z != 2) return 5;
  Gemm1::Arguments args;
  args.problem_size = GemmCoord(2048, 6144, 12288);
  args.split_k_slices = 2;
  if (Gemm1::get_workspace_size(args) != (size_t)2 * 8 * 48 * 256 * 128 * 4 + 2 * 8 * 48 * 4) return 6;      // partial sums, two counters per tile
  typedef CuSyncImplicitGemmConvolution<Cons, CUSYNC_CONV_TILE_128x64x32> Conv;
  const dim3 cg = Conv::get_grid_shape(Conv2dProblemSize(32, 56, 56, 64, 64));
  if (cg.x != 1 || cg.y != 32 * 56 * 56 / 128 || cg.z != 1) return 7;
  return 0;
}
''')
    exe = tmp_path / "host_only"
    subprocess.check_call(["g++", "-std=c++14", "-Wall", "-I", os.path.join(ROOT, "include"), str(src),
                           "-o", str(exe), "-L", _lib.LIB_DIR, "-lcusync_amd",
                           "-Wl,-rpath," + _lib.LIB_DIR, "-Wl,--allow-shlib-undefined"])
    assert subprocess.call([str(exe)]) == 0
