"""GPU test of cusync_gemm_run_static_workspace, the GEMM entry point that allocates nothing: its split-K
workspace is an array the library holds in device memory.  Two calls in a row through the C ABI, the second on
a smaller problem, each compared bit for bit with cusync_gemm_run on a workspace of the caller's (same kernel,
slices added in index order, so the results must be identical), plus the refusal of a problem beyond the limit."""
import ctypes as C

import numpy as np
import pytest

import oracle as orc
from cusync_amd import _lib, api
from util import assert_close, empty_dev, normal_f16, to_dev, to_host, uniform_f16

pytestmark = pytest.mark.gpu

LIMIT = 32 << 20      # CUSYNC_GEMM_STATIC_WORKSPACE_BYTES


def both_ways(M, N, K, tile, split, seed):
    import torch
    L = _lib.load()
    a = uniform_f16((M, K), seed)
    b = normal_f16((K, N), seed + 1, std=0.05)
    da, db = to_dev(a), to_dev(b)
    outs = []
    for static in (False, True):
        dd = empty_dev((M, N), fill=float("nan"))
        st = api.Stage(api.gemm_grid(tile, M, N, split), (1, 1, 1), api.no_sync(), api.no_sync())
        args = api.gemm_args(st, M, N, K, da.data_ptr(), K, db.data_ptr(), N, dd.data_ptr(), N, tile, split_k=split,
                             epilogue=api.EPI.GELU)
        need = L.cusync_gemm_workspace_size(C.byref(args))
        ws = None
        if not static:
            ws = torch.zeros(max(16, need), dtype=torch.uint8, device="cuda")
            args.workspace = ws.data_ptr()
        torch.cuda.synchronize()
        run = L.cusync_gemm_run_static_workspace if static else L.cusync_gemm_run
        for _ in range(2):          # twice each: the second launch finds the counters as the first left them
            dd.fill_(float("nan"))
            torch.cuda.synchronize()
            assert run(C.byref(args), None) == api.ERR.SUCCESS, api.last_error()
            assert L.cusync_rt_device_sync() == 0, api.last_error()
        state = st.read_state()
        assert state.tile_counter == 0 and state.spin_timeouts == 0
        st.destroy()
        outs.append(to_host(dd))
    assert_close(outs[0], orc.gemm(a, b, orc.EPI_GELU), "existing entry point against the oracle")
    assert np.array_equal(outs[0].view(np.uint16), outs[1].view(np.uint16)), "static workspace changed the result"
    return need


def test_static_workspace_two_calls_second_smaller():
    print("no-alloc gemm: 200x392x1024, 4 slices, then 64x264x512, 2 slices", flush=True)
    need1 = both_ways(200, 392, 1024, api.TILE.T128x128x32, 4, 31)
    # smaller problem, other tile: its counters sit where the first call kept partial sums
    need2 = both_ways(64, 264, 512, api.TILE.D32x128x64, 2, 41)
    assert 0 < need2 < need1 <= LIMIT
    # and the first shape again after the smaller one
    both_ways(200, 392, 1024, api.TILE.T128x128x32, 4, 31)


def test_static_workspace_without_slices_and_beyond_limit():
    L = _lib.load()
    both_ways(130, 264, 256, api.TILE.T128x128x64, 1, 51)          # split_k == 1: no workspace at all
    # 2048 x 6144 with 256x192 tiles and 8 slices needs 8 * 8 * 32 * 256 * 192 * 4 bytes = 403 MB
    M, N, K, tile, split = 2048, 6144, 12288, api.TILE.T256x192x32, 8
    st = api.Stage(api.gemm_grid(tile, M, N, split), (1, 1, 1), api.no_sync(), api.no_sync())
    buf = empty_dev((16,))
    args = api.gemm_args(st, M, N, K, buf.data_ptr(), K, buf.data_ptr(), N, buf.data_ptr(), N, tile, split_k=split)
    assert L.cusync_gemm_workspace_size(C.byref(args)) > LIMIT
    assert L.cusync_gemm_run_static_workspace(C.byref(args), None) == api.ERR.NOT_INITIALIZED      # refused before any launch
    assert "workspace" in api.last_error()
    st.destroy()


def test_static_workspace_calls_leave_device_memory_as_it_is():
    """What the entry point is for: after one warm-up call on a device (which looks the kernel's occupancy and the
    array's address up) further calls neither allocate nor free device memory."""
    import torch
    L = _lib.load()
    M, N, K, tile, split = 200, 392, 1024, api.TILE.T128x128x32, 4
    da, db = to_dev(uniform_f16((M, K), 61)), to_dev(normal_f16((K, N), 62, std=0.05))
    dd = empty_dev((M, N), fill=float("nan"))
    st = api.Stage(api.gemm_grid(tile, M, N, split), (1, 1, 1), api.no_sync(), api.no_sync())
    args = api.gemm_args(st, M, N, K, da.data_ptr(), K, db.data_ptr(), N, dd.data_ptr(), N, tile, split_k=split)
    assert L.cusync_gemm_run_static_workspace(C.byref(args), None) == api.ERR.SUCCESS, api.last_error()      # warm-up
    assert L.cusync_rt_device_sync() == 0
    free_before, total = torch.cuda.mem_get_info()
    for _ in range(5):
        assert L.cusync_gemm_run_static_workspace(C.byref(args), None) == api.ERR.SUCCESS, api.last_error()
        assert torch.cuda.mem_get_info()[0] == free_before          # also while the launch is in flight
    assert L.cusync_rt_device_sync() == 0
    assert torch.cuda.mem_get_info() == (free_before, total)
    st.destroy()
