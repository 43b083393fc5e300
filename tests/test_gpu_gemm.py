"""GPU parity of the sync-aware fp16 GEMM (C ABI: cusync_gemm_run) against the
CPU oracle, including the chained two-GEMM configuration (M=256, N=K=1024,
TileSync, producer and consumer on two streams)."""
import ctypes as C

import numpy as np
import pytest

import oracle as orc
from cusync_amd import _lib, api
from util import assert_close, empty_dev, normal_f16, to_dev, to_host, uniform_f16

pytestmark = pytest.mark.gpu

ALL_TILES = list(range(api.TILE.COUNT))


def plain_stage(tile, M, N, split_k=1):
    return api.Stage(api.gemm_grid(tile, M, N, split_k), (1, 1, 1), api.no_sync(), api.no_sync())


def run_gemm(a, b, tile, epilogue=api.EPI.NONE, a_mode=0, K=None, max_workgroups=0, split_k=1, launches=1, shared_reduction=0):
    import torch
    L = _lib.load()
    M = a.shape[0]
    K = K if K is not None else a.shape[1]
    N = b.shape[1]
    da, db = to_dev(a), to_dev(b)
    dd = empty_dev((M, N), fill=float("nan"))
    torch.cuda.synchronize()
    st = plain_stage(tile, M, N, split_k)
    args = api.gemm_args(st, M, N, K, da.data_ptr(), a.shape[1], db.data_ptr(), N, dd.data_ptr(), N, tile,
                         epilogue=epilogue, a_mode=a_mode, max_workgroups=max_workgroups, split_k=split_k,
                         shared_reduction=shared_reduction)
    ws = None
    if split_k > 1:
        ws = torch.zeros(L.cusync_gemm_workspace_size(C.byref(args)), dtype=torch.uint8, device="cuda")   # zeroed once
        torch.cuda.synchronize()
        args.workspace = ws.data_ptr()
    for _ in range(launches):          # a second launch checks that the arrival counters re-armed themselves
        dd.fill_(float("nan"))
        torch.cuda.synchronize()
        rc = L.cusync_gemm_run(C.byref(args), None)
        assert rc == api.ERR.SUCCESS, api.last_error()
        assert L.cusync_rt_device_sync() == 0, api.last_error()
    state = st.read_state()
    assert state.tile_counter == 0       # dispenser re-armed
    assert state.spin_timeouts == 0      # no k-slice gave up waiting for its siblings
    st.destroy()
    return to_host(dd)


@pytest.mark.parametrize("tile", ALL_TILES)
def test_gemm_exact_on_integer_data(tile):
    # small integers: every product and partial sum is exact in fp32 and fits fp16,
    # so the result must be bit-identical and any indexing slip shows up exactly
    print("tile", tile, flush=True)
    rng = np.random.default_rng(tile)
    M, N, K = 300, 328, 192
    a = rng.integers(-2, 3, (M, K)).astype(np.float16)
    b = rng.integers(-2, 3, (K, N)).astype(np.float16)
    got = run_gemm(a, b, tile)
    want = (a.astype(np.int64) @ b.astype(np.int64)).astype(np.float16)
    assert np.array_equal(got, want)
    assert np.array_equal(got, orc.gemm(a, b))


@pytest.mark.parametrize("tile", ALL_TILES)
@pytest.mark.parametrize("shape", [(256, 1024, 1024), (1, 256, 512), (17, 136, 64), (513, 264, 1000)])
def test_gemm_matches_oracle(tile, shape):
    print("tile", tile, "shape", shape, flush=True)
    M, N, K = shape
    if tile in (api.TILE.T256x384x32, api.TILE.T256x192x64) and K % 64:
        pytest.skip("the tiles with the K loop in assembly take K 64 columns at a time (refused by cusync_gemm_can_implement, see test_gemm_can_implement_rejects)")
    a = uniform_f16((M, K), 1)
    b = normal_f16((K, N), 2, std=0.05)
    got = run_gemm(a, b, tile)
    assert_close(got, orc.gemm(a, b), "gemm tile %d %s" % (tile, shape))


@pytest.mark.parametrize("epilogue,orc_epi", [(api.EPI.GELU, orc.EPI_GELU), (api.EPI.RELU, orc.EPI_RELU)])
def test_gemm_epilogues(epilogue, orc_epi):
    a = uniform_f16((130, 512), 3)
    b = normal_f16((512, 256), 4, std=0.1)
    got = run_gemm(a, b, api.TILE.T128x128x64, epilogue=epilogue)
    assert_close(got, orc.gemm(a, b, orc_epi), "epilogue %d" % epilogue)


@pytest.mark.parametrize("tile", [api.TILE.T128x128x64, api.TILE.T256x128x64, api.TILE.T32x128x64])
def test_gemm_swiglu_a_operand(tile):
    # A[m,k] = silu(G[m,k]) * G[m,k+d];  d = 344*8 = 2752 is not a multiple of 128
    d, M, N = 2752, 70, 256
    gu = uniform_f16((M, 2 * d), 5) * np.float16(3)
    w = normal_f16((d, N), 6, std=0.05)
    got = run_gemm(gu, w, tile, a_mode=1, K=d)
    want = orc.gemm(orc.swiglu(gu, d), w)
    assert_close(got, want, "swiglu tile %d" % tile)


def test_gemm_persistent_launch_smaller_than_grid():
    # 4 x 11 = 44 tiles on 5 workgroups: every workgroup loops over several tickets
    a = uniform_f16((512, 256), 7)
    b = normal_f16((256, 1400), 8, std=0.05)
    got = run_gemm(a, b, api.TILE.T128x128x64, max_workgroups=5)
    assert_close(got, orc.gemm(a, b), "persistent")


@pytest.mark.parametrize("tile", [api.TILE.T256x192x32, api.TILE.T256x256x32, api.TILE.T256x128x32, api.TILE.T128x128x32,
                                  api.TILE.T128x192x32, api.TILE.T128x256x32, api.TILE.T128x192x32_ALONE, api.TILE.D64x192x64,
                                  api.TILE.T256x384x32, api.TILE.T256x192x64, api.TILE.D128x192x64])
@pytest.mark.parametrize("K", [24, 200, 1032])
def test_gemm_several_tiles_per_workgroup_direct_to_lds(tile, K):
    # 3 workgroups for 12 to 88 tiles with ragged edges: every workgroup goes from one tile's stores straight into
    # the next tile's loads, and the stores outside the matrix are issued all the same (with an offset the buffer
    # descriptor rejects).  K = 24 is a single, partly filled chunk (fewer chunks than pipeline stages), 200 a
    # few, 1032 many and a ragged last one.  Two launches, GeLU epilogue.
    if tile in (api.TILE.T256x384x32, api.TILE.T256x192x64):
        K = {24: 64, 200: 192, 1032: 1024}[K]        # these tiles take K 64 columns at a time: one slot of A, three, many
    print("several tiles per workgroup, tile", tile, "K", K, flush=True)
    M, N = 600, 1000
    a = uniform_f16((M, K), 41)
    b = normal_f16((K, N), 42, std=0.05)
    got = run_gemm(a, b, tile, epilogue=api.EPI.GELU, max_workgroups=3, launches=2)
    assert_close(got, orc.gemm(a, b, orc.EPI_GELU), "tile %d K %d" % (tile, K))
    # exact arithmetic: any chunk read before it arrived, or read from a stage the next tile's loads had
    # already overwritten, changes an integer sum
    rng = np.random.default_rng(tile * 100 + K)
    a = rng.integers(-2, 3, (M, K)).astype(np.float16)
    b = rng.integers(-2, 3, (K, N)).astype(np.float16)
    want = (a.astype(np.int64) @ b.astype(np.int64)).astype(np.float16)
    assert np.array_equal(run_gemm(a, b, tile, max_workgroups=3), want)


@pytest.mark.parametrize("tile", [api.TILE.T128x128x64, api.TILE.T32x128x64, api.TILE.T128x256x32, api.TILE.T256x256x32,
                                  api.TILE.T128x128x32, api.TILE.T256x384x32, api.TILE.T256x192x64, api.TILE.D128x192x64])
@pytest.mark.parametrize("split", [2, 3, 8])
def test_gemm_split_k(tile, split):
    print("split-k tile", tile, "slices", split, flush=True)
    if tile == api.TILE.T256x384x32 and split == 3:
        pytest.skip("32 chunks in three slices of eleven: the 256x384x32 tile takes whole pairs of chunks per slice")
    rng = np.random.default_rng(tile * 10 + split)
    M, N, K = 200, 392, 1024
    a = rng.integers(-2, 3, (M, K)).astype(np.float16)
    b = rng.integers(-2, 3, (K, N)).astype(np.float16)
    want = (a.astype(np.int64) @ b.astype(np.int64)).astype(np.float16)
    assert np.array_equal(run_gemm(a, b, tile, split_k=split, launches=2), want)
    # random data, GeLU applied after the slices are added
    a = uniform_f16((M, K), 21)
    b = normal_f16((K, N), 22, std=0.05)
    got = run_gemm(a, b, tile, split_k=split, epilogue=api.EPI.GELU)
    assert_close(got, orc.gemm(a, b, orc.EPI_GELU), "split-k %d tile %d" % (split, tile))


@pytest.mark.parametrize("tile,split", [(api.TILE.T256x192x32, 2), (api.TILE.T256x192x32, 4), (api.TILE.T256x192x32, 8),
                                        (api.TILE.T128x192x32_ALONE, 4), (api.TILE.D64x192x64, 2), (api.TILE.T256x256x32, 4),
                                        (api.TILE.T256x192x32, 3), (api.TILE.D32x128x64, 4), (api.TILE.T256x384x32, 2),
                                        (api.TILE.T256x384x32, 4), (api.TILE.T256x192x64, 2), (api.TILE.T256x192x64, 4),
                                        (api.TILE.D128x192x64, 2), (api.TILE.D128x192x64, 4)])      # as the 256-row MLP runs it
def test_gemm_split_k_with_the_reduction_shared_among_the_slices(tile, split):
    # every k-slice has a workgroup of its own, so the slices of a tile each add up and store a share of it (where
    # the tile has 128 rows or more and its 32-row pieces divide among them: not for 3 slices, not for the 64- and
    # 32-row tiles, which fall back to the last slice doing all of it).  Same sums in the same order: bit-identical to the unshared reduction, launch
    # after launch (the counters re-arm), ragged edges included.
    print("shared reduction tile", tile, "slices", split, flush=True)
    M, N, K = 300, 392, 2048
    a = uniform_f16((M, K), 31)
    b = normal_f16((K, N), 32, std=0.05)
    plain = run_gemm(a, b, tile, split_k=split, epilogue=api.EPI.GELU)
    shared = run_gemm(a, b, tile, split_k=split, epilogue=api.EPI.GELU, shared_reduction=1, launches=3)
    assert np.array_equal(plain.view(np.uint16), shared.view(np.uint16))
    assert_close(shared, orc.gemm(a, b, orc.EPI_GELU), "shared reduction, %d slices, tile %d" % (split, tile))


def test_gemm_split_k_is_deterministic():
    a = uniform_f16((64, 4096), 23)
    b = normal_f16((4096, 256), 24, std=0.05)
    first = run_gemm(a, b, api.TILE.T64x128x64, split_k=16)
    for _ in range(3):
        assert np.array_equal(run_gemm(a, b, api.TILE.T64x128x64, split_k=16).view(np.uint16), first.view(np.uint16))


def test_gemm_can_implement_rejects():
    L = _lib.load()
    st = plain_stage(api.TILE.T128x128x64, 64, 64)
    bad = api.gemm_args(st, 64, 64, 60, 16, 64, 16, 64, 16, 64, api.TILE.T128x128x64)   # K % 8 != 0
    assert L.cusync_gemm_can_implement(C.byref(bad)) == api.ERR.NOT_INITIALIZED and "multiples of 8" in api.last_error()
    bad = api.gemm_args(st, 64, 64, 64, 16, 64, 16, 64, 16, 64, api.TILE.T128x128x64, split_k=2)   # more slices than K chunks
    assert L.cusync_gemm_can_implement(C.byref(bad)) == api.ERR.NOT_INITIALIZED and "k-slices" in api.last_error()
    # 2816 / 64 = 44 chunks in 16 slices of three: the sixteenth would begin past the end of K
    st16 = plain_stage(api.TILE.T64x128x64, 64, 128, split_k=16)
    bad = api.gemm_args(st16, 64, 128, 2816, 16, 2816, 16, 128, 16, 128, api.TILE.T64x128x64, split_k=16)
    assert L.cusync_gemm_can_implement(C.byref(bad)) == api.ERR.NOT_INITIALIZED and "without a K chunk" in api.last_error()
    st16.destroy()
    bad = api.gemm_args(st, 64, 64, 64, 16, 64, 16, 64, 16, 64, api.TILE.T128x128x64, split_k=0)
    assert L.cusync_gemm_can_implement(C.byref(bad)) == api.ERR.NOT_INITIALIZED
    bad = api.gemm_args(st, 300, 64, 64, 16, 64, 16, 64, 16, 64, api.TILE.T128x128x64)   # grid mismatch
    assert L.cusync_gemm_can_implement(C.byref(bad)) == api.ERR.NOT_INITIALIZED and "grid" in api.last_error()
    st.destroy()
    # the 256x384x32 tile walks K 64 columns at a time, in every k-slice
    stw = plain_stage(api.TILE.T256x384x32, 64, 64)
    bad = api.gemm_args(stw, 64, 64, 96, 16, 96, 16, 64, 16, 64, api.TILE.T256x384x32)
    assert L.cusync_gemm_can_implement(C.byref(bad)) == api.ERR.NOT_INITIALIZED and "multiple of 64" in api.last_error()
    stw.destroy()
    stw = plain_stage(api.TILE.T256x384x32, 64, 64, split_k=3)
    ws = api.gemm_args(stw, 64, 64, 1024, 16, 1024, 16, 64, 16, 64, api.TILE.T256x384x32, split_k=3, workspace=16)   # 32 chunks in slices of 11
    assert L.cusync_gemm_can_implement(C.byref(ws)) == api.ERR.NOT_INITIALIZED and "multiple of 64" in api.last_error()
    stw.destroy()
    # NoAtomicAdd with a counting policy is refused (RowSync counts to gN)
    g = api.gemm_grid(api.TILE.T128x128x64, 256, 512)
    rs = api.row_sync(128, g[0])
    prod = api.Stage(g, (1, 1, 1), api.no_sync(), rs, opts=api.OPT.NO_ATOMIC_ADD)
    bad = api.gemm_args(prod, 256, 512, 64, 16, 64, 16, 512, 16, 512, api.TILE.T128x128x64)
    assert L.cusync_gemm_can_implement(C.byref(bad)) == api.ERR.NOT_INITIALIZED and "NoAtomicAdd" in api.last_error()
    prod.destroy()


def chained(M, N, K, tile1, tile2, policy_kind, iters=1, opts=0, max_wg=0, seed=10, split=(1, 1), ordered=False, c_offset=0, host_hold=False):
    """C = A*B on one stream, E = C*D on another, synchronised per `policy_kind`.  `ordered`: the wait kernel
    goes behind an event recorded on the producer's stream right before the producer's launch.  `c_offset`:
    C starts that many halfs into its allocation (a base that is 16-byte but not 128-byte aligned)."""
    import torch
    L = _lib.load()
    a = uniform_f16((M, K), seed)
    b = uniform_f16((K, N), seed + 1) * np.float16(0.05)
    d = uniform_f16((N, N), seed + 2) * np.float16(0.05)
    da, db, dd = to_dev(a), to_dev(b), to_dev(d)
    dc_store = empty_dev((M * N + c_offset,), fill=float("nan"))
    dc = dc_store[c_offset:].view(M, N)
    de = empty_dev((M, N), fill=float("nan"))
    torch.cuda.synchronize()
    tm, tn, _ = api.tile_shape(tile1)
    g1, g2 = api.gemm_grid(tile1, M, N, split[0]), api.gemm_grid(tile2, M, N, split[1])
    if policy_kind == "tile":
        pol = api.tile_sync(api.ORDER.TRANSPOSE_XY, tm, tn)
        opol = orc.policy(orc.TILESYNC, orc.ORDER_TRANSPOSE_XY, tm, tn)
    else:
        pol = api.row_sync(tm, g1[0])
        opol = orc.policy(orc.ROWSYNC, tileM=tm, waitValue=g1[0])
    prod = api.Stage(g1, (1, 1, 1), api.no_sync(), pol, opts=opts)
    cons = api.Stage(g2, (1, 1, 1), pol, api.no_sync(), opts=opts)
    assert api.set_producer_consumer_pair(prod, cons) == api.ERR.SUCCESS
    s1, s2 = C.c_void_p(), C.c_void_p()
    assert L.cusync_rt_stream_create(C.byref(s1)) == 0 and L.cusync_rt_stream_create(C.byref(s2)) == 0
    a1 = api.gemm_args(prod, M, N, K, da.data_ptr(), K, db.data_ptr(), N, dc.data_ptr(), N, tile1, split_k=split[0], max_workgroups=max_wg)
    a2 = api.gemm_args(cons, M, N, N, dc.data_ptr(), N, dd.data_ptr(), N, de.data_ptr(), N, tile2, split_k=split[1], max_workgroups=max_wg)
    ws = [torch.zeros(max(16, L.cusync_gemm_workspace_size(C.byref(x))), dtype=torch.uint8, device="cuda") for x in (a1, a2)]
    torch.cuda.synchronize()
    ev = C.c_void_p()
    assert L.cusync_rt_event_create(C.byref(ev)) == 0
    for _ in range(iters):
        dc_store.fill_(float("nan")); de.fill_(float("nan"))
        torch.cuda.synchronize()
        if ordered:
            assert L.cusync_rt_event_record(ev, s1) == 0
        assert api.gemm(prod, M, N, K, da.data_ptr(), K, db.data_ptr(), N, dc.data_ptr(), N, tile1, stream=s1,
                        max_workgroups=max_wg, split_k=split[0], workspace=ws[0].data_ptr()) == api.ERR.SUCCESS, api.last_error()
        if host_hold == "library":      # cusync_hold_back: the library picks the host-side hold or the wait kernel from the launch it just made
            assert L.cusync_hold_back(C.byref(prod.desc), s2) == api.ERR.SUCCESS, api.last_error()
        elif host_hold:      # the host waits until every producer workgroup has started, then launches the consumer
            assert L.cusync_wait_producer_started(C.byref(prod.desc), 0) == api.ERR.SUCCESS, api.last_error()
        else:
            assert prod.invokeWaitKernel(s2, after=ev if ordered else None) == api.ERR.SUCCESS
        assert api.gemm(cons, M, N, N, dc.data_ptr(), N, dd.data_ptr(), N, de.data_ptr(), N, tile2, stream=s2,
                        max_workgroups=max_wg, split_k=split[1], workspace=ws[1].data_ptr()) == api.ERR.SUCCESS, api.last_error()
        assert L.cusync_rt_device_sync() == 0, api.last_error()
        prod.incrementIter(); cons.incrementIter()
    ps, cs = prod.read_state(), cons.read_state()
    want_sems = orc.expected_sems_gemm(opol, g1, tm, tn, iters, opts)
    L.cusync_rt_stream_destroy(s1); L.cusync_rt_stream_destroy(s2); L.cusync_rt_event_destroy(ev)
    prod.destroy(); cons.destroy()
    return a, b, d, to_host(dc), to_host(de), ps, cs, want_sems


@pytest.mark.parametrize("policy_kind,opts", [("tile", 0), ("tile", api.OPT.NO_ATOMIC_ADD | api.OPT.REORDER_TILE_LOADS), ("row", 0)])
@pytest.mark.parametrize("tiles", [(api.TILE.T128x128x64, api.TILE.T128x128x64), (api.TILE.T32x128x64, api.TILE.T64x128x64),
                                   (api.TILE.T256x128x64, api.TILE.T128x128x64),
                                   (api.TILE.T256x192x32, api.TILE.T256x192x32),      # eight wavefronts, pipelined order
                                   (api.TILE.D32x128x64, api.TILE.D64x192x64),        # few-row direct-to-LDS tiles
                                   (api.TILE.D64x192x64, api.TILE.T128x192x32),
                                   (api.TILE.T256x192x32, api.TILE.T256x384x32),      # consumer with the K loop in assembly
                                   (api.TILE.T256x384x32, api.TILE.T256x192x32),
                                   (api.TILE.T256x192x64, api.TILE.T256x384x32),      # as the 2048-row MLP runs them
                                   (api.TILE.D128x192x64, api.TILE.D128x192x64), (api.TILE.D64x192x64, api.TILE.D128x192x64)])
def test_two_chained_gemms_config1(policy_kind, opts, tiles):
    # BASELINE config 1: M=256, N=K=1024, fp32 accumulate, inputs uniform from a seed
    print("chained", policy_kind, opts, tiles, flush=True)
    M, N, K = 256, 1024, 1024
    iters = 2
    a, b, d, c, e, ps, cs, want_sems = chained(M, N, K, tiles[0], tiles[1], policy_kind, iters=iters, opts=opts)
    c_ref = orc.gemm(a, b)
    assert_close(c, c_ref, "C")
    # E's reference multiplies the C the GPU produced (fp16), isolating the second GEMM
    assert_close(e, orc.gemm(c, d), "E")
    assert cs.spin_timeouts == 0
    assert np.array_equal(ps.sems, want_sems)                 # bit-exact semaphore end state
    assert ps.tile_counter == 0 and cs.tile_counter == 0 and ps.start_counter == 0
    assert ps.kernel_executed == iters


@pytest.mark.parametrize("policy_kind", ["row", "tile"])
@pytest.mark.parametrize("tile", [api.TILE.T256x192x32, api.TILE.T128x128x32])
def test_chained_direct_to_lds_gemms_with_few_workgroups(policy_kind, tile):
    # 24 to 72 tiles per GEMM on 5 workgroups each, K with a ragged last chunk: every workgroup works through
    # several tickets of the producer and of the consumer, and a producer workgroup's post follows all of its
    # tile's stores.
    print("chained, few workgroups", policy_kind, tile, flush=True)
    a, b, d, c, e, ps, cs, want_sems = chained(768, 1536, 520, tile, tile, policy_kind, iters=3, max_wg=5)
    assert_close(c, orc.gemm(a, b), "C")
    assert_close(e, orc.gemm(c, d), "E")
    assert cs.spin_timeouts == 0 and np.array_equal(ps.sems, want_sems) and ps.kernel_executed == 3
    assert ps.tile_counter == 0 and cs.tile_counter == 0 and ps.start_counter == 0


@pytest.mark.parametrize("policy_kind", ["row", "tile"])
@pytest.mark.parametrize("tile", [api.TILE.T128x192x32, api.TILE.D64x192x64])
def test_three_gemms_in_one_launch(policy_kind, tile):
    # cusync_gemm_chain_run: C = A*B, E = C*D, G = E*F in ONE launch, three stages paired as for separate launches
    # (the middle one waits and posts).  The GEMMs have 6 to 36 tiles each: the launch has as many workgroups as the
    # largest, and a workgroup without a tile of an earlier GEMM goes straight on to the next and waits there.
    import torch
    print("three GEMMs in one launch", policy_kind, tile, flush=True)
    L = _lib.load()
    M, K, N1, N2, N3 = 300, 520, 384, 1152, 192
    a = uniform_f16((M, K), 50)
    b = uniform_f16((K, N1), 51) * np.float16(0.05)
    d = uniform_f16((N1, N2), 52) * np.float16(0.05)
    f = uniform_f16((N2, N3), 53) * np.float16(0.05)
    da, db, dd, df = to_dev(a), to_dev(b), to_dev(d), to_dev(f)
    dc, de, dg = (empty_dev((M, n), fill=float("nan")) for n in (N1, N2, N3))
    torch.cuda.synchronize()
    tm, tn, _ = api.tile_shape(tile)
    grids = [api.gemm_grid(tile, M, n, 1) for n in (N1, N2, N3)]

    def policy(g):
        return api.tile_sync(api.ORDER.TRANSPOSE_XY, tm, tn) if policy_kind == "tile" else api.row_sync(tm, g[0])

    p1, p2 = policy(grids[0]), policy(grids[1])
    st = [api.Stage(grids[0], (1, 1, 1), api.no_sync(), p1), api.Stage(grids[1], (1, 1, 1), p1, p2),
          api.Stage(grids[2], (1, 1, 1), p2, api.no_sync())]
    assert api.set_producer_consumer_pair(st[0], st[1]) == api.ERR.SUCCESS
    assert api.set_producer_consumer_pair(st[1], st[2]) == api.ERR.SUCCESS
    args = (_lib.GemmArgs * 3)(
        api.gemm_args(st[0], M, N1, K, da.data_ptr(), K, db.data_ptr(), N1, dc.data_ptr(), N1, tile),
        api.gemm_args(st[1], M, N2, N1, dc.data_ptr(), N1, dd.data_ptr(), N2, de.data_ptr(), N2, tile, epilogue=api.EPI.RELU),
        api.gemm_args(st[2], M, N3, N2, de.data_ptr(), N2, df.data_ptr(), N3, dg.data_ptr(), N3, tile))
    for it in range(3):
        for t in (dc, de, dg):
            t.fill_(float("nan"))
        torch.cuda.synchronize()
        assert L.cusync_gemm_chain_run(args, 3, None) == api.ERR.SUCCESS, api.last_error()
        assert L.cusync_rt_device_sync() == 0, api.last_error()
        for s_ in st:
            s_.incrementIter()
        for k in range(3):                  # the descriptors are copied into the arguments: take the new iteration over
            args[k].stage = st[k].desc
    states = [s_.read_state() for s_ in st]
    c, e, g = to_host(dc), to_host(de), to_host(dg)
    for s_ in st:
        s_.destroy()
    assert all(s_.spin_timeouts == 0 for s_ in states)
    assert all(s_.tile_counter == 0 for s_ in states)
    assert_close(c, orc.gemm(a, b), "C")
    assert_close(e, orc.gemm(c, d, orc.EPI_RELU), "E")
    assert_close(g, orc.gemm(e, f), "G")


def test_chained_gemms_with_few_workgroups():
    # both launches hold fewer workgroups than tiles: tickets keep producer rows ahead of consumers
    a, b, d, c, e, ps, cs, want_sems = chained(512, 1024, 512, api.TILE.T128x128x64, api.TILE.T128x128x64,
                                               "tile", iters=3, max_wg=6)
    assert_close(c, orc.gemm(a, b), "C")
    assert_close(e, orc.gemm(c, d), "E")
    assert cs.spin_timeouts == 0 and np.array_equal(ps.sems, want_sems) and ps.kernel_executed == 3


@pytest.mark.parametrize("policy_kind", ["tile", "row"])
def test_chained_gemms_wait_kernel_behind_launch_event(policy_kind):
    # cusync_invoke_wait_kernel_after: same results and semaphore end state as the unordered wait kernel
    print("chained, ordered wait kernel", policy_kind, flush=True)
    M, N, K = 512, 1536, 1024
    tile = api.TILE.T256x192x32
    a, b, d, c, e, ps, cs, want_sems = chained(M, N, K, tile, tile, policy_kind, iters=3, ordered=True)
    assert_close(c, orc.gemm(a, b), "C")
    assert_close(e, orc.gemm(c, d), "E")
    assert cs.spin_timeouts == 0
    assert np.array_equal(ps.sems, want_sems)
    assert ps.tile_counter == 0 and cs.tile_counter == 0 and ps.start_counter == 0
    assert ps.kernel_executed == 3


@pytest.mark.parametrize("policy_kind,opts", [("tile", api.OPT.NO_ATOMIC_ADD), ("row", 0)])
@pytest.mark.parametrize("tiles", [(api.TILE.T64x128x64, api.TILE.T128x128x32), (api.TILE.D32x128x64, api.TILE.D32x128x64),
                                   (api.TILE.D64x192x64, api.TILE.T256x192x32)])
def test_chained_gemms_with_split_k(policy_kind, opts, tiles):
    # split-K on both sides: only the slice that completes a tile posts it, and a consumer slice waits
    # for the producer tiles of its own K range only (CC/gemm/kernel/cusyncgemm.h:374-398)
    a, b, d, c, e, ps, cs, want_sems = chained(256, 1024, 1024, tiles[0], tiles[1],
                                               policy_kind, iters=2, opts=opts, split=(4, 2))
    assert_close(c, orc.gemm(a, b), "C")
    assert_close(e, orc.gemm(c, d), "E")
    assert cs.spin_timeouts == 0
    assert np.array_equal(ps.sems, want_sems)      # entries of the k-slices beyond the first stay 0
    assert ps.tile_counter == 0 and cs.tile_counter == 0 and ps.kernel_executed == 2


@pytest.mark.parametrize("policy_kind", ["tile", "row"])
@pytest.mark.parametrize("tiles", [(api.TILE.T128x128x32, api.TILE.T128x128x32), (api.TILE.T128x128x64, api.TILE.T64x128x64)])
def test_chained_gemms_avoid_wait_kernel(policy_kind, tiles):
    # AvoidWaitKernel (CS/cusync.h:193-196, 205-206; cusync_device_defs.h:78-83): no flag is allocated, the
    # producer raises none, invokeWaitKernel launches nothing.  Valid because both launches (16 + 16 or
    # 16 + 32 workgroups) are resident together, so the producer cannot be kept off the device.
    print("chained, no wait kernel", policy_kind, tiles, flush=True)
    opts = api.OPT.AVOID_WAIT_KERNEL | (api.OPT.NO_ATOMIC_ADD if policy_kind == "tile" else 0)
    a, b, d, c, e, ps, cs, want_sems = chained(256, 1024, 1024, tiles[0], tiles[1], policy_kind, iters=3, opts=opts)
    assert_close(c, orc.gemm(a, b), "C")
    assert_close(e, orc.gemm(c, d), "E")
    assert cs.spin_timeouts == 0 and ps.spin_timeouts == 0
    assert np.array_equal(ps.sems, want_sems)
    assert ps.tile_counter == 0 and cs.tile_counter == 0 and ps.start_counter == 0
    assert ps.kernel_executed == 0                       # nobody raised a flag ...
    st = api.Stage(api.gemm_grid(tiles[0], 256, 1024), (1, 1, 1), api.no_sync(), api.tile_sync(api.ORDER.TRANSPOSE_XY, 128, 128),
                   opts=api.OPT.AVOID_WAIT_KERNEL)
    assert not st.desc.kernelExecuted                    # ... because there is none
    assert st.invokeWaitKernel(None) == api.ERR.SUCCESS  # and the call is a no-op
    st.destroy()


@pytest.mark.parametrize("policy_kind", ["tile", "row"])
@pytest.mark.parametrize("tiles,N,c_offset", [((api.TILE.T128x128x64, api.TILE.T128x128x64), 264, 0),     # pitch 528 bytes
                                              ((api.TILE.T64x128x64, api.TILE.T128x128x64), 1000, 8),    # pitch 2000, base + 16
                                              ((api.TILE.T128x128x64, api.TILE.T128x128x64), 1024, 8),   # aligned pitch, base + 16
                                              ((api.TILE.T128x128x32, api.TILE.T128x128x32), 264, 0)])
def test_chained_gemms_unaligned_intermediate(policy_kind, tiles, N, c_offset):
    # A producer tile of C is not a whole number of 128-byte lines here, so a line can hold columns of a posted
    # and of an unposted tile: every successful wait, the early poll included, has to end with the agent-scope
    # acquire.  C is refilled with NaN before every iteration.
    print("chained, unaligned C", policy_kind, tiles, N, c_offset, flush=True)
    a, b, d, c, e, ps, cs, want_sems = chained(300, N, 512, tiles[0], tiles[1], policy_kind, iters=3, c_offset=c_offset)
    assert_close(c, orc.gemm(a, b), "C")
    assert_close(e, orc.gemm(c, d), "E")
    assert cs.spin_timeouts == 0
    assert np.array_equal(ps.sems, want_sems)


@pytest.mark.parametrize("policy_kind", ["tile", "row"])
def test_chained_gemms_consumer_held_back_by_the_host(policy_kind):
    # cusync_wait_producer_started instead of a wait kernel: what the chain handles do when the producer's launch
    # takes every workgroup slot of the device (2 x 128 tiles of 256x192 here: one per CU)
    print("chained, host-side hold", policy_kind, flush=True)
    M, N, K = 2048, 6144, 256
    tile = api.TILE.T256x192x32
    L = _lib.load()
    a, b, d, c, e, ps, cs, want_sems = chained(M, N, K, tile, tile, policy_kind, iters=3, host_hold=True)
    rows = [0, 255, 256, 1000, 2047]
    assert_close(c[rows], orc.gemm(np.ascontiguousarray(a[rows]), b), "C rows")
    assert_close(e[rows], orc.gemm(np.ascontiguousarray(c[rows]), d), "E rows")
    assert cs.spin_timeouts == 0 and np.array_equal(ps.sems, want_sems) and ps.kernel_executed == 3
    # a stage whose producer never ran: the host-side wait gives up after its time-out, nothing hangs
    st = api.Stage((2, 2, 1), (1, 1, 1), api.no_sync(), api.tile_sync(api.ORDER.TRANSPOSE_XY, 128, 128))
    assert L.cusync_wait_producer_started(C.byref(st.desc), 50) == api.ERR.DEVICE and "did not all start" in api.last_error()
    st.destroy()


@pytest.mark.parametrize("shape", [(2048, 6144, 256, "fills"), (512, 768, 256, "leaves slots free")])
def test_chained_gemms_held_back_by_the_library(shape):
    # cusync_hold_back behind a producer launch that takes every workgroup slot (host-side hold) and behind one that
    # does not (wait kernel): what CuStage::invokeWaitKernel and the chain handles call
    M, N, K, what = shape
    print("chained, cusync_hold_back,", what, flush=True)
    tile = api.TILE.T256x192x64
    L = _lib.load()
    a, b, d, c, e, ps, cs, want_sems = chained(M, N, K, tile, tile, "row", iters=3, host_hold="library")
    rows = [0, 255, 256, M - 1]
    assert_close(c[rows], orc.gemm(np.ascontiguousarray(a[rows]), b), "C rows")
    assert_close(e[rows], orc.gemm(np.ascontiguousarray(c[rows]), d), "E rows")
    assert cs.spin_timeouts == 0 and np.array_equal(ps.sems, want_sems) and ps.kernel_executed == 3


def test_hold_back_error_paths():
    L = _lib.load()
    cons = api.Stage((2, 2, 1), (1, 1, 1), api.tile_sync(api.ORDER.TRANSPOSE_XY, 128, 128), api.no_sync())
    assert L.cusync_hold_back(C.byref(cons.desc), None) == api.ERR.NOT_PRODUCER
    cons.destroy()
    assert L.cusync_hold_back(None, None) == api.ERR.NOT_INITIALIZED
    # AvoidWaitKernel: nothing to hold back
    prod = api.Stage((2, 2, 1), (1, 1, 1), api.no_sync(), api.tile_sync(api.ORDER.TRANSPOSE_XY, 128, 128), opts=api.OPT.AVOID_WAIT_KERNEL)
    assert L.cusync_hold_back(C.byref(prod.desc), None) == api.ERR.SUCCESS
    prod.destroy()
    # a producer no launcher has run: no note of a launch that filled the device, so the wait kernel (which gives up
    # by itself and is counted)
    st = api.Stage((2, 2, 1), (1, 1, 1), api.no_sync(), api.tile_sync(api.ORDER.TRANSPOSE_XY, 128, 128))
    assert L.cusync_hold_back(C.byref(st.desc), None) == api.ERR.SUCCESS
    assert L.cusync_rt_device_sync() == 0, api.last_error()
    assert st.read_state().spin_timeouts == 1
    st.destroy()


def test_wait_kernel_that_gives_up_is_counted():
    # A wait kernel on a stage whose producer never runs: the bounded spin ends by itself (about a second) and
    # the give-up is counted where the chain handles look for it.
    import torch
    L = _lib.load()
    st = api.Stage((2, 2, 1), (1, 1, 1), api.no_sync(), api.tile_sync(api.ORDER.TRANSPOSE_XY, 128, 128))
    assert st.read_state().spin_timeouts == 0
    assert st.invokeWaitKernel(None) == api.ERR.SUCCESS
    assert L.cusync_rt_device_sync() == 0, api.last_error()
    assert st.read_state().spin_timeouts == 1
    st.destroy()
