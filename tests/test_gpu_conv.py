"""GPU parity tests of the sync-aware NHWC convolution (cusync_conv2d_*) against the CPU
oracle: closed forms, the 1x1 case that reduces to a GEMM, ragged shapes, and the chained
convolution pair of the ResNet benchmark (src/ml-bench/volta_conv2d/resnet.cu:107-116,
626-631, 704-744) with TileSync -> Conv2DTileSync, TileSync -> TileSync and RowSync."""
import ctypes as C

import numpy as np
import pytest

import oracle as orc
from cusync_amd import _lib, api
from util import assert_close, empty_dev, to_dev, to_host, uniform_f16

pytestmark = pytest.mark.gpu

CONV_TILES = list(range(api.CONV_TILE.COUNT))


def fits(tile, Cc, R=3, S=3, pad=1, stride=1, W=8):
    """The halo tiles only do 3x3 / pad 1 / stride 1 with a power-of-two channel count of at least 64, and
    need their rows plus 2W + 2 pixels of the image in LDS next to the filter stages."""
    halo = {api.CONV_TILE.HALO_256x64x64: (256, 4 * 8192), api.CONV_TILE.HALO_128x128x64: (128, 3 * 16384),
            api.CONV_TILE.HALO_64x128x64: (64, 3 * 16384)}
    if tile not in halo:
        return True
    rows, filt = halo[tile]
    lds = filt + -(-(rows + 2 * W + 3) * Cc * 2 // 1024) * 1024      # the run of pixels and one pixel of zeros
    return (R, S, pad, stride) == (3, 3, 1, 1) and Cc >= 64 and Cc & (Cc - 1) == 0 and lds <= 159 * 1024


def he_filters(K, R, S, Cc, seed):
    rng = np.random.default_rng(seed)
    return (rng.standard_normal((K, R, S, Cc)) * np.sqrt(2.0 / (R * S * Cc))).astype(np.float16)


def run_conv(x, w, tile, pad=1, stride=1, epilogue=api.EPI.NONE, max_workgroups=0, launches=1, split_k=1):
    import torch
    L = _lib.load()
    N, H, W, Cc = x.shape
    K, R, S, _ = w.shape
    P, Q = (H + 2 * pad - R) // stride + 1, (W + 2 * pad - S) // stride + 1
    dx, dw = to_dev(x), to_dev(w)
    dy = empty_dev((N, P, Q, K), fill=float("nan"))
    ws = torch.zeros(max(16, api.conv2d_workspace_size(N, H, W, Cc, K, tile, split_k, R, S, pad, stride)), dtype=torch.uint8, device="cuda")
    torch.cuda.synchronize()
    st = api.Stage(api.conv2d_grid(tile, N, H, W, K, R, S, pad, stride, split_k), (1, 1, 1), api.no_sync(), api.no_sync())
    for _ in range(launches):
        dy.fill_(float("nan"))
        torch.cuda.synchronize()
        rc = api.conv2d(st, N, H, W, Cc, K, dx.data_ptr(), dw.data_ptr(), dy.data_ptr(), tile, R=R, S=S, pad=pad,
                        stride=stride, epilogue=epilogue, max_workgroups=max_workgroups, split_k=split_k,
                        workspace=ws.data_ptr() if split_k > 1 else None)
        assert rc == api.ERR.SUCCESS, api.last_error()
        assert L.cusync_rt_device_sync() == 0, api.last_error()
    assert st.read_state().tile_counter == 0
    st.destroy()
    return to_host(dy)


@pytest.mark.parametrize("tile", CONV_TILES)
def test_conv_all_ones_closed_form(tile):
    # all-ones image and 3x3 filter, pad 1: interior = 9C, edges = 6C, corners = 4C, exact in fp16
    print("conv ones", tile, flush=True)
    N, H, W, Cc, K = 3, 9, 11, 64, 72
    y = run_conv(np.ones((N, H, W, Cc), np.float16), np.ones((K, 3, 3, Cc), np.float16), tile).astype(np.float32)
    rows = np.minimum(np.arange(H) + 1, H - 1) - np.maximum(np.arange(H) - 1, 0) + 1
    cols = np.minimum(np.arange(W) + 1, W - 1) - np.maximum(np.arange(W) - 1, 0) + 1
    want = (rows[:, None] * cols[None, :] * Cc).astype(np.float32)
    assert y.shape == (N, H, W, K)
    assert np.array_equal(y, np.broadcast_to(want[None, :, :, None], y.shape))


@pytest.mark.parametrize("tile", CONV_TILES)
def test_conv_exact_on_integer_data(tile):
    # small integers: sums are exact, so a wrong pixel, channel or filter tap shows up bit-exactly
    print("conv int", tile, flush=True)
    rng = np.random.default_rng(tile)
    Cc = 96 if fits(tile, 96) else 128
    x = rng.integers(-2, 3, (2, 13, 10, Cc)).astype(np.float16)
    w = rng.integers(-2, 3, (40, 3, 3, Cc)).astype(np.float16)
    got = run_conv(x, w, tile, launches=2)
    want = orc.conv2d_nhwc(x, w)
    assert np.array_equal(got.view(np.uint16), want.view(np.uint16))


def test_conv_1x1_reduces_to_gemm():
    x = uniform_f16((2, 16, 16, 128), 3)
    w = he_filters(64, 1, 1, 128, 4)
    got = run_conv(x, w, api.CONV_TILE.T128x64x32, pad=0)
    want = orc.gemm(x.reshape(-1, 128), np.ascontiguousarray(w.reshape(64, 128).T))
    assert_close(got.reshape(-1, 64), want, "1x1")


@pytest.mark.parametrize("tile", CONV_TILES)
@pytest.mark.parametrize("geom", [(2, 12, 12, 64, 64, 3, 3, 1, 1), (3, 7, 9, 32, 72, 3, 3, 1, 1), (2, 5, 3, 128, 136, 3, 3, 1, 1),
                                  (1, 1, 1, 64, 8, 3, 3, 1, 1), (3, 30, 200, 64, 64, 3, 3, 1, 1), (1, 9, 7, 256, 72, 3, 3, 1, 1), (1, 15, 15, 64, 136, 5, 5, 2, 1),
                                  (2, 14, 14, 64, 64, 3, 3, 1, 2), (2, 9, 9, 96, 32, 3, 3, 0, 1), (1, 8, 20, 64, 64, 1, 3, 0, 1)])
def test_conv_matches_oracle(tile, geom):
    print("conv", tile, geom, flush=True)
    N, H, W, Cc, K, R, S, pad, stride = geom
    if not fits(tile, Cc, R, S, pad, stride, W):
        pytest.skip("geometry outside the halo tile's domain")
    x = uniform_f16((N, H, W, Cc), 5)
    w = he_filters(K, R, S, Cc, 6)
    got = run_conv(x, w, tile, pad=pad, stride=stride)
    assert_close(got, orc.conv2d_nhwc(x, w, pad, stride), "y")


HALO_TILES = [api.CONV_TILE.HALO_256x64x64, api.CONV_TILE.HALO_128x128x64, api.CONV_TILE.HALO_64x128x64]


@pytest.mark.parametrize("tile", HALO_TILES)
@pytest.mark.parametrize("geom,split", [((2, 12, 12, 64, 64), 2), ((2, 12, 12, 64, 64), 4),      # 9 steps in 4 runs: 3, 3, 3, 0
                                        ((2, 12, 12, 64, 64), 9), ((3, 7, 9, 128, 72), 3), ((4, 14, 14, 256, 256), 2),
                                        ((4, 14, 14, 256, 256), 4), ((1, 7, 7, 512, 136), 5), ((6, 7, 7, 512, 512), 2)])
def test_conv_steps_cut_into_runs(tile, geom, split):
    # the reference's --split_k_slices (resnet.cu:329, 689): partial sums of the runs put together, ReLU behind them,
    # two launches through one workspace (the counters are left at zero)
    print("conv in runs", tile, geom, split, flush=True)
    N, H, W, Cc, K = geom
    if not fits(tile, Cc, W=W):
        pytest.skip("geometry outside the halo tile's domain")
    x = uniform_f16((N, H, W, Cc), 15)
    w = he_filters(K, 3, 3, Cc, 16)
    got = run_conv(x, w, tile, epilogue=api.EPI.RELU, split_k=split, launches=2)
    assert_close(got, orc.conv2d_nhwc(x, w, epilogue=orc.EPI_RELU), "y")
    x = np.round(uniform_f16((N, H, W, Cc), 17) * 4).astype(np.float16)       # integers: every order of adding is exact
    w = np.round(he_filters(K, 3, 3, Cc, 18) * 16).astype(np.float16)
    assert np.array_equal(run_conv(x, w, tile, split_k=split), run_conv(x, w, tile))


def test_conv_relu_and_persistent_launch():
    x = uniform_f16((4, 20, 20, 64), 7)
    w = he_filters(64, 3, 3, 64, 8)
    got = run_conv(x, w, api.CONV_TILE.T128x64x32, epilogue=api.EPI.RELU, max_workgroups=3, launches=2)
    assert_close(got, orc.conv2d_nhwc(x, w, epilogue=orc.EPI_RELU), "relu")
    assert got.min() >= 0


def test_conv_can_implement_rejects():
    import torch
    L = _lib.load()
    buf = torch.zeros(1 << 20, dtype=torch.float16, device="cuda")
    tile = api.CONV_TILE.T128x64x32
    g = api.conv2d_grid(tile, 1, 8, 8, 64)
    st = api.Stage(g, (1, 1, 1), api.no_sync(), api.no_sync())

    def rc(**kw):
        base = dict(N=1, H=8, W=8, Cc=64, K=64, tile=tile)
        base.update(kw)
        a = api.conv2d_args(st, base.pop("N"), base.pop("H"), base.pop("W"), base.pop("Cc"), base.pop("K"),
                            buf.data_ptr(), buf.data_ptr(), buf.data_ptr(), base.pop("tile"), **base)
        return L.cusync_conv2d_can_implement(C.byref(a))

    assert rc() == api.ERR.SUCCESS
    assert rc(Cc=48) != api.ERR.SUCCESS               # channels not a multiple of the K chunk
    assert rc(K=60) != api.ERR.SUCCESS                # output channels not a multiple of 8
    assert rc(tile=99) != api.ERR.SUCCESS
    assert rc(H=40) != api.ERR.SUCCESS                # grid of the stage no longer matches
    assert rc(pad=3) != api.ERR.SUCCESS
    assert rc(stride=0) != api.ERR.SUCCESS
    assert rc(epilogue=7) != api.ERR.SUCCESS
    assert "conv2d" in api.last_error()
    # input 0.5 GiB, output 2 GiB (four times the channels): the output no longer fits one buffer descriptor
    assert rc(N=64, H=256, W=256, Cc=64, K=256) != api.ERR.SUCCESS and "2 GiB" in api.last_error()
    halo = api.CONV_TILE.HALO_256x64x64
    assert rc(tile=halo) == api.ERR.SUCCESS
    assert rc(tile=halo, stride=2) != api.ERR.SUCCESS and rc(tile=halo, pad=0) != api.ERR.SUCCESS
    assert rc(tile=halo, R=1, S=1, pad=0) != api.ERR.SUCCESS
    assert rc(tile=halo, Cc=96) != api.ERR.SUCCESS              # channels not a power of two
    assert rc(tile=halo, H=2, W=4096) != api.ERR.SUCCESS        # halo does not fit LDS (and the grid differs)
    st.destroy()
    # a tile's steps in runs: halo tiles only, a workspace, no more runs than steps, the stage's grid with the runs in z
    st2 = api.Stage(api.conv2d_grid(halo, 1, 8, 8, 64, split_k=2), (1, 1, 1), api.no_sync(), api.no_sync())
    st = st2
    assert rc(tile=halo, split_k=2, workspace=buf.data_ptr()) == api.ERR.SUCCESS
    assert rc(tile=halo, split_k=2) != api.ERR.SUCCESS and "workspace" in api.last_error()
    assert rc(tile=halo, split_k=3, workspace=buf.data_ptr()) != api.ERR.SUCCESS and "grid" in api.last_error()
    assert rc(tile=halo, split_k=10, workspace=buf.data_ptr()) != api.ERR.SUCCESS and "more runs than steps" in api.last_error()
    assert rc(tile=api.CONV_TILE.T128x64x32, split_k=2, workspace=buf.data_ptr()) != api.ERR.SUCCESS and "halo tile" in api.last_error()
    assert api.conv2d_workspace_size(1, 8, 8, 64, 64, halo, 2) == 2 * 256 * 64 * 4 + 2 * 4 and api.conv2d_workspace_size(1, 8, 8, 64, 64, halo, 1) == 0
    st2.destroy()


def chained_convs(N, H, W, Cc, tile1, tile2, kind, iters=1, opts=0, max_wg=(0, 0), seed=20):
    """y1 = relu(conv(x, w1)) on one stream, y2 = conv(y1, w2) on another (3x3, pad 1, C channels throughout)."""
    import torch
    L = _lib.load()
    x = uniform_f16((N, H, W, Cc), seed)
    w1, w2 = he_filters(Cc, 3, 3, Cc, seed + 1), he_filters(Cc, 3, 3, Cc, seed + 2)
    dx, dw1, dw2 = to_dev(x), to_dev(w1), to_dev(w2)
    dy1 = empty_dev((N, H, W, Cc), fill=float("nan"))
    dy2 = empty_dev((N, H, W, Cc), fill=float("nan"))
    torch.cuda.synchronize()
    tm, tn, _ = api.conv2d_tile_shape(tile1)
    g1, g2 = api.conv2d_grid(tile1, N, H, W, Cc), api.conv2d_grid(tile2, N, H, W, Cc)
    if kind == "row":
        out_pol = in_pol = api.row_sync(tm, g1[0])
        opol = orc.policy(orc.ROWSYNC, tileM=tm, waitValue=g1[0])
    else:
        out_pol = api.tile_sync(api.ORDER.TRANSPOSE_XY, tm, tn)
        opol = orc.policy(orc.TILESYNC, orc.ORDER_TRANSPOSE_XY, tm, tn)
        in_pol = api.conv2d_tile_sync(api.ORDER.TRANSPOSE_XY, 3, 3, tm, tn) if kind == "conv2dtile" else out_pol
    prod = api.Stage(g1, (1, 1, 1), api.no_sync(), out_pol, opts=opts)
    cons = api.Stage(g2, (1, 1, 1), in_pol, api.no_sync(), opts=opts)
    assert api.set_producer_consumer_pair(prod, cons) == api.ERR.SUCCESS
    s1, s2 = C.c_void_p(), C.c_void_p()
    assert L.cusync_rt_stream_create(C.byref(s1)) == 0 and L.cusync_rt_stream_create(C.byref(s2)) == 0
    for _ in range(iters):
        dy1.fill_(float("nan")); dy2.fill_(float("nan"))
        torch.cuda.synchronize()
        assert api.conv2d(prod, N, H, W, Cc, Cc, dx.data_ptr(), dw1.data_ptr(), dy1.data_ptr(), tile1, stream=s1,
                          epilogue=api.EPI.RELU, max_workgroups=max_wg[0]) == api.ERR.SUCCESS, api.last_error()
        assert prod.invokeWaitKernel(s2) == api.ERR.SUCCESS
        assert api.conv2d(cons, N, H, W, Cc, Cc, dy1.data_ptr(), dw2.data_ptr(), dy2.data_ptr(), tile2, stream=s2,
                          max_workgroups=max_wg[1]) == api.ERR.SUCCESS, api.last_error()
        assert L.cusync_rt_device_sync() == 0, api.last_error()
        prod.incrementIter(); cons.incrementIter()
    ps, cs = prod.read_state(), cons.read_state()
    want_sems = orc.expected_sems_gemm(opol, g1, tm, tn, iters, opts)
    L.cusync_rt_stream_destroy(s1); L.cusync_rt_stream_destroy(s2)
    prod.destroy(); cons.destroy()
    return x, w1, w2, to_host(dy1), to_host(dy2), ps, cs, want_sems


def check_chain(res, iters):
    x, w1, w2, y1, y2, ps, cs, want_sems = res
    assert_close(y1, orc.conv2d_nhwc(x, w1, epilogue=orc.EPI_RELU), "y1")
    # y2's reference convolves the y1 the GPU produced, isolating the second convolution; with the
    # same kernel on the same y1 a stream-ordered run gives the same bits, checked in the bitwise test below
    assert_close(y2, orc.conv2d_nhwc(y1, w2), "y2")
    assert cs.spin_timeouts == 0
    assert np.array_equal(ps.sems, want_sems)
    assert ps.tile_counter == 0 and cs.tile_counter == 0 and ps.start_counter == 0
    assert ps.kernel_executed == iters


@pytest.mark.parametrize("kind,opts", [("conv2dtile", 0), ("conv2dtile", api.OPT.NO_ATOMIC_ADD), ("tile", 0), ("row", 0)])
@pytest.mark.parametrize("tiles", [(api.CONV_TILE.T128x64x32, api.CONV_TILE.T128x64x32),
                                   (api.CONV_TILE.T256x64x32, api.CONV_TILE.T128x64x32),
                                   (api.CONV_TILE.HALO_256x64x64, api.CONV_TILE.HALO_256x64x64),
                                   (api.CONV_TILE.T128x64x32, api.CONV_TILE.HALO_128x128x64)])
def test_chained_conv_pair_small(kind, opts, tiles):
    print("conv chain", kind, opts, tiles, flush=True)
    check_chain(chained_convs(4, 20, 20, 64, tiles[0], tiles[1], kind, iters=2, opts=opts), 2)


@pytest.mark.parametrize("kind", ["conv2dtile", "row"])
def test_chained_conv_pair_two_channel_tiles(kind):
    # C = 128 with 64-wide producer tiles: a K chunk (r, s, c0..c0+31) must wait for channel tile c0/64,
    # not for (k/64)/(R*S) as the reference's Conv2DTileSync::tileIndex would give (policies.h:197-199)
    print("conv chain 2 channel tiles", kind, flush=True)
    check_chain(chained_convs(2, 14, 14, 128, api.CONV_TILE.T128x64x32, api.CONV_TILE.T128x64x32, kind, iters=2), 2)
    check_chain(chained_convs(2, 14, 14, 128, api.CONV_TILE.HALO_256x64x64, api.CONV_TILE.HALO_128x128x64, kind, iters=2), 2)


def test_chained_conv_pair_producer_trails():
    # one producer workgroup against many consumer workgroups: every halo wait really has to hold
    print("conv chain trailing producer", flush=True)
    check_chain(chained_convs(4, 20, 20, 64, api.CONV_TILE.T128x64x32, api.CONV_TILE.T128x64x32, "conv2dtile",
                              iters=2, max_wg=(1, 0)), 2)
    check_chain(chained_convs(4, 20, 20, 64, api.CONV_TILE.HALO_256x64x64, api.CONV_TILE.HALO_256x64x64, "conv2dtile",
                              iters=2, max_wg=(1, 0)), 2)


@pytest.mark.parametrize("shape,tile", [((32, 56, 56, 64), api.CONV_TILE.T128x64x32), ((32, 28, 28, 128), api.CONV_TILE.T128x128x32),
                                        ((32, 56, 56, 64), api.CONV_TILE.HALO_256x64x64), ((32, 28, 28, 128), api.CONV_TILE.HALO_128x128x64)])
@pytest.mark.parametrize("kind", ["conv2dtile", "row"])
def test_resnet_conv_pair_full_size(shape, tile, kind):
    # the two benchmark shapes of resnet_results.csv (batch 32): 56x56x64 and 28x28x128
    print("resnet pair", shape, kind, flush=True)
    res = chained_convs(*shape, tile, tile, kind, iters=1)
    check_chain(res, 1)
    # bitwise: the overlapped pair equals the same two kernels run back to back on one stream
    x, w1, w2, y1, y2 = res[:5]
    y1s = run_conv(x, w1, tile, epilogue=api.EPI.RELU)
    y2s = run_conv(y1s, w2, tile)
    assert np.array_equal(y1.view(np.uint16), y1s.view(np.uint16))
    assert np.array_equal(y2.view(np.uint16), y2s.view(np.uint16))


def run_chain(N, H, W, Cc, layers, sync, runs=2, seed=30, **kw):
    """`runs` passes through one handle; every pass starts from outputs full of NaN and the passes before the
    last read another image, so that a layer that read its input before the post shows in what is returned."""
    import torch
    x = uniform_f16((N, H, W, Cc), seed)
    ws = [he_filters(Cc, 3, 3, Cc, seed + 1 + i) for i in range(layers)]
    dx, dx_other = to_dev(x), to_dev(uniform_f16((N, H, W, Cc), seed + 100))
    dws = [to_dev(w) for w in ws]
    dys = [empty_dev((N, H, W, Cc)) for _ in range(layers)]
    torch.cuda.synchronize()
    chain = api.ConvChain(N, H, W, Cc, [w.data_ptr() for w in dws], sync, **kw)
    times = []
    for r in range(runs):
        for y in dys:
            y.fill_(float("nan"))
        torch.cuda.synchronize()
        times += chain.run((dx if r == runs - 1 else dx_other).data_ptr(), [y.data_ptr() for y in dys], runs=1)
    states = [chain.stage_state(i) for i in range(layers)]
    tile = chain.tile()
    run_chain.split = chain.split()
    chain.destroy()
    return x, ws, [to_host(y) for y in dys], states, tile, times


@pytest.mark.parametrize("shape,layers", [((4, 20, 20, 64), 2), ((32, 56, 56, 64), 2), ((32, 28, 28, 128), 2),
                                          ((2, 24, 24, 64), 4), ((8, 28, 28, 128), 4), ((16, 56, 56, 64), 4),
                                          # the deep layers of the ResNet table (resnet_results.csv, 256 and 512 channels):
                                          # few tiles, whose steps the chain cuts into runs by itself
                                          ((32, 14, 14, 256), 2), ((32, 7, 7, 512), 2), ((4, 14, 14, 256), 2), ((1, 7, 7, 512), 4)])
def test_conv_chain_all_sync_modes(shape, layers):
    # two layers: the ResNet block; four layers: the VGG block whose middle layers both wait and post
    print("conv chain", shape, layers, flush=True)
    outs = {}
    for sync in (api.SYNC.STREAM, api.SYNC.ROW, api.SYNC.TILE):
        x, ws, ys, states, tile, _ = run_chain(*shape, layers, sync, runs=2)
        outs[sync] = ys
        if shape[3] >= 256:
            assert run_chain.split > 1 and tile in HALO_TILES, (tile, run_chain.split)
        elif shape[0] == 32:      # the benchmark's pairs have tiles for every CU
            assert run_chain.split == 1
        tm, tn, _ = api.conv2d_tile_shape(tile)
        for i, st in enumerate(states):
            assert st.spin_timeouts == 0 and st.tile_counter == 0 and st.start_counter == 0
            if sync != api.SYNC.STREAM and i + 1 < layers:
                d = st.desc
                p = orc.Policy(d.out.kind, d.out.order, d.out.tileM, d.out.tileN, d.out.waitValue, d.out.postValue,
                               d.out.gridN, d.out.stride, d.out.R, d.out.S, d.out.H)
                assert np.array_equal(st.sems, orc.expected_sems_gemm(p, st.grid, tm, tn, 2, d.opts))
                assert st.kernel_executed == 2
    ys = outs[api.SYNC.STREAM]
    src = x
    for i in range(layers):      # each layer is checked on the input the GPU produced for it
        assert_close(ys[i], orc.conv2d_nhwc(src, ws[i], epilogue=orc.EPI_RELU if i + 1 < layers else orc.EPI_NONE), "y%d" % i)
        src = ys[i]
    for sync in (api.SYNC.ROW, api.SYNC.TILE):
        for i in range(layers):
            assert np.array_equal(outs[sync][i].view(np.uint16), ys[i].view(np.uint16)), (sync, i)


@pytest.mark.parametrize("shape,layers", [((4, 20, 20, 64), 2), ((32, 56, 56, 64), 2), ((32, 28, 28, 128), 2),
                                          ((2, 24, 24, 64), 4), ((16, 56, 56, 64), 4), ((8, 28, 28, 128), 8)])
@pytest.mark.parametrize("sync", [api.SYNC.ROW, api.SYNC.TILE])
def test_conv_chain_in_one_launch(shape, layers, sync):
    # all layers in one launch: same semaphores, same results bit for bit as the stream-ordered chain
    print("conv chain, one launch", shape, layers, sync, flush=True)
    x, ws, want, _, _, _ = run_chain(*shape, layers, api.SYNC.STREAM, runs=1, split_k=1)      # one launch never cuts a tile's steps
    _, _, got, states, tile, _ = run_chain(*shape, layers, sync, runs=3, fused=True)
    tm, tn, _ = api.conv2d_tile_shape(tile)
    for i, st in enumerate(states):
        assert st.spin_timeouts == 0 and st.tile_counter == 0 and st.start_counter == 0
        if i + 1 < layers:
            d = st.desc
            p = orc.Policy(d.out.kind, d.out.order, d.out.tileM, d.out.tileN, d.out.waitValue, d.out.postValue,
                           d.out.gridN, d.out.stride, d.out.R, d.out.S, d.out.H)
            assert np.array_equal(st.sems, orc.expected_sems_gemm(p, st.grid, tm, tn, 3, d.opts))
    for i in range(layers):
        assert np.array_equal(got[i].view(np.uint16), want[i].view(np.uint16)), i


def test_conv_chain_in_one_launch_rejects():
    import torch
    w = [to_dev(he_filters(64, 3, 3, 64, 1)) for _ in range(2)]
    torch.cuda.synchronize()
    with pytest.raises(RuntimeError):      # the implicit-GEMM tiles have no chain kernel
        api.ConvChain(4, 20, 20, 64, [t.data_ptr() for t in w], api.SYNC.ROW, tile=api.CONV_TILE.T256x64x32, fused=True)
    # runs of a tile's steps: not in one launch for all layers, not on the implicit-GEMM tiles, no more than steps
    for kw, what in ((dict(fused=True, split_k=2), "one launch per layer"), (dict(tile=api.CONV_TILE.T256x64x32, split_k=2), "halo tile"),
                     (dict(split_k=10), "more runs")):
        with pytest.raises(RuntimeError, match=what):
            api.ConvChain(4, 20, 20, 64, [t.data_ptr() for t in w], api.SYNC.ROW, **kw)
