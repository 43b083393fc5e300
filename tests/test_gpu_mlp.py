"""GPU parity of the MLP chains (C ABI: cusync_mlp_*) against the CPU oracle:
GPT-3 175B 1/8 shard (X[B,12288] W1[12288,6144] GeLU W2[6144,12288]) and the
LLaMA 65B SwiGLU shard (d = 2752 and the reference's d = 2816), stream-ordered
and under RowSync / TileSync / StridedSync.  The oracle is evaluated on sampled
rows (each output row depends on one input row only); across sync modes the
outputs must be bit-identical because synchronisation only changes timing."""
import numpy as np
import pytest

import oracle as orc
from cusync_amd import api
from util import assert_close, empty_dev, normal_f16, sample_rows, to_dev, to_host, uniform_f16

pytestmark = pytest.mark.gpu

GPT3 = dict(hidden=12288, inner=6144)
_weights = {}


def weights(model, hidden, inner):
    key = (model, hidden, inner)
    if key not in _weights:
        n1 = inner if model == api.MODEL.GPT3 else 2 * inner
        w1 = normal_f16((hidden, n1), 2)       # seeds: X 1, W1 2, W2 3
        w2 = normal_f16((inner, hidden), 3)
        _weights[key] = (w1, w2, to_dev(w1), to_dev(w2))
    return _weights[key]


def run_mlp(model, batch, hidden, inner, sync, runs=2, activation=1, **kw):
    """`runs` passes through one handle.  Every pass starts from intermediates and outputs full of NaN, and the
    passes before the last one read another input: a consumer that read a tile before its post, or a line of
    the previous pass left in a cache, would show in the outputs of the last pass, which are the ones returned."""
    import torch
    w1, w2, dw1, dw2 = weights(model, hidden, inner)
    x = uniform_f16((batch, hidden), 1)
    dx, dx_other = to_dev(x), to_dev(uniform_f16((batch, hidden), 101))
    dh = empty_dev((batch, w1.shape[1]))
    dy = empty_dev((batch, hidden))
    torch.cuda.synchronize()
    mlp = api.Mlp(model, batch, hidden, inner, sync, dw1.data_ptr(), dw2.data_ptr(), activation=activation, **kw)
    times = []
    for r in range(runs):
        dh.fill_(float("nan")); dy.fill_(float("nan"))
        torch.cuda.synchronize()
        times += mlp.run((dx if r == runs - 1 else dx_other).data_ptr(), dh.data_ptr(), dy.data_ptr(), runs=1)
    prod, cons = mlp.stage_state(0), mlp.stage_state(1)
    tiles = mlp.tiles() + mlp.splits()
    mlp.destroy()
    return x, w1, w2, to_host(dh), to_host(dy), prod, cons, tiles, times


def check_against_oracle(model, x, w1, w2, h, y, inner, activation=1, fused=False):
    rows = sample_rows(x.shape[0])
    xs = np.ascontiguousarray(x[rows])
    if model == api.MODEL.GPT3:
        h_ref = orc.gemm(xs, w1, orc.EPI_GELU if activation else orc.EPI_NONE)
        assert_close(h[rows], h_ref, "H rows")
        a2 = np.ascontiguousarray(h[rows])
    elif fused:
        # silu(gate) * up is GEMM1's epilogue: the intermediate is [batch][inner], packed at the front of the buffer
        hh = h.reshape(-1)[:x.shape[0] * inner].reshape(x.shape[0], inner)
        assert_close(hh[rows], orc.gemm_swiglu(xs, w1, inner), "silu(gate)*up rows")
        a2 = np.ascontiguousarray(hh[rows])
    else:
        h_ref = orc.gemm(xs, w1)
        assert_close(h[rows], h_ref, "gate|up rows")
        a2 = orc.swiglu(np.ascontiguousarray(h[rows]), inner) if activation else np.ascontiguousarray(h[rows][:, :inner])
    # second GEMM is checked on the intermediate the GPU produced
    assert_close(y[rows], orc.gemm(a2, w2), "Y rows")


def expected_sems(prod, tiles, iters, fused=False):
    d = prod.desc
    p = orc.Policy(d.out.kind, d.out.order, d.out.tileM, d.out.tileN, d.out.waitValue, d.out.postValue,
                   d.out.gridN, d.out.stride, d.out.R, d.out.S, d.out.H)
    tm, tn, _ = api.tile_shape(tiles[0])
    if fused and d.out.kind == api.POLICY.STRIDEDSYNC:
        # the reference's grid has a gate tile and an up tile per column range, folded onto one semaphore that
        # counts to 2 per run (TB/mlp.cu:90-96); a tile of the SwiGLU epilogue is both
        want = np.zeros(prod.grid[0] * prod.grid[1] * prod.grid[2], np.uint32)
        want[:prod.grid[0] * prod.grid[1]] = 2 * iters
        return want
    return orc.expected_sems_gemm(p, prod.grid, tm, tn // 2 if fused else tn, iters, d.opts)


# 160, 320 and 1280 rows are not whole tiles: 160 is two tiles of 128 rows with the second one ragged, 320 two of 256,
# and at 1280 the producer's tiles have 256 rows and the consumer's 128
@pytest.mark.parametrize("batch", [1, 16, 64, 160, 256, 320, 512, 1280])
def test_gpt3_mlp_all_sync_modes(batch):
    print("gpt3 batch", batch, flush=True)
    outs = {}
    for sync in (api.SYNC.STREAM, api.SYNC.ROW, api.SYNC.TILE):
        x, w1, w2, h, y, prod, cons, tiles, _ = run_mlp(api.MODEL.GPT3, batch, sync=sync, runs=2, **GPT3)
        outs[sync] = (h, y)
        assert cons.spin_timeouts == 0
        assert prod.tile_counter == 0 and cons.tile_counter == 0 and prod.start_counter == 0
        if sync != api.SYNC.STREAM:
            assert np.array_equal(prod.sems, expected_sems(prod, tiles, 2))
            assert prod.kernel_executed == 2
        rc, want_order = orc.build_schedule(orc.ORDER_TRANSPOSE_XY, prod.grid)
        assert np.array_equal(prod.tile_order, want_order)
    check_against_oracle(api.MODEL.GPT3, x, w1, w2, *outs[api.SYNC.STREAM], inner=6144)
    for sync in (api.SYNC.ROW, api.SYNC.TILE):
        assert np.array_equal(outs[sync][0].view(np.uint16), outs[api.SYNC.STREAM][0].view(np.uint16))
        assert np.array_equal(outs[sync][1].view(np.uint16), outs[api.SYNC.STREAM][1].view(np.uint16))


@pytest.mark.parametrize("batch", [1024, 2048])
def test_gpt3_mlp_full_size(batch):
    print("gpt3 full batch", batch, flush=True)
    x, w1, w2, h0, y0, _, _, _, _ = run_mlp(api.MODEL.GPT3, batch, sync=api.SYNC.STREAM, runs=1, **GPT3)
    check_against_oracle(api.MODEL.GPT3, x, w1, w2, h0, y0, inner=6144)
    # size-independent property: rows are independent, so a permuted batch permutes the output
    for sync in (api.SYNC.ROW, api.SYNC.TILE):
        _, _, _, h, y, prod, cons, tiles, _ = run_mlp(api.MODEL.GPT3, batch, sync=sync, runs=3, **GPT3)
        assert cons.spin_timeouts == 0
        assert np.array_equal(h.view(np.uint16), h0.view(np.uint16))
        assert np.array_equal(y.view(np.uint16), y0.view(np.uint16))
        assert np.array_equal(prod.sems, expected_sems(prod, tiles, 3)) and prod.kernel_executed == 3


def test_gpt3_without_activation_matches_reference_check_build():
    # the reference's --check build has no GeLU (TB/mlp.cu:148-151)
    x, w1, w2, h, y, _, _, _, _ = run_mlp(api.MODEL.GPT3, 64, sync=api.SYNC.TILE, activation=0, **GPT3)
    check_against_oracle(api.MODEL.GPT3, x, w1, w2, h, y, inner=6144, activation=0)


@pytest.mark.parametrize("in_gemm2", [2, -1, 1])
@pytest.mark.parametrize("inner", [2752, 2816])
@pytest.mark.parametrize("batch", [1, 16, 64, 256, 512, 1024, 2048])
def test_llama_mlp(inner, batch, in_gemm2):
    # silu(gate) * up as GEMM1's epilogue (2, the built-in choice), as a stage of its own between the GEMMs (-1) or in
    # GEMM2's A loader (1)
    print("llama", inner, batch, in_gemm2, flush=True)
    fused = in_gemm2 == 2
    outs = {}
    # StridedSync constrains the tile width when gate|up is the intermediate (the split on a tile boundary); the other
    # modes are run with the same tiles and k-slices so that all execute the same kernels and must agree bit for bit
    same = {}
    modes = (api.SYNC.STRIDED, api.SYNC.STREAM, api.SYNC.ROW) + ((api.SYNC.TILE,) if fused else ())
    for sync in modes:
        x, w1, w2, h, y, prod, cons, tiles, _ = run_mlp(api.MODEL.LLAMA, batch, 8192, inner, sync, runs=2, swiglu_in_gemm2=in_gemm2, **same)
        same = dict(tile1=tiles[0], tile2=tiles[1], split_k1=tiles[2], split_k2=tiles[3])
        outs[sync] = (h, y)
        assert cons.spin_timeouts == 0
        if sync != api.SYNC.STREAM:
            assert np.array_equal(prod.sems, expected_sems(prod, tiles, 2, fused))
    check_against_oracle(api.MODEL.LLAMA, x, w1, w2, *outs[api.SYNC.STREAM], inner=inner, fused=fused)
    for sync in modes:
        assert np.array_equal(outs[sync][1].view(np.uint16), outs[api.SYNC.STREAM][1].view(np.uint16))


def test_llama_built_in_choice_is_the_fused_epilogue():
    # swiglu_in_gemm2 = 0: two kernels, the intermediate is silu(gate) * up
    x, w1, w2, h, y, prod, cons, tiles, _ = run_mlp(api.MODEL.LLAMA, 300, 8192, 2752, api.SYNC.STRIDED, runs=2)
    assert api.tile_shape(tiles[0])[2] in (32, 64) and cons.spin_timeouts == 0
    check_against_oracle(api.MODEL.LLAMA, x, w1, w2, h, y, inner=2752, fused=True)
    # against the unfused arithmetic on the caller's weights: round gate|up to fp16, then the activation
    rows = sample_rows(300)
    hh = h.reshape(-1)[:300 * 2752].reshape(300, 2752)
    assert_close(hh[rows], orc.swiglu(orc.gemm(np.ascontiguousarray(x[rows]), w1), 2752), "against swiglu(gemm)")


def test_llama_reference_wiring_no_activation():
    # the reference's timed path reads the gate half as is (TB/mlp.cu:785-792): TileSync suffices
    x, w1, w2, h, y, prod, cons, tiles, _ = run_mlp(api.MODEL.LLAMA, 128, 8192, 2816, api.SYNC.TILE, activation=0)
    assert cons.spin_timeouts == 0
    check_against_oracle(api.MODEL.LLAMA, x, w1, w2, h, y, inner=2816, activation=0)


def test_strided_sync_rejects_unaligned_split():
    import torch
    w = torch.zeros(16, device="cuda", dtype=torch.float16)
    with pytest.raises(RuntimeError, match="inner % tileN"):
        api.Mlp(api.MODEL.LLAMA, 256, 8192, 2752, api.SYNC.STRIDED, w.data_ptr(), w.data_ptr(),
                tile1=api.TILE.T256x128x64, swiglu_in_gemm2=-1)


@pytest.mark.parametrize("batch", [1, 16, 64, 256, 512, 1024, 2048])
@pytest.mark.parametrize("sync", [api.SYNC.ROW, api.SYNC.TILE])
def test_gpt3_mlp_in_one_launch(batch, sync):
    # both GEMMs in one launch: same stages and semaphores, results bit for bit those of the stream-ordered pair
    print("gpt3 one launch", batch, sync, flush=True)
    x, w1, w2, h, y, prod, cons, tiles, _ = run_mlp(api.MODEL.GPT3, batch, sync=sync, runs=3, one_launch=True, **GPT3)
    assert tiles[0] == tiles[1]            # one kernel for both
    # the same tiles and k-slices as two stream-ordered launches
    _, _, _, h0, y0, _, _, tiles0, _ = run_mlp(api.MODEL.GPT3, batch, sync=api.SYNC.STREAM, runs=1, tile1=tiles[0], tile2=tiles[1],
                                               split_k1=tiles[2], split_k2=tiles[3], **GPT3)
    assert tiles == tiles0
    assert cons.spin_timeouts == 0
    assert prod.tile_counter == 0 and cons.tile_counter == 0
    assert np.array_equal(prod.sems, expected_sems(prod, tiles, 3))
    assert np.array_equal(h.view(np.uint16), h0.view(np.uint16))
    assert np.array_equal(y.view(np.uint16), y0.view(np.uint16))


@pytest.mark.parametrize("batch", [1, 64, 512])
@pytest.mark.parametrize("sync", [api.SYNC.ROW, api.SYNC.STRIDED])
def test_llama_mlp_in_one_launch(batch, sync):
    # The two GEMMs of the LLaMA shard have different numbers of tiles (5504 and 8192 columns): the launch has as many
    # workgroups as the larger one, and a workgroup without a tile of GEMM1 goes straight on to GEMM2 and waits there.
    # Results bit for bit those of the stream-ordered pair with the same tiles and k-slices, and the oracle's.
    print("llama one launch", batch, sync, flush=True)
    x, w1, w2, h, y, prod, cons, tiles, _ = run_mlp(api.MODEL.LLAMA, batch, 8192, 2752, sync, runs=3, one_launch=True)
    assert tiles[0] == tiles[1]
    _, _, _, h0, y0, _, _, tiles0, _ = run_mlp(api.MODEL.LLAMA, batch, 8192, 2752, api.SYNC.STREAM, runs=1, tile1=tiles[0], tile2=tiles[1],
                                               split_k1=tiles[2], split_k2=tiles[3])
    assert tiles == tiles0
    assert cons.spin_timeouts == 0 and prod.spin_timeouts == 0
    assert prod.tile_counter == 0 and cons.tile_counter == 0
    assert np.array_equal(prod.sems, expected_sems(prod, tiles, 3, True))
    assert np.array_equal(h.view(np.uint16), h0.view(np.uint16))
    assert np.array_equal(y.view(np.uint16), y0.view(np.uint16))
    check_against_oracle(api.MODEL.LLAMA, x, w1, w2, h, y, inner=2752, fused=True)


def test_mlp_in_one_launch_rejects():
    w1, w2, dw1, dw2 = weights(api.MODEL.GPT3, 12288, 6144)
    with pytest.raises(RuntimeError):       # two different tiles cannot share a launch
        api.Mlp(api.MODEL.GPT3, 256, 12288, 6144, api.SYNC.ROW, dw1.data_ptr(), dw2.data_ptr(),
                tile1=api.TILE.T128x192x32, tile2=api.TILE.T128x128x32, one_launch=True)
    with pytest.raises(RuntimeError):       # the register-staged tiles have no chain kernel
        api.Mlp(api.MODEL.GPT3, 256, 12288, 6144, api.SYNC.ROW, dw1.data_ptr(), dw2.data_ptr(),
                tile1=api.TILE.T128x128x64, tile2=api.TILE.T128x128x64, one_launch=True)


@pytest.mark.parametrize("model,inner,batch,sync", [(api.MODEL.GPT3, 6144, 16, api.SYNC.STREAM), (api.MODEL.GPT3, 6144, 256, api.SYNC.ROW),
                                                    (api.MODEL.GPT3, 6144, 2048, api.SYNC.TILE), (api.MODEL.LLAMA, 2752, 64, api.SYNC.ROW),
                                                    (api.MODEL.LLAMA, 2752, 1024, api.SYNC.TILE)])
def test_mlp_with_repacked_weights(model, inner, batch, sync):
    # repack_weights: the GEMMs read padded copies of the weights; same arithmetic, so bit-identical outputs
    print("repacked weights", model, inner, batch, sync, flush=True)
    hidden = 12288 if model == api.MODEL.GPT3 else 8192
    x, w1, w2, h0, y0, _, _, tiles0, _ = run_mlp(model, batch, hidden, inner, sync)
    _, _, _, h1, y1, prod, cons, tiles1, _ = run_mlp(model, batch, hidden, inner, sync, repack_weights=True)
    assert tiles0 == tiles1
    # bit for bit (the LLaMA intermediate fills only the front of its buffer, the rest stays NaN)
    assert np.array_equal(h0.view(np.uint16), h1.view(np.uint16)) and np.array_equal(y0.view(np.uint16), y1.view(np.uint16))
    assert cons.spin_timeouts == 0
    check_against_oracle(model, x, w1, w2, h1, y1, inner, fused=model == api.MODEL.LLAMA)


def test_mlp_repacked_weights_reload():
    # the handle keeps its own copies: a change of the caller's weights shows only after reload_weights()
    import torch
    batch, hidden, inner = 32, GPT3["hidden"], GPT3["inner"]
    w1, w2, dw1, dw2 = weights(api.MODEL.GPT3, hidden, inner)
    mine1, mine2 = dw1.clone(), dw2.clone()
    x = uniform_f16((batch, hidden), 1)
    dx = to_dev(x)
    dh, dy = empty_dev((batch, inner)), empty_dev((batch, hidden))
    torch.cuda.synchronize()
    mlp = api.Mlp(api.MODEL.GPT3, batch, hidden, inner, api.SYNC.ROW, mine1.data_ptr(), mine2.data_ptr(), repack_weights=True)
    mlp.run(dx.data_ptr(), dh.data_ptr(), dy.data_ptr(), runs=1)
    y_first = to_host(dy)
    mine2.neg_()
    torch.cuda.synchronize()
    mlp.run(dx.data_ptr(), dh.data_ptr(), dy.data_ptr(), runs=1)
    assert np.array_equal(to_host(dy), y_first)
    assert mlp.reload_weights() == api.ERR.SUCCESS
    mlp.run(dx.data_ptr(), dh.data_ptr(), dy.data_ptr(), runs=1)
    y_reloaded = to_host(dy)
    # same arithmetic as a handle that reads the changed weights in place
    fresh = api.Mlp(api.MODEL.GPT3, batch, hidden, inner, api.SYNC.ROW, mine1.data_ptr(), mine2.data_ptr())
    fresh.run(dx.data_ptr(), dh.data_ptr(), dy.data_ptr(), runs=1)
    fresh.destroy()
    assert np.array_equal(y_reloaded, to_host(dy))
    assert not np.array_equal(y_reloaded, y_first)
    assert_close(y_reloaded, -y_first, "Y with W2 negated")
    assert mlp.stage_state(1).spin_timeouts == 0
    mlp.destroy()
    check_against_oracle(api.MODEL.GPT3, x, w1, w2, to_host(dh), y_first, inner)


def test_mlp_run_reports_waits_that_gave_up():
    # A consumer wait that runs out of polls lets its kernel go on with unposted data; the run call then
    # returns an error instead of success.  Forced from the host: the stage's give-up counter is bumped
    # by hand, exactly what a timed-out wait does, and no kernel is made to spin.
    import ctypes as C
    import torch
    from cusync_amd import _lib
    L = _lib.load()
    batch = 64
    w1, w2, dw1, dw2 = weights(api.MODEL.GPT3, **GPT3)
    dx = to_dev(uniform_f16((batch, GPT3["hidden"]), 1))
    dh, dy = empty_dev((batch, GPT3["inner"])), empty_dev((batch, GPT3["hidden"]))
    torch.cuda.synchronize()
    mlp = api.Mlp(api.MODEL.GPT3, batch, GPT3["hidden"], GPT3["inner"], api.SYNC.ROW, dw1.data_ptr(), dw2.data_ptr())
    mlp.run(dx.data_ptr(), dh.data_ptr(), dy.data_ptr(), runs=1)
    cons = L.cusync_mlp_stage(mlp.h, 1).contents
    C.c_uint32.from_address(cons.spinTimeouts).value = 3          # the counter lives in pinned host memory
    with pytest.raises(api.CuSyncError) as err:
        mlp.run(dx.data_ptr(), dh.data_ptr(), dy.data_ptr(), runs=1)
    assert err.value.code == api.ERR.DEVICE and "3 wait(s) gave up" in str(err.value)
    mlp.run(dx.data_ptr(), dh.data_ptr(), dy.data_ptr(), runs=1)       # the count did not move again: fine
    mlp.destroy()


@pytest.mark.parametrize("model,hidden,inner", [(api.MODEL.GPT3, 12288, 6144), (api.MODEL.LLAMA, 8192, 2752)])
def test_mlp_choice_is_what_the_handle_takes(model, hidden, inner):
    """cusync_mlp_choice (the tile table without a handle) against the tiles and k-slices of a handle made from the
    same configuration, for every benchmark batch size and sync mode; explicit tiles and slices pass through; the
    number of launches is the table's where the configuration leaves it open (one_launch = -1)."""
    import ctypes as C
    from cusync_amd import _lib
    L = _lib.load()
    _, _, dw1, dw2 = weights(model, hidden, inner)

    def choice(cfg):
        v = [C.c_int(-1) for _ in range(5)]
        assert L.cusync_mlp_choice(C.byref(cfg), *[C.byref(x) for x in v]) == 0, api.last_error()
        return tuple(x.value for x in v)

    for batch in (1, 16, 64, 256, 512, 1024, 1280, 2048):
        for sync in (api.SYNC.STREAM, api.SYNC.ROW, api.SYNC.TILE):
            for one in (-1, 0):
                m = api.Mlp(model, batch, hidden, inner, sync, dw1.data_ptr(), dw2.data_ptr(), one_launch=one)
                got = choice(m.cfg)
                assert m.choice() == got
                assert m.tiles() == got[:2] and m.splits() == got[2:4], (batch, sync)
                in_one = one == -1 and model == api.MODEL.GPT3 and sync != api.SYNC.STREAM and (batch <= 64 or 512 <= batch <= 1024)
                assert got[4] == int(in_one), (batch, sync, one, got)
                if in_one:
                    assert got[0] == got[1]
                m.destroy()
    cfg = _lib.MlpConfig(model, 512, hidden, inner, api.SYNC.ROW, api.TILE.T128x128x32, api.TILE.T128x256x32, -1, 1, 2, 1, 0, 0, -1, 0, 0)
    assert choice(cfg) == (api.TILE.T128x128x32, api.TILE.T128x256x32, 2, 1, 0)      # the caller's tiles: two launches
    cfg.one_launch = 1
    assert L.cusync_mlp_choice(C.byref(cfg), None, None, None, None, None) == 1 and "one launch" in api.last_error()
    empty = _lib.MlpConfig(model, 0, hidden, inner, api.SYNC.ROW, -1, -1, -1, 1, 0, 0, 0, 0, 0, 0, 0)
    assert L.cusync_mlp_choice(C.byref(empty), None, None, None, None, None) == 1 and "empty" in api.last_error()
