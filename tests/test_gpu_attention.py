"""GPU parity of the fused attention stage (cusync_attention_*) and of the self-attention chain
X Wqkv -> softmax(mask(Q K^T / sqrt(128))) V -> O Wo (cusync_attn_layer_*) against the CPU oracle,
stream-ordered and under RowSync / TileSync / ConsecutiveSync (the wiring of
src/ml-bench/transformer/attention.cu:84-110).  Shapes of the benchmark: 12 heads x 128 per GPU,
hidden 12288, sequence 256..2048."""
import ctypes as C

import numpy as np
import pytest

import oracle as orc
from cusync_amd import _lib, api
from util import assert_close, empty_dev, normal_f16, sample_rows, to_dev, to_host, uniform_f16

pytestmark = pytest.mark.gpu


def run_attention(qkv, heads, causal=True, max_workgroups=0, launches=1):
    import torch
    L = _lib.load()
    S = qkv.shape[0]
    dq = to_dev(qkv)
    do = empty_dev((S, heads * 128), fill=float("nan"))
    torch.cuda.synchronize()
    st = api.Stage(api.attention_grid(S, heads), (1, 1, 1), api.no_sync(), api.no_sync())
    for _ in range(launches):
        do.fill_(float("nan"))
        torch.cuda.synchronize()
        rc = api.attention(st, S, heads, dq.data_ptr(), qkv.shape[1], do.data_ptr(), heads * 128, causal=causal,
                           max_workgroups=max_workgroups)
        assert rc == api.ERR.SUCCESS, api.last_error()
        assert L.cusync_rt_device_sync() == 0, api.last_error()
    assert st.read_state().tile_counter == 0
    st.destroy()
    return to_host(do)


@pytest.mark.parametrize("causal", [True, False])
@pytest.mark.parametrize("S,heads", [(1, 1), (64, 1), (100, 2), (128, 1), (129, 1), (200, 3), (256, 12), (448, 2), (1000, 1)])
def test_attention_matches_oracle(S, heads, causal):
    print("attention", S, heads, causal, flush=True)
    qkv = normal_f16((S, 3 * heads * 128), 11, std=1.0)
    got = run_attention(qkv, heads, causal)
    assert_close(got, orc.attention(qkv, heads, 128, causal), "O")


def test_attention_closed_forms():
    S, heads = 300, 2
    E = heads * 128
    rng = np.random.default_rng(5)
    qkv = normal_f16((S, 3 * E), 12, std=1.0)
    # Q = 0: every visible key weighs the same, row i of O is the mean of V rows 0..i
    qkv[:, :E] = 0
    v = rng.integers(-4, 5, (S, E)).astype(np.float16)
    qkv[:, 2 * E:] = v
    got = run_attention(qkv, heads, True).astype(np.float32)
    want = np.cumsum(v.astype(np.float64), axis=0) / np.arange(1, S + 1)[:, None]
    assert np.array_equal(got[0], v[0].astype(np.float32))          # first row sees only itself
    assert np.max(np.abs(got - want)) < 4e-3
    # all V rows equal: the weights sum to one, so O repeats that row whatever Q and K are
    qkv = normal_f16((S, 3 * E), 13, std=1.0)
    qkv[:, 2 * E:] = v[7]
    got = run_attention(qkv, heads, False).astype(np.float32)
    assert np.max(np.abs(got - v[7].astype(np.float32)[None, :])) < 4e-3
    # a key that dominates: K row 5 = 16 * Q direction for every query, so O is V row 5 for rows >= 5
    qkv = np.zeros((S, 3 * E), np.float16)
    qkv[:, :E] = 1.0
    qkv[5, E:2 * E] = 16.0
    qkv[:, 2 * E:] = v
    got = run_attention(qkv, heads, True).astype(np.float32)
    assert np.array_equal(got[5:], np.broadcast_to(v[5].astype(np.float32), got[5:].shape))


def test_attention_persistent_launch_and_relaunch():
    qkv = normal_f16((512, 3 * 4 * 128), 14, std=1.0)
    got = run_attention(qkv, 4, True, max_workgroups=3, launches=2)
    assert_close(got, orc.attention(qkv, 4, 128, True), "O")


def test_attention_can_implement_rejects():
    import torch
    L = _lib.load()
    buf = torch.zeros(1 << 20, dtype=torch.float16, device="cuda")
    st = api.Stage(api.attention_grid(256, 2), (1, 1, 1), api.no_sync(), api.no_sync())

    def rc(seq=256, heads=2, ldqkv=768, ldo=256, **kw):
        a = api.attention_args(st, seq, heads, buf.data_ptr(), ldqkv, buf.data_ptr(), ldo, **kw)
        return L.cusync_attention_can_implement(C.byref(a))

    assert rc() == api.ERR.SUCCESS
    assert rc(head_dim=64) != api.ERR.SUCCESS
    assert rc(ldqkv=512) != api.ERR.SUCCESS          # narrower than Q|K|V
    assert rc(ldo=128) != api.ERR.SUCCESS
    assert rc(seq=512) != api.ERR.SUCCESS            # stage grid no longer matches
    assert rc(heads=3, ldqkv=1152, ldo=384) != api.ERR.SUCCESS
    assert "attention" in api.last_error()
    cons = api.Stage(api.attention_grid(256, 2), (1, 1, 1), api.strided_sync(api.ORDER.TRANSPOSE_XY, 256, 128, 128, 2), api.no_sync())
    a = api.attention_args(cons, 256, 2, buf.data_ptr(), 768, buf.data_ptr(), 256)
    assert L.cusync_attention_can_implement(C.byref(a)) != api.ERR.SUCCESS   # unpaired, and not a supported policy
    st.destroy(); cons.destroy()


_weights = {}


def layer_weights(hidden, heads):
    key = (hidden, heads)
    if key not in _weights:
        E = heads * 128
        wqkv = normal_f16((hidden, 3 * E), 2)
        wo = normal_f16((E, hidden), 3)
        _weights[key] = (wqkv, wo, to_dev(wqkv), to_dev(wo))
    return _weights[key]


def run_layer(S, hidden, heads, sync, runs=2, **kw):
    """`runs` passes through one handle; every pass starts from intermediates full of NaN and the passes before
    the last read another input, so that a stage that read before the post shows in what is returned."""
    import torch
    wqkv, wo, dwqkv, dwo = layer_weights(hidden, heads)
    E = heads * 128
    x = uniform_f16((S, hidden), 1)
    dx, dx_other = to_dev(x), to_dev(uniform_f16((S, hidden), 101))
    dqkv = empty_dev((S, 3 * E))
    do = empty_dev((S, E))
    dy = empty_dev((S, hidden))
    torch.cuda.synchronize()
    layer = api.AttnLayer(S, hidden, heads, sync, dwqkv.data_ptr(), dwo.data_ptr(), **kw)
    times = []
    for r in range(runs):
        dqkv.fill_(float("nan")); do.fill_(float("nan")); dy.fill_(float("nan"))
        torch.cuda.synchronize()
        times += layer.run((dx if r == runs - 1 else dx_other).data_ptr(), dqkv.data_ptr(), do.data_ptr(), dy.data_ptr(), runs=1)
    states = [layer.stage_state(i) for i in range(3)]
    tiles = layer.tiles()
    layer.destroy()
    return x, wqkv, wo, to_host(dqkv), to_host(do), to_host(dy), states, tiles, times


def expected_sems(state, tile_m, tile_n, iters):
    d = state.desc
    p = orc.Policy(d.out.kind, d.out.order, d.out.tileM, d.out.tileN, d.out.waitValue, d.out.postValue,
                   d.out.gridN, d.out.stride, d.out.R, d.out.S, d.out.H)
    return orc.expected_sems_gemm(p, state.grid, tile_m, tile_n, iters, d.opts)


def check_layer(S, hidden, heads, sampled, **kw):
    outs = {}
    for sync in (api.SYNC.STREAM, api.SYNC.ROW, api.SYNC.TILE, api.SYNC.STRIDED):
        print("  sync", sync, flush=True)
        x, wqkv, wo, qkv, o, y, states, tiles, _ = run_layer(S, hidden, heads, sync, runs=2, **kw)
        outs[sync] = (qkv, o, y)
        for st in states:
            assert st.spin_timeouts == 0 and st.tile_counter == 0 and st.start_counter == 0
        if sync != api.SYNC.STREAM:
            tm, tn, _ = api.tile_shape(tiles[0])
            assert np.array_equal(states[0].sems, expected_sems(states[0], tm, tn, 2))
            assert np.array_equal(states[1].sems, expected_sems(states[1], 128, 128, 2))
            assert states[0].kernel_executed == 2 and states[1].kernel_executed == 2
    qkv, o, y = outs[api.SYNC.STREAM]
    rows = sample_rows(S) if sampled else list(range(S))
    assert_close(qkv[rows], orc.gemm(np.ascontiguousarray(x[rows]), wqkv), "QKV rows")
    # later stages are checked on the intermediates the GPU produced
    assert_close(o, orc.attention(qkv, heads, 128, True), "O")
    assert_close(y[rows], orc.gemm(np.ascontiguousarray(o[rows]), wo), "Y rows")
    for sync in (api.SYNC.ROW, api.SYNC.TILE, api.SYNC.STRIDED):       # synchronisation only changes timing
        for got, want, name in zip(outs[sync], outs[api.SYNC.STREAM], ("QKV", "O", "Y")):
            assert np.array_equal(got.view(np.uint16), want.view(np.uint16)), (sync, name)


@pytest.mark.parametrize("S,tile", [(256, api.TILE.T128x128x64), (200, api.TILE.T64x128x64), (384, api.TILE.T128x256x32)])
def test_attention_layer_small(S, tile):
    print("attn layer small", S, tile, flush=True)
    check_layer(S, 512, 2, sampled=False, tile1=tile, tile3=tile)


# 320, 768 and 1280 rows fall between the tuned lengths: ragged row tiles, and tile shapes that differ from one stage to the next
@pytest.mark.parametrize("S", [256, 320, 512, 768, 1024, 1280, 1536, 2048])
def test_attention_layer_gpt3_shard(S):
    print("attn layer gpt3", S, flush=True)
    check_layer(S, 12288, 12, sampled=True)


# ---- key/value cache variant (src/ml-bench/transformer/attention.cu:265-276, 289) ----------------

def run_attention_kv(qkv, cached, heads, causal=True):
    import torch
    L = _lib.load()
    S = qkv.shape[0] - cached
    dq = to_dev(qkv)
    do = empty_dev((S, heads * 128), fill=float("nan"))
    torch.cuda.synchronize()
    st = api.Stage(api.attention_grid(S, heads), (1, 1, 1), api.no_sync(), api.no_sync())
    rc = api.attention(st, S, heads, dq.data_ptr(), qkv.shape[1], do.data_ptr(), heads * 128, causal=causal, cached_rows=cached)
    assert rc == api.ERR.SUCCESS, api.last_error()
    assert L.cusync_rt_device_sync() == 0, api.last_error()
    st.destroy()
    return to_host(do)


@pytest.mark.parametrize("causal", [True, False])
@pytest.mark.parametrize("S,cached,heads", [(1, 1, 1), (1, 2047, 2), (16, 64, 1), (16, 100, 3), (200, 500, 2), (130, 63, 1), (256, 1024, 12)])
def test_attention_with_cache_matches_oracle(S, cached, heads, causal):
    print("attention kv", S, cached, heads, causal, flush=True)
    qkv = normal_f16((cached + S, 3 * heads * 128), 15, std=1.0)
    got = run_attention_kv(qkv, cached, heads, causal)
    assert_close(got, orc.attention_kv(qkv, cached, heads, 128, causal), "O")
    if causal:
        # the same rows of plain causal attention over the whole sequence, bit for bit
        full = run_attention(qkv, heads, True)
        assert np.array_equal(got.view(np.uint16), full[cached:].view(np.uint16))


@pytest.mark.parametrize("S,cached", [(16, 512), (64, 1024), (256, 2048), (200, 300)])
def test_attention_layer_with_cache(S, cached):
    # the reference's decode-time shape: `batch` new rows behind `seqlen` cached ones; the projection writes
    # its rows behind the cache and the attention only waits for those
    import torch
    print("attn layer kv", S, cached, flush=True)
    hidden, heads = 12288, 12
    E = heads * 128
    wqkv, wo, dwqkv, dwo = layer_weights(hidden, heads)
    x = uniform_f16((S, hidden), 1)
    cache = normal_f16((cached, 3 * E), 16, std=1.0)
    dx = to_dev(x)
    outs = {}
    for sync in (api.SYNC.STREAM, api.SYNC.ROW, api.SYNC.TILE, api.SYNC.STRIDED):
        dqkv = empty_dev((cached + S, 3 * E), fill=float("nan"))
        dqkv[:cached] = to_dev(cache)
        do = empty_dev((S, E), fill=float("nan"))
        dy = empty_dev((S, hidden), fill=float("nan"))
        torch.cuda.synchronize()
        layer = api.AttnLayer(S, hidden, heads, sync, dwqkv.data_ptr(), dwo.data_ptr(), cached_rows=cached)
        dx_other = to_dev(uniform_f16((S, hidden), 101))
        layer.run(dx_other.data_ptr(), dqkv.data_ptr(), do.data_ptr(), dy.data_ptr(), runs=1)
        dqkv[cached:] = float("nan"); do.fill_(float("nan")); dy.fill_(float("nan"))       # second pass: fresh NaN, another input
        torch.cuda.synchronize()
        layer.run(dx.data_ptr(), dqkv.data_ptr(), do.data_ptr(), dy.data_ptr(), runs=1)
        for i in range(3):
            st = layer.stage_state(i)
            assert st.spin_timeouts == 0 and st.tile_counter == 0
        layer.destroy()
        outs[sync] = (to_host(dqkv), to_host(do), to_host(dy))
    qkv, o, y = outs[api.SYNC.STREAM]
    assert np.array_equal(qkv[:cached].view(np.uint16), cache.view(np.uint16))       # the cache rows are untouched
    rows = sample_rows(S)
    assert_close(qkv[cached:][rows], orc.gemm(np.ascontiguousarray(x[rows]), wqkv), "new QKV rows")
    assert_close(o, orc.attention_kv(qkv, cached, heads, 128, True), "O")
    assert_close(y[rows], orc.gemm(np.ascontiguousarray(o[rows]), wo), "Y rows")
    for sync in (api.SYNC.ROW, api.SYNC.TILE, api.SYNC.STRIDED):
        for got, want, name in zip(outs[sync], outs[api.SYNC.STREAM], ("QKV", "O", "Y")):
            assert np.array_equal(got.view(np.uint16), want.view(np.uint16)), (sync, name)


# ---- key range split over several workgroups --------------------------------------------------------------

def run_attention_split(qkv, cached, heads, causal, blocks, launches=2, max_workgroups=0):
    import torch
    L = _lib.load()
    S = qkv.shape[0] - cached
    dq = to_dev(qkv)
    do = empty_dev((S, heads * 128), fill=float("nan"))
    grid = api.attention_grid(S, heads, cached, blocks)
    ws_bytes = api.attention_workspace_size(S, heads, cached, blocks)
    ws = torch.zeros(max(16, ws_bytes), dtype=torch.uint8, device="cuda")
    torch.cuda.synchronize()
    st = api.Stage(grid, (1, 1, 1), api.no_sync(), api.no_sync())
    for _ in range(launches):           # the second launch finds the arrival counters re-armed
        do.fill_(float("nan"))
        torch.cuda.synchronize()
        rc = api.attention(st, S, heads, dq.data_ptr(), qkv.shape[1], do.data_ptr(), heads * 128, causal=causal, cached_rows=cached,
                           kv_split_blocks=blocks, workspace=ws.data_ptr(), max_workgroups=max_workgroups)
        assert rc == api.ERR.SUCCESS, api.last_error()
        assert L.cusync_rt_device_sync() == 0, api.last_error()
    assert st.read_state().tile_counter == 0
    st.destroy()
    return to_host(do), grid


@pytest.mark.parametrize("causal", [True, False])
@pytest.mark.parametrize("S,cached,heads,blocks", [(300, 0, 2, 1), (512, 0, 3, 2), (1000, 0, 1, 3), (129, 200, 2, 2), (16, 500, 1, 4),
                                                   (2048, 0, 2, 8), (64, 0, 1, 8)])
def test_attention_split_key_range(S, cached, heads, blocks, causal):
    print("attention split", S, cached, heads, blocks, causal, flush=True)
    qkv = normal_f16((cached + S, 3 * heads * 128), 21, std=1.0)
    got, grid = run_attention_split(qkv, cached, heads, causal, blocks)
    kv_blocks = -(-(cached + S) // 64)
    assert grid == (heads, (S + 127) // 128, max(1, -(-kv_blocks // blocks)))
    assert_close(got, orc.attention_kv(qkv, cached, heads, 128, causal), "O")
    # few workgroups: splits of one tile run one after the other, the last one still puts the tile together
    got2, _ = run_attention_split(qkv, cached, heads, causal, blocks, launches=1, max_workgroups=2)
    assert np.array_equal(got.view(np.uint16), got2.view(np.uint16))      # the result does not depend on arrival order


def test_attention_split_closed_form():
    # Q = 0: row i of O is the mean of V rows 0..i, however the key range is cut
    S, heads = 700, 1
    rng = np.random.default_rng(6)
    qkv = normal_f16((S, 3 * 128), 22, std=1.0)
    qkv[:, :128] = 0
    v = rng.integers(-4, 5, (S, 128)).astype(np.float16)
    qkv[:, 256:] = v
    got, _ = run_attention_split(qkv, 0, heads, True, 2)
    want = np.cumsum(v.astype(np.float64), axis=0) / np.arange(1, S + 1)[:, None]
    assert np.max(np.abs(got.astype(np.float32) - want)) < 4e-3


def test_attention_split_needs_workspace():
    st = api.Stage(api.attention_grid(512, 1, 0, 2), (1, 1, 1), api.no_sync(), api.no_sync())
    dq = to_dev(normal_f16((512, 384), 23)); do = empty_dev((512, 128))
    a = api.attention_args(st, 512, 1, dq.data_ptr(), 384, do.data_ptr(), 128, kv_split_blocks=2, workspace=None)
    assert _lib.load().cusync_attention_can_implement(C.byref(a)) != api.ERR.SUCCESS
    st.destroy()
