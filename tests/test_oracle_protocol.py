"""Pins the integer half of the oracle (tile orders, policies, semaphore end
state) against closed forms, brute force and the reference's own known answers,
so that a dropped term, a swapped x/y or a wrong divisor fails here."""
import itertools

import numpy as np
import pytest

import oracle as orc


# ---- tile orders -----------------------------------------------------------

@pytest.mark.parametrize("order", [orc.ORDER_IDENTITY, orc.ORDER_TRANSPOSE_XY])
def test_block_index_closed_form(order):
    # CS/tile-orders.h:52-54,68-70
    for grid in itertools.product(range(1, 6), repeat=3):
        seen = set()
        for z, y, x in itertools.product(range(grid[2]), range(grid[1]), range(grid[0])):
            i = orc.block_index(order, grid, (x, y, z))
            assert i == x + y * grid[0] + z * grid[0] * grid[1]
            seen.add(i)
        assert seen == set(range(grid[0] * grid[1] * grid[2]))  # bijection


def test_tile_to_block():
    assert orc.tile_to_block(orc.ORDER_IDENTITY, (3, 5, 7)) == (3, 5, 7)
    assert orc.tile_to_block(orc.ORDER_TRANSPOSE_XY, (3, 5, 7)) == (5, 3, 7)


def test_tile_index_transposes():
    # tile (m-idx, n-idx) on a grid (n-tiles, m-tiles): index = n + m * gx
    grid = (48, 8, 1)
    assert orc.tile_index(orc.ORDER_TRANSPOSE_XY, (1, 3, 0), grid) == 3 + 1 * 48
    assert orc.tile_index(orc.ORDER_IDENTITY, (1, 3, 0), grid) == 1 + 3 * 48


@pytest.mark.parametrize("grid", [(1, 1, 1), (8192, 1, 1), (48, 8, 1), (24, 8, 3), (5, 4, 3)])
def test_schedule_buffer_is_identity_linearisation(grid):
    # closed form: tileOrder[id] = (id % gx, (id/gx) % gy, id/(gx*gy))
    rc, sched = orc.build_schedule(orc.ORDER_TRANSPOSE_XY, grid)
    assert rc == orc.SUCCESS == 5
    ids = np.arange(grid[0] * grid[1] * grid[2])
    want = np.stack([ids % grid[0], (ids // grid[0]) % grid[1], ids // (grid[0] * grid[1])], 1)
    assert np.array_equal(sched, want.astype(np.uint32))


def test_error_enum_order():
    # CS/cusync.h:46-53 — success is the LAST enumerator
    assert (orc.ERR_NOT_PRODUCER, orc.ERR_NOT_CONSUMER, orc.ERR_NOT_INITIALIZED,
            orc.ERR_INVALID_LINEAR_BLOCK_INDEX, orc.ERR_DEVICE, orc.SUCCESS) == (0, 1, 2, 3, 4, 5)
    assert (orc.OPT_NO_ATOMIC_ADD, orc.OPT_AVOID_WAIT_KERNEL, orc.OPT_AVOID_CUSTOM_ORDER,
            orc.OPT_REORDER_TILE_LOADS) == (1, 2, 4, 8)


# ---- policies ----------------------------------------------------------------

def test_tilesync_hand_worked():
    # TileSync<TransposeXY,256,128> on grid (48,8): tile{256,384,0} -> {1,3} -> block{3,1} -> 51
    p = orc.policy(orc.TILESYNC, orc.ORDER_TRANSPOSE_XY, 256, 128)
    assert orc.policy_tile_index(p, (256, 384, 0), (48, 8, 1)) == 51
    assert orc.policy_wait_value(p, (0, 0, 0), (48, 8, 1)) == 1
    assert orc.policy_post_value(p, (0, 0, 0), (48, 8, 1)) == 1
    assert orc.policy_is_sync(p, (256, 384, 0), (48, 8, 1))
    assert not orc.policy_is_sync(p, (256, 384 + 32, 0), (48, 8, 1))
    # Identity order, the example's (col,row) convention (EX/twoMatMuls/matrixMul.cu:91,120)
    q = orc.policy(orc.TILESYNC, orc.ORDER_IDENTITY, 32, 32)
    assert orc.policy_tile_index(q, (64, 96, 0), (8, 8, 1)) == 2 + 3 * 8


def test_rowsync():
    p = orc.policy(orc.ROWSYNC, tileM=256, waitValue=24)
    assert p.postValue == 1
    assert orc.policy_tile_index(p, (512 + 17, 999, 0), (24, 8, 1)) == 2
    assert orc.policy_wait_value(p, (0, 0, 0), (24, 8, 1)) == 24
    assert orc.policy_post_value(p, (0, 0, 0), (24, 8, 1)) == 1
    assert orc.policy_is_sync(p, (0, 0, 1), (24, 8, 1))
    assert not orc.policy_is_sync(p, (0, 0, 0), (24, 8, 1))
    d = orc.policy(orc.ROWSYNC, tileM=1)   # default ctor: both zero (CS/policies.h:49)
    assert (d.waitValue, d.postValue) == (0, 0)


def test_stridedsync_folds_upper_half():
    # TB/mlp.cu:76-101 with GridN=2816, TileN=128: 22 tiles per group
    p = orc.policy(orc.STRIDEDSYNC, orc.ORDER_TRANSPOSE_XY, 256, 128, gridN=2816, stride=2)
    grid = (44, 4, 1)
    for ty in range(44):
        want = (ty % 22) + 3 * 44
        assert orc.policy_tile_index(p, (3 * 256, ty * 128, 0), grid) == want
    assert orc.policy_wait_value(p, (0, 0, 0), grid) == 2
    assert orc.policy_post_value(p, (0, 0, 0), grid) == 1
    assert orc.policy_is_sync(p, (0, 256, 0), grid) and not orc.policy_is_sync(p, (0, 200, 0), grid)


def test_conv2dtilesync():
    # CS/policies.h:160-210, R=S=3, TileN=64: K-tiles 0..8 map to channel tile 0
    p = orc.policy(orc.CONV2DTILESYNC, orc.ORDER_TRANSPOSE_XY, 64, 64, R=3, S=3)
    grid = (1, 1568, 1)
    for kt in range(9):
        assert orc.policy_tile_index(p, (5 * 64, kt * 64, 0), grid) == 0 + 5 * 1
        assert orc.policy_is_sync(p, (5 * 64, kt * 64, 0), grid) == (kt == 0)
    grid2 = (2, 392, 1)
    assert orc.policy_tile_index(p, (7 * 64, 9 * 64, 0), grid2) == 1 + 7 * 2
    assert orc.policy_is_sync(p, (0, 9 * 64, 0), grid2)


def test_consecutivesync():
    # TB/attention.cu:51-70, H=12288, TileN=128: g = 1536/128 = 12, grid.x = 36 -> 3 groups
    p = orc.policy(orc.CONSECUTIVESYNC, orc.ORDER_TRANSPOSE_XY, 128, 128, H=12288)
    grid = (36, 4, 1)
    assert orc.policy_wait_value(p, (0, 0, 0), grid) == 12
    for nt in range(36):
        assert orc.policy_tile_index(p, (2 * 128, nt * 128, 1), grid) == nt // 12 + 2 * 3
    assert orc.policy_is_sync(p, (0, 0, 1), grid) and not orc.policy_is_sync(p, (0, 0, 0), grid)


def test_nosync():
    p = orc.policy(orc.NOSYNC)
    assert orc.policy_tile_index(p, (9, 9, 9), (3, 3, 3)) == 0
    assert orc.policy_wait_value(p, (9, 9, 9), (3, 3, 3)) == 0
    assert orc.policy_post_value(p, (9, 9, 9), (3, 3, 3)) == 0
    assert not orc.policy_is_sync(p, (0, 0, 1), (3, 3, 3))


# ---- semaphore end state -------------------------------------------------------

@pytest.mark.parametrize("iters", [1, 2, 5])
@pytest.mark.parametrize("opts", [0, orc.OPT_NO_ATOMIC_ADD])
def test_simple_test_known_answer(iters, opts):
    # tests/simple-test.cu:59-66,108-137: 8192 blocks, TileSync<Identity,1,1>, every sem == iters
    p = orc.policy(orc.TILESYNC, orc.ORDER_IDENTITY, 1, 1)
    sems = orc.expected_sems_blocks(p, (8192, 1, 1), iters, opts)
    assert sems.shape == (8192,) and np.all(sems == iters)


def test_matrixmul_example_known_answer():
    # EX/twoMatMuls/matrixMul.cu: grid (8,8), TileSync<Identity,32,32>, posts {bx*32, by*32, 0}
    p = orc.policy(orc.TILESYNC, orc.ORDER_IDENTITY, 32, 32)
    # the example posts (col,row): emulate through the block variant with tile = block*32
    sems = np.zeros(64, dtype=np.uint32)
    for by in range(8):
        for bx in range(8):
            sems[orc.policy_tile_index(p, (bx * 32, by * 32, 0), (8, 8, 1))] += 1
    assert np.all(sems == 1)


@pytest.mark.parametrize("iters", [1, 3])
def test_gemm_sems_closed_forms(iters):
    gx, gy = 24, 8
    ts = orc.policy(orc.TILESYNC, orc.ORDER_TRANSPOSE_XY, 256, 256)
    for opts in (0, orc.OPT_NO_ATOMIC_ADD):
        assert np.all(orc.expected_sems_gemm(ts, (gx, gy, 1), 256, 256, iters, opts) == iters)
    # split-K: only the last slice posts; entries >= gx*gy stay 0
    s = orc.expected_sems_gemm(ts, (gx, gy, 3), 256, 256, iters)
    assert np.all(s[:gx * gy] == iters) and np.all(s[gx * gy:] == 0)
    rs = orc.policy(orc.ROWSYNC, tileM=256, waitValue=gx)
    s = orc.expected_sems_gemm(rs, (gx, gy, 1), 256, 256, iters)
    assert np.all(s[:gy] == iters * gx) and np.all(s[gy:] == 0)
    # StridedSync(stride 2), d = 2816, TileN = 128 -> gx = 44
    st = orc.policy(orc.STRIDEDSYNC, orc.ORDER_TRANSPOSE_XY, 256, 128, gridN=2816, stride=2)
    s = orc.expected_sems_gemm(st, (44, gy, 1), 256, 128, iters).reshape(gy, 44)
    assert np.all(s[:, :22] == 2 * iters) and np.all(s[:, 22:] == 0)
    # ConsecutiveSync: 3 semaphores per M-row, each I*g
    cs = orc.policy(orc.CONSECUTIVESYNC, orc.ORDER_TRANSPOSE_XY, 128, 128, H=12288)
    s = orc.expected_sems_gemm(cs, (36, 4, 1), 128, 128, iters)
    assert np.all(s[:12] == 12 * iters) and np.all(s[12:] == 0)


# ---- CPU replay of the wait/post protocol --------------------------------------

def _mlp_case(tm, tn, B=1024):
    prod = (6144 // tn, -(-B // tm), 1)
    cons = (12288 // tn, -(-B // tm), 1)
    return prod, cons


@pytest.mark.parametrize("slots", [(1, 1), (4, 7), (1000, 1000)])
def test_replay_tilesync_and_rowsync_complete(slots):
    prod, cons = _mlp_case(256, 256)
    ts = orc.policy(orc.TILESYNC, orc.ORDER_TRANSPOSE_XY, 256, 256)
    ok, sems = orc.replay_chain(ts, prod, cons, (256, 256), 256, 64, 6144, slots[0], slots[1], iters=2)
    assert ok and np.all(sems == 2)
    rs = orc.policy(orc.ROWSYNC, tileM=256, waitValue=prod[0])
    ok, sems = orc.replay_chain(rs, prod, cons, (256, 256), 256, 64, 6144, slots[0], slots[1], iters=2)
    assert ok and np.all(sems[:prod[1]] == 2 * prod[0])


def test_replay_detects_incompatible_no_atomic_add():
    # RowSync counts to gN; a plain store of postValue*iter can never reach it
    prod, cons = _mlp_case(256, 256)
    rs = orc.policy(orc.ROWSYNC, tileM=256, waitValue=prod[0])
    ok, _ = orc.replay_chain(rs, prod, cons, (256, 256), 256, 64, 6144, 8, 8, iters=1,
                             opts=orc.OPT_NO_ATOMIC_ADD)
    assert not ok
    ts = orc.policy(orc.TILESYNC, orc.ORDER_TRANSPOSE_XY, 256, 256)
    ok, sems = orc.replay_chain(ts, prod, cons, (256, 256), 256, 64, 6144, 8, 8, iters=3,
                                opts=orc.OPT_NO_ATOMIC_ADD)
    assert ok and np.all(sems == 3)


def test_replay_detects_wrong_wait_value():
    prod, cons = _mlp_case(256, 256)
    rs = orc.policy(orc.ROWSYNC, tileM=256, waitValue=prod[0] + 1)   # one post too many expected
    ok, _ = orc.replay_chain(rs, prod, cons, (256, 256), 256, 64, 6144, 8, 8)
    assert not ok
