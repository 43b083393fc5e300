"""GPU tests of the CuStage protocol through user-written kernels, following the
reference's own test file (tests/simple-test.cu) and example
(src/examples/twoMatMuls/matrixMul.cu).  Semaphores, tile-order maps and
counters are compared bit-exactly with the CPU oracle."""
import ctypes as C

import numpy as np
import pytest

import oracle as orc
from cusync_amd import _lib, api

pytestmark = pytest.mark.gpu


class SimpleResult(C.Structure):
    _fields_ = [(n, C.c_int32) for n in ("data_ok", "sems_ok", "prod_status", "cons_status", "pair_status", "wait_status")] + \
               [(n, C.c_uint32) for n in ("tile_counter_prod", "tile_counter_cons", "kernel_executed", "spin_timeouts")]


def run_simple(variant, iters, blocks=8192):
    T = _lib.load_stage_tests()
    res = SimpleResult()
    sems = np.full(blocks, 0xFFFFFFFF, np.uint32)
    order = np.zeros((blocks, 3), np.uint32)
    rc = T.run_simple_test(variant, iters, C.c_uint32(blocks), C.byref(res),
                           sems.ctypes.data_as(C.c_void_p), order.ctypes.data_as(C.c_void_p))
    assert rc == 0
    return res, sems, order


# tests/simple-test.cu:107-137 — the four reference cases (+ more iterations)
@pytest.mark.parametrize("variant,iters,opts", [
    (0, 1, orc.OPT_NONE), (0, 2, orc.OPT_NONE), (1, 1, orc.OPT_NO_ATOMIC_ADD),
    (2, 1, orc.OPT_AVOID_CUSTOM_ORDER), (0, 5, orc.OPT_NONE), (1, 3, orc.OPT_NO_ATOMIC_ADD),
])
def test_simple_copy_pair(variant, iters, opts):
    print("case variant=%d iters=%d" % (variant, iters), flush=True)
    blocks = 8192
    res, sems, order = run_simple(variant, iters, blocks)
    assert res.prod_status == res.cons_status == res.pair_status == res.wait_status == api.ERR.SUCCESS
    assert res.spin_timeouts == 0
    assert res.data_ok == 1          # out[i] == i for both stages
    assert res.sems_ok == 1          # sem[waitTileIndex] == expectedWaitValue * iter at every consumer block
    p = orc.policy(orc.TILESYNC, orc.ORDER_IDENTITY, 1, 1)
    assert np.array_equal(sems, orc.expected_sems_blocks(p, (blocks, 1, 1), iters, opts))
    rc, want_order = orc.build_schedule(orc.ORDER_IDENTITY, (blocks, 1, 1))
    assert rc == orc.SUCCESS and np.array_equal(order, want_order)
    assert res.tile_counter_prod == 0 and res.tile_counter_cons == 0    # re-armed by the last ticket
    assert res.kernel_executed == iters


def test_two_matmuls_known_answer():
    # matrixMul.cu:149-152,235-272: A = 1, B = D = 0.01, n = 256 -> C = 2.56, E = 2.56 * 2.56
    import torch
    T = _lib.load_stage_tests()
    n = 256
    A = torch.ones(n, n, device="cuda")
    B = torch.full((n, n), 0.01, device="cuda")
    D = torch.full((n, n), 0.01, device="cuda")
    Cm = torch.zeros(n, n, device="cuda")
    E = torch.zeros(n, n, device="cuda")
    torch.cuda.synchronize()
    sems = np.zeros((n // 32) ** 2, np.uint32)
    status = (C.c_int * 3)()
    rc = T.run_two_matmuls(n, C.c_void_p(A.data_ptr()), C.c_void_p(B.data_ptr()), C.c_void_p(D.data_ptr()),
                           C.c_void_p(Cm.data_ptr()), C.c_void_p(E.data_ptr()), sems.ctypes.data_as(C.c_void_p), status)
    assert rc == 0 and status[0] == status[1] == api.ERR.SUCCESS and status[2] == 0
    c, e = Cm.cpu().numpy().astype(np.float64), E.cpu().numpy().astype(np.float64)
    eps = 1e-5
    assert np.all(np.abs(c - n * 0.01) / np.abs(c) / n < eps)
    assert np.all(np.abs(e - (n * 0.01) ** 2) / np.abs(e) / n < eps)
    assert np.all(sems == 1)       # 64 semaphores, one post each


def test_two_matmuls_random_against_oracle_order():
    # random data: a consumer that read a C tile before it was posted would be wrong
    import torch
    T = _lib.load_stage_tests()
    n = 512
    g = torch.Generator().manual_seed(7)
    A = (torch.rand(n, n, generator=g) * 2 - 1).cuda()
    B = (torch.rand(n, n, generator=g) * 2 - 1).cuda()
    D = (torch.rand(n, n, generator=g) * 2 - 1).cuda()
    Cm = torch.full((n, n), float("nan"), device="cuda")
    E = torch.zeros(n, n, device="cuda")
    torch.cuda.synchronize()
    sems = np.zeros((n // 32) ** 2, np.uint32)
    status = (C.c_int * 3)()
    rc = T.run_two_matmuls(n, C.c_void_p(A.data_ptr()), C.c_void_p(B.data_ptr()), C.c_void_p(D.data_ptr()),
                           C.c_void_p(Cm.data_ptr()), C.c_void_p(E.data_ptr()), sems.ctypes.data_as(C.c_void_p), status)
    assert rc == 0 and status[2] == 0
    c_ref = A.double().cpu() @ B.double().cpu()
    e_ref = c_ref @ D.double().cpu()
    assert torch.allclose(Cm.double().cpu(), c_ref, rtol=1e-4, atol=1e-3)
    assert torch.allclose(E.double().cpu(), e_ref, rtol=1e-4, atol=1e-2)
    assert np.all(sems == 1)


def test_error_paths():
    # CS/cusync.h:289-294, :204 — wrong roles are reported, nothing is launched
    T = _lib.load_stage_tests()
    out = (C.c_int * 5)()
    assert T.run_error_paths(out) == 0
    assert out[0] == api.ERR.NOT_PRODUCER
    assert out[1] == api.ERR.NOT_CONSUMER
    assert out[2] == api.ERR.NOT_PRODUCER
    assert out[3] == api.ERR.SUCCESS
    assert out[4] == api.ERR.NOT_INITIALIZED


def test_stage_state_after_create():
    p = api.tile_sync(api.ORDER.TRANSPOSE_XY, 256, 128)
    s = api.Stage((48, 8, 1), (1, 1, 1), api.no_sync(), p)
    st = s.read_state()
    rc, want = orc.build_schedule(orc.ORDER_TRANSPOSE_XY, (48, 8, 1))
    assert np.array_equal(st.tile_order, want)
    assert np.all(st.sems == 0) and st.tile_counter == 0 and st.kernel_executed == 0 and st.start_counter == 0
    c = api.Stage((96, 8, 1), (1, 1, 1), p, api.no_sync())
    assert api.set_producer_consumer_pair(s, c) == api.ERR.SUCCESS
    assert c.desc.prodGrid.tup() == (48, 8, 1) and c.desc.tileStatusRead == s.desc.tileStatusWrite
    assert api.set_producer_consumer_pair(c, s) == api.ERR.NOT_PRODUCER
    assert c.invokeWaitKernel(None) == api.ERR.NOT_PRODUCER     # rejected on the host, nothing is enqueued
    s.destroy(); c.destroy()
