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


@pytest.mark.parametrize("policy,split_k1", [(0, 1), (1, 1), (0, 2), (1, 4)])
def test_mlp_loop_on_the_launcher_objects(policy, split_k1):
    """The reference's runCuSyncGPT3 loop (TB/mlp.cu:645-716), written on cusync::CuSyncGemm (include/cusync/gemm.h):
    Arguments -> get_workspace_size -> can_implement -> initialize, then run(true, NULL, stream) per iteration with
    incrementIter on the stages and on params_.custage.  H is refilled with NaN before the call; the outputs are
    compared with the oracle, the semaphores with iters (TileSync) / iters * gN (RowSync)."""
    import torch
    from util import assert_close, normal_f16, to_dev, to_host, uniform_f16
    print("launcher mlp", policy, split_k1, flush=True)
    T = _lib.load_stage_tests()
    M, K1, N1, N2 = 300, 1024, 512, 768
    x, w1, w2 = uniform_f16((M, K1), 1), normal_f16((K1, N1), 2, std=0.05), normal_f16((N1, N2), 3, std=0.05)
    dx, dw1, dw2 = to_dev(x), to_dev(w1), to_dev(w2)
    dh = torch.full((M, N1), float("nan"), dtype=torch.float16, device="cuda")
    dy = torch.full((M, N2), float("nan"), dtype=torch.float16, device="cuda")
    torch.cuda.synchronize()
    out = (C.c_int * 4)(-1, -1, -1, -1)
    iters = 3
    rc = T.run_launcher_mlp(policy, C.c_uint32(M), C.c_uint32(K1), C.c_uint32(N1), C.c_uint32(N2), C.c_void_p(dx.data_ptr()),
                            C.c_void_p(dw1.data_ptr()), C.c_void_p(dh.data_ptr()), C.c_void_p(dw2.data_ptr()), C.c_void_p(dy.data_ptr()),
                            split_k1, iters, out)
    assert rc == 0
    assert list(out) == [0, 0, iters, 0], list(out)       # every status success, no time-out, flag == iters, semaphores as expected
    h, y = to_host(dh), to_host(dy)
    assert_close(h, orc.gemm(x, w1, orc.EPI_GELU), "H")
    assert_close(y, orc.gemm(h, w2), "Y")


def test_resnet_pair_on_the_convolution_launcher():
    """The ResNet pair (CV/resnet.cu:107-116, 704-744) on cusync::CuSyncImplicitGemmConvolution: TileSync producer,
    Conv2DTileSync consumer, run(true, NULL, stream) per iteration."""
    import torch
    from util import assert_close, to_dev, to_host, uniform_f16
    T = _lib.load_stage_tests()
    N, H, W, Cc = 4, 20, 20, 64
    rng = np.random.default_rng(5)
    x = uniform_f16((N, H, W, Cc), 4)
    w1, w2 = ((rng.standard_normal((Cc, 3, 3, Cc)) * np.sqrt(2.0 / (9 * Cc))).astype(np.float16) for _ in range(2))
    dx, dw1, dw2 = to_dev(x), to_dev(w1), to_dev(w2)
    dy1 = torch.full((N, H, W, Cc), float("nan"), dtype=torch.float16, device="cuda")
    dy2 = torch.full((N, H, W, Cc), float("nan"), dtype=torch.float16, device="cuda")
    torch.cuda.synchronize()
    out = (C.c_int * 4)(-1, -1, -1, -1)
    rc = T.run_launcher_conv_pair(C.c_uint32(N), C.c_uint32(H), C.c_uint32(W), C.c_uint32(Cc), C.c_void_p(dx.data_ptr()), C.c_void_p(dw1.data_ptr()),
                                  C.c_void_p(dy1.data_ptr()), C.c_void_p(dw2.data_ptr()), C.c_void_p(dy2.data_ptr()), 2, out)
    assert rc == 0
    assert list(out) == [0, 0, 2, 0], list(out)
    y1, y2 = to_host(dy1), to_host(dy2)
    assert_close(y1, orc.conv2d_nhwc(x, w1, epilogue=orc.EPI_RELU), "y1")
    assert_close(y2, orc.conv2d_nhwc(y1, w2), "y2")


@pytest.mark.parametrize("runs", [1, 2, 4])
def test_resnet_pair_on_the_convolution_launcher_with_runs(runs):
    """Conv2dProblemSize::split_k_slices (CV/resnet.cu:246, 689) on the launcher objects: get_workspace_size, initialize with the
    workspace (refused without), the 128x128 halo tile, a deep layer's shape."""
    import torch
    from util import assert_close, to_dev, to_host, uniform_f16
    T = _lib.load_stage_tests()
    N, H, W, Cc = 4, 14, 14, 256
    rng = np.random.default_rng(6)
    x = uniform_f16((N, H, W, Cc), 7)
    w1, w2 = ((rng.standard_normal((Cc, 3, 3, Cc)) * np.sqrt(2.0 / (9 * Cc))).astype(np.float16) for _ in range(2))
    dx, dw1, dw2 = to_dev(x), to_dev(w1), to_dev(w2)
    dy1 = torch.full((N, H, W, Cc), float("nan"), dtype=torch.float16, device="cuda")
    dy2 = torch.full((N, H, W, Cc), float("nan"), dtype=torch.float16, device="cuda")
    torch.cuda.synchronize()
    out = (C.c_int * 4)(-1, -1, -1, -1)
    rc = T.run_launcher_conv_pair_runs(C.c_uint32(N), C.c_uint32(H), C.c_uint32(W), C.c_uint32(Cc), C.c_void_p(dx.data_ptr()), C.c_void_p(dw1.data_ptr()),
                                       C.c_void_p(dy1.data_ptr()), C.c_void_p(dw2.data_ptr()), C.c_void_p(dy2.data_ptr()), runs, 3, out)
    assert rc == 0
    assert list(out) == [0, 0, 3, 0], list(out)
    y1, y2 = to_host(dy1), to_host(dy2)
    assert_close(y1, orc.conv2d_nhwc(x, w1, epilogue=orc.EPI_RELU), "y1")
    assert_close(y2, orc.conv2d_nhwc(y1, w2), "y2")
