"""ctypes front end of the CPU oracle (``cusync_oracle.c``).

TEST INFRASTRUCTURE ONLY.  Importers are limited to ``tests/``,
``__graft_entry__.smoke()`` and the ``cpu_baseline`` leg of ``bench.py``.  The
shipped package (``cusync_amd``) never imports this module.
"""
import ctypes as C
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_SO = os.path.join(_HERE, "libcusync_oracle.so")

ORDER_IDENTITY, ORDER_TRANSPOSE_XY = 0, 1
NOSYNC, ROWSYNC, TILESYNC, STRIDEDSYNC, CONV2DTILESYNC, CONSECUTIVESYNC = range(6)
(ERR_NOT_PRODUCER, ERR_NOT_CONSUMER, ERR_NOT_INITIALIZED,
 ERR_INVALID_LINEAR_BLOCK_INDEX, ERR_DEVICE, SUCCESS) = range(6)
OPT_NONE, OPT_NO_ATOMIC_ADD, OPT_AVOID_WAIT_KERNEL, OPT_AVOID_CUSTOM_ORDER, OPT_REORDER_TILE_LOADS = 0, 1, 2, 4, 8
EPI_NONE, EPI_GELU, EPI_RELU = 0, 1, 2


class Dim3(C.Structure):
    _fields_ = [("x", C.c_uint32), ("y", C.c_uint32), ("z", C.c_uint32)]

    def tup(self):
        return (self.x, self.y, self.z)


class Policy(C.Structure):
    _fields_ = [("kind", C.c_int32), ("order", C.c_int32),
                ("tileM", C.c_uint32), ("tileN", C.c_uint32),
                ("waitValue", C.c_uint32), ("postValue", C.c_uint32),
                ("gridN", C.c_uint32), ("stride", C.c_uint32),
                ("R", C.c_uint32), ("S", C.c_uint32), ("H", C.c_uint32)]


def build(force=False):
    """Compile the oracle with the Makefile next to it."""
    if force or not os.path.exists(_SO):
        subprocess.check_call(["make", "-C", _HERE, "-B" if force else "-s"],
                              stdout=subprocess.DEVNULL)
    return _SO


_lib = None


def lib():
    global _lib
    if _lib is not None:
        return _lib
    build()
    L = C.CDLL(_SO)
    u32, i32, vp = C.c_uint32, C.c_int, C.c_void_p
    PP = C.POINTER(Policy)
    L.orc_block_index.restype = u32
    L.orc_block_index.argtypes = [i32, Dim3, Dim3]
    L.orc_tile_to_block.restype = Dim3
    L.orc_tile_to_block.argtypes = [i32, Dim3]
    L.orc_tile_index.restype = u32
    L.orc_tile_index.argtypes = [i32, Dim3, Dim3]
    L.orc_build_schedule.restype = i32
    L.orc_build_schedule.argtypes = [i32, Dim3, vp]
    for name in ("wait_value", "post_value", "tile_index"):
        f = getattr(L, "orc_policy_" + name)
        f.restype = u32
        f.argtypes = [PP, Dim3, Dim3]
    L.orc_policy_is_sync.restype = i32
    L.orc_policy_is_sync.argtypes = [PP, Dim3, Dim3]
    L.orc_expected_sems_gemm.restype = None
    L.orc_expected_sems_gemm.argtypes = [PP, Dim3, u32, u32, i32, i32, vp]
    L.orc_expected_sems_blocks.restype = None
    L.orc_expected_sems_blocks.argtypes = [PP, Dim3, i32, i32, vp]
    L.orc_replay_chain.restype = i32
    L.orc_replay_chain.argtypes = [PP, Dim3, Dim3, u32, u32, u32, u32, u32, i32, i32, i32, i32, vp]
    L.orc_h2f.restype = C.c_float
    L.orc_h2f.argtypes = [C.c_uint16]
    L.orc_f2h.restype = C.c_uint16
    L.orc_f2h.argtypes = [C.c_float]
    L.orc_h2f_array.argtypes = [vp, vp, C.c_size_t]
    L.orc_f2h_array.argtypes = [vp, vp, C.c_size_t]
    L.orc_gelu.restype = C.c_float
    L.orc_gelu.argtypes = [C.c_float]
    L.orc_silu.restype = C.c_float
    L.orc_silu.argtypes = [C.c_float]
    L.orc_gemm_f16.restype = None
    L.orc_gemm_f16.argtypes = [u32, u32, u32, vp, u32, vp, u32, vp, u32, i32]
    L.orc_swiglu_f16.restype = None
    L.orc_swiglu_f16.argtypes = [u32, u32, vp, u32, vp, u32]
    L.orc_gemm_swiglu_f16.restype = None
    L.orc_gemm_swiglu_f16.argtypes = [u32, u32, u32, vp, u32, vp, u32, vp, u32]
    L.orc_attention_f16.restype = None
    L.orc_attention_f16.argtypes = [u32, u32, u32, vp, u32, vp, u32, i32]
    L.orc_attention_kv_f16.restype = None
    L.orc_attention_kv_f16.argtypes = [u32, u32, u32, u32, vp, u32, vp, u32, i32]
    L.orc_conv2d_nhwc_f16.restype = None
    L.orc_conv2d_nhwc_f16.argtypes = [u32] * 9 + [vp, vp, vp, i32]
    L.orc_equals_f16.restype = i32
    L.orc_equals_f16.argtypes = [C.c_size_t, vp, vp, C.c_float]
    L.orc_count_mismatch_f16.restype = C.c_size_t
    L.orc_count_mismatch_f16.argtypes = [C.c_size_t, vp, vp, C.c_float, C.c_float, C.POINTER(C.c_float)]
    L.orc_num_threads.restype = i32
    _lib = L
    return L


def d3(t):
    t = tuple(t) + (0,) * (3 - len(t))
    return Dim3(*[int(v) for v in t])


def policy(kind, order=ORDER_TRANSPOSE_XY, tileM=1, tileN=1, waitValue=None, postValue=None,
           gridN=0, stride=0, R=1, S=1, H=0):
    """Mirrors the constructors' defaults: RowSync() -> 0/0, RowSync(w) -> w/1
    (CS/policies.h:49-60); TileSync()/Conv2DTileSync() -> 1/1 (:109, :169)."""
    if waitValue is None:
        waitValue = 0 if kind == ROWSYNC else 1
    if postValue is None:
        postValue = 1 if (kind != ROWSYNC or waitValue) else 0
    return Policy(kind, order, tileM, tileN, waitValue, postValue, gridN, stride, R, S, H)


def _ptr(a):
    return a.ctypes.data_as(C.c_void_p)


def block_index(order, grid, block):
    return lib().orc_block_index(order, d3(grid), d3(block))


def tile_to_block(order, tile):
    return lib().orc_tile_to_block(order, d3(tile)).tup()


def tile_index(order, tile, grid):
    return lib().orc_tile_index(order, d3(tile), d3(grid))


def build_schedule(order, grid):
    g = d3(grid)
    n = g.x * g.y * g.z
    out = np.zeros((n, 3), dtype=np.uint32)
    rc = lib().orc_build_schedule(order, g, _ptr(out))
    return rc, out


def policy_wait_value(p, tile, grid):
    return lib().orc_policy_wait_value(C.byref(p), d3(tile), d3(grid))


def policy_post_value(p, tile, grid):
    return lib().orc_policy_post_value(C.byref(p), d3(tile), d3(grid))


def policy_tile_index(p, tile, grid):
    return lib().orc_policy_tile_index(C.byref(p), d3(tile), d3(grid))


def policy_is_sync(p, tile, grid):
    return bool(lib().orc_policy_is_sync(C.byref(p), d3(tile), d3(grid)))


def expected_sems_gemm(p, grid, kernel_tile_m, kernel_tile_n, iters, opts=0):
    g = d3(grid)
    out = np.zeros(g.x * g.y * g.z, dtype=np.uint32)
    lib().orc_expected_sems_gemm(C.byref(p), g, kernel_tile_m, kernel_tile_n, iters, opts, _ptr(out))
    return out


def expected_sems_blocks(p, grid, iters, opts=0):
    g = d3(grid)
    out = np.zeros(g.x * g.y * g.z, dtype=np.uint32)
    lib().orc_expected_sems_blocks(C.byref(p), g, iters, opts, _ptr(out))
    return out


def replay_chain(p, prod_grid, cons_grid, prod_tile, cons_tile_m, cons_tile_k, cons_k,
                 prod_slots, cons_slots, iters=1, opts=0):
    pg = d3(prod_grid)
    out = np.zeros(pg.x * pg.y * pg.z, dtype=np.uint32)
    ok = lib().orc_replay_chain(C.byref(p), pg, d3(cons_grid), prod_tile[0], prod_tile[1],
                                cons_tile_m, cons_tile_k, cons_k, prod_slots, cons_slots,
                                iters, opts, _ptr(out))
    return bool(ok), out


def _h(a):
    a = np.ascontiguousarray(a)
    if a.dtype == np.float16:
        return a.view(np.uint16)
    assert a.dtype == np.uint16
    return a


def h2f(bits):
    bits = np.ascontiguousarray(bits, dtype=np.uint16)
    out = np.empty(bits.shape, dtype=np.float32)
    lib().orc_h2f_array(_ptr(bits), _ptr(out), bits.size)
    return out


def f2h(vals):
    vals = np.ascontiguousarray(vals, dtype=np.float32)
    out = np.empty(vals.shape, dtype=np.uint16)
    lib().orc_f2h_array(_ptr(vals), _ptr(out), vals.size)
    return out


def gemm(a, b, epilogue=EPI_NONE):
    """C[M,N] = epilogue(A[M,K] @ B[K,N]); fp16 arrays in, fp16 array out."""
    a, b = _h(a), _h(b)
    M, K = a.shape
    K2, N = b.shape
    assert K == K2
    c = np.empty((M, N), dtype=np.uint16)
    lib().orc_gemm_f16(M, N, K, _ptr(a), K, _ptr(b), N, _ptr(c), N, epilogue)
    return c.view(np.float16)


def swiglu(gu, d):
    gu = _h(gu)
    M, ld = gu.shape
    h = np.empty((M, d), dtype=np.uint16)
    lib().orc_swiglu_f16(M, d, _ptr(gu), ld, _ptr(h), d)
    return h.view(np.float16)


def gemm_swiglu(a, w, d):
    """H[M,d] = silu(A @ W[:, :d]) * (A @ W[:, d:]) with the activation applied to the fp32 accumulators."""
    a, w = _h(a), _h(w)
    M, K = a.shape
    assert w.shape == (K, 2 * d)
    h = np.empty((M, d), dtype=np.uint16)
    lib().orc_gemm_swiglu_f16(M, d, K, _ptr(a), K, _ptr(w), 2 * d, _ptr(h), d)
    return h.view(np.float16)


def attention(qkv, heads, hd, causal=True):
    qkv = _h(qkv)
    S, ld = qkv.shape
    out = np.empty((S, heads * hd), dtype=np.uint16)
    lib().orc_attention_f16(S, heads, hd, _ptr(qkv), ld, _ptr(out), heads * hd, int(causal))
    return out.view(np.float16)


def attention_kv(qkv, cached, heads, hd, causal=True):
    """Attention of the rows behind `cached` cache rows over all rows of qkv ([cached + S, 3*heads*hd])."""
    qkv = _h(qkv)
    total, ld = qkv.shape
    S = total - cached
    out = np.empty((S, heads * hd), dtype=np.uint16)
    lib().orc_attention_kv_f16(S, cached, heads, hd, _ptr(qkv), ld, _ptr(out), heads * hd, int(causal))
    return out.view(np.float16)


def conv2d_nhwc(x, w, pad=1, stride=1, epilogue=EPI_NONE):
    x, w = _h(x), _h(w)
    N, H, W, Cc = x.shape
    K, R, S, C2 = w.shape
    assert Cc == C2
    P = (H + 2 * pad - R) // stride + 1
    Q = (W + 2 * pad - S) // stride + 1
    y = np.empty((N, P, Q, K), dtype=np.uint16)
    lib().orc_conv2d_nhwc_f16(N, H, W, Cc, K, R, S, pad, stride, _ptr(x), _ptr(w), _ptr(y), epilogue)
    return y.view(np.float16)


def equals(a, b, tol):
    a, b = _h(a), _h(b)
    return bool(lib().orc_equals_f16(a.size, _ptr(a), _ptr(b), tol))


def count_mismatch(a, ref, rel_tol=1e-2, abs_tol=1e-3):
    a, ref = _h(a), _h(ref)
    assert a.shape == ref.shape
    mx = C.c_float(0)
    bad = lib().orc_count_mismatch_f16(a.size, _ptr(a), _ptr(ref), rel_tol, abs_tol, C.byref(mx))
    return int(bad), float(mx.value)


def num_threads():
    return lib().orc_num_threads()
