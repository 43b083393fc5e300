"""Python mirror of the host-side CuSync interface, bound to the C ABI.

Names follow the reference's C++ API (CuStage, setProducerConsumerPair,
invokeWaitKernel, incrementIter; src/include/cusync/cusync.h:87-299) so that the
parity tests read like the reference's own tests.  Nothing here computes on the
CPU: every operation is a call into ``libcusync_amd.so``.
"""
import ctypes as C
from types import SimpleNamespace

from . import _lib
from ._lib import AttentionArgs, AttnLayerConfig, Conv2dArgs, ConvChainConfig, Dim3, GemmArgs, MlpConfig, PolicyDesc, StageDesc

ERR = SimpleNamespace(NOT_PRODUCER=0, NOT_CONSUMER=1, NOT_INITIALIZED=2,
                      INVALID_LINEAR_BLOCK_INDEX=3, DEVICE=4, SUCCESS=5)
OPT = SimpleNamespace(NONE=0, NO_ATOMIC_ADD=1, AVOID_WAIT_KERNEL=2, AVOID_CUSTOM_ORDER=4, REORDER_TILE_LOADS=8)
ORDER = SimpleNamespace(IDENTITY=0, TRANSPOSE_XY=1)
POLICY = SimpleNamespace(NOSYNC=0, ROWSYNC=1, TILESYNC=2, STRIDEDSYNC=3, CONV2DTILESYNC=4, CONSECUTIVESYNC=5)
EPI = SimpleNamespace(NONE=0, GELU=1, RELU=2, SWIGLU=3)
TILE = SimpleNamespace(T256x256x32=0, T256x128x64=1, T128x128x64=2, T64x128x64=3, T32x128x64=4,
                       T128x256x64=5, T256x64x64=6, T128x64x64=7, T256x128x32=8, T128x256x32=9, T128x128x32=10,
                       T128x192x32=11, T256x192x32=12, D32x128x64=13, D64x128x64=14, D64x192x64=15, T128x192x32_ALONE=16, T256x384x32=17, T256x192x64=18, D128x192x64=19, COUNT=20)
CONV_TILE = SimpleNamespace(T128x64x32=0, T128x128x32=1, T256x64x32=2, HALO_256x64x64=3, HALO_128x128x64=4, HALO_64x128x64=5, COUNT=6)
SYNC = SimpleNamespace(STREAM=0, ROW=1, TILE=2, STRIDED=3)
MODEL = SimpleNamespace(GPT3=0, LLAMA=1)


class CuSyncError(RuntimeError):
    def __init__(self, code, what=""):
        self.code = code
        super().__init__("%s: cusync error %d (%s)" % (what, code, last_error()))


def last_error():
    return _lib.load().cusync_rt_last_error().decode()


def check(code, what=""):
    if code != ERR.SUCCESS:
        raise CuSyncError(code, what)


def d3(t):
    t = tuple(int(v) for v in t) + (0,) * (3 - len(t))
    return Dim3(*t)


def device_info():
    L = _lib.load()
    cus, clk = C.c_int(0), C.c_int(0)
    lds, hbm = C.c_size_t(0), C.c_size_t(0)
    name = C.create_string_buffer(128)
    if L.cusync_rt_device_info(C.byref(cus), C.byref(clk), C.byref(lds), C.byref(hbm), name, 128):
        raise RuntimeError(last_error())
    return dict(cus=cus.value, clock_khz=clk.value, lds_per_cu=lds.value, hbm_bytes=hbm.value, arch=name.value.decode())


# ---- policies ------------------------------------------------------------------

def policy_desc(kind, order=ORDER.TRANSPOSE_XY, tileM=1, tileN=1, waitValue=0, postValue=0,
                gridN=0, stride=0, R=1, S=1, H=0):
    return PolicyDesc(kind, order, tileM, tileN, waitValue, postValue, gridN, stride, R, S, H)


def no_sync():
    return policy_desc(POLICY.NOSYNC)


def row_sync(tileM, waitValue=0, postValue=None):
    if postValue is None:
        postValue = 1 if waitValue else 0
    return policy_desc(POLICY.ROWSYNC, ORDER.TRANSPOSE_XY, tileM, 1, waitValue, postValue)


def tile_sync(order, tileM, tileN, waitValue=1, postValue=1):
    return policy_desc(POLICY.TILESYNC, order, tileM, tileN, waitValue, postValue)


def strided_sync(order, gridN, tileM, tileN, stride):
    return policy_desc(POLICY.STRIDEDSYNC, order, tileM, tileN, stride, 1, gridN=gridN, stride=stride)


def conv2d_tile_sync(order, R, S, tileM, tileN, waitValue=1, postValue=1):
    return policy_desc(POLICY.CONV2DTILESYNC, order, tileM, tileN, waitValue, postValue, R=R, S=S)


def consecutive_sync(order, H, tileM, tileN):
    return policy_desc(POLICY.CONSECUTIVESYNC, order, tileM, tileN, (H // 8) // tileN, 1, H=H)


def policy_tile_index(p, tile, grid):
    return _lib.load().cusync_policy_tile_index(C.byref(p), d3(tile), d3(grid))


def policy_wait_value(p, tile=(0, 0, 0), grid=(1, 1, 1)):
    return _lib.load().cusync_policy_wait_value(C.byref(p), d3(tile), d3(grid))


def policy_post_value(p, tile=(0, 0, 0), grid=(1, 1, 1)):
    return _lib.load().cusync_policy_post_value(C.byref(p), d3(tile), d3(grid))


def policy_is_sync(p, tile, grid=(1, 1, 1)):
    return bool(_lib.load().cusync_policy_is_sync(C.byref(p), d3(tile), d3(grid)))


# ---- stages ----------------------------------------------------------------------

class Stage:
    """CuStage<TileOrder, InputSyncPolicy, OutputSyncPolicy, Opts> (run-time form)."""

    def __init__(self, grid, tile_size, input_policy, output_policy, order=ORDER.TRANSPOSE_XY, opts=OPT.NONE):
        self.L = _lib.load()
        self.order = order
        self.desc = StageDesc()
        self.desc.grid = d3(grid)
        self.desc.tileSize = d3(tile_size)
        self.desc.iter = 1
        self.desc.opts = opts
        self.desc.in_ = input_policy
        self.desc.out = output_policy
        self.status = self.L.cusync_stage_create(C.byref(self.desc), order)
        if self.status not in (ERR.SUCCESS, ERR.INVALID_LINEAR_BLOCK_INDEX):
            raise CuSyncError(self.status, "cusync_stage_create")
        self._alive = True

    def grid(self):
        return self.desc.grid.tup()

    def isProducer(self):
        return self.desc.out.kind != POLICY.NOSYNC

    def isConsumer(self):
        return self.desc.in_.kind != POLICY.NOSYNC

    def numTiles(self):
        g = self.desc.grid
        return g.x * g.y * g.z

    def invokeWaitKernel(self, stream, after=None):
        """`after`: an event recorded on the producer's stream right before the
        producer's launch; the wait kernel is then dispatched behind it."""
        if after is not None:
            return self.L.cusync_invoke_wait_kernel_after(C.byref(self.desc), stream, after)
        return self.L.cusync_invoke_wait_kernel(C.byref(self.desc), stream)

    def incrementIter(self):
        self.desc.iter += 1

    def read_state(self):
        import numpy as np
        n = self.numTiles()
        sems = np.zeros(n, np.uint32)
        order = np.zeros((n, 3), np.uint32)
        tc, sc, ke, to = C.c_uint32(0), C.c_uint32(0), C.c_uint32(0), C.c_uint32(0)
        check(self.L.cusync_stage_read_state(
            C.byref(self.desc), sems.ctypes.data_as(C.c_void_p) if self.isProducer() else None,
            order.ctypes.data_as(C.c_void_p), C.byref(tc), C.byref(sc), C.byref(ke), C.byref(to)), "read_state")
        return SimpleNamespace(sems=sems, tile_order=order, tile_counter=tc.value, start_counter=sc.value,
                               kernel_executed=ke.value, spin_timeouts=to.value)

    def destroy(self):
        if self._alive:
            self.L.cusync_stage_free(C.byref(self.desc))
            self._alive = False


def set_producer_consumer_pair(prod, cons):
    """CuSync::setProducerConsumerPair; returns the CuSyncError code."""
    return _lib.load().cusync_set_producer_consumer_pair(C.byref(prod.desc), C.byref(cons.desc))


# ---- GEMM ------------------------------------------------------------------------

def tile_shape(tile):
    m, n, k = C.c_uint32(0), C.c_uint32(0), C.c_uint32(0)
    if _lib.load().cusync_gemm_tile_shape(tile, C.byref(m), C.byref(n), C.byref(k)):
        raise ValueError("unknown tile id %r" % (tile,))
    return m.value, n.value, k.value


def gemm_grid(tile, M, N, split_k=1):
    return _lib.load().cusync_gemm_grid(tile, M, N, split_k).tup()


def gemm_args(stage, M, N, K, A, lda, B, ldb, D, ldd, tile, epilogue=EPI.NONE, a_mode=0, split_k=1,
              max_workgroups=0, workspace=None, shared_reduction=0):
    a = GemmArgs()
    a.stage = stage.desc
    a.M, a.N, a.K = M, N, K
    a.A, a.lda, a.B, a.ldb, a.D, a.ldd = A, lda, B, ldb, D, ldd
    a.epilogue, a.a_mode, a.tile, a.split_k = epilogue, a_mode, tile, split_k
    a.workspace = workspace
    a.max_workgroups = max_workgroups
    a.shared_reduction = shared_reduction
    return a


def gemm(stage, M, N, K, A, lda, B, ldb, D, ldd, tile, stream=None, **kw):
    """Launch one sync-aware GEMM; pointers are raw device addresses."""
    a = gemm_args(stage, M, N, K, A, lda, B, ldb, D, ldd, tile, **kw)
    return _lib.load().cusync_gemm_run(C.byref(a), stream)


# ---- convolution -------------------------------------------------------------------

def conv2d_tile_shape(tile):
    m, n, k = C.c_uint32(0), C.c_uint32(0), C.c_uint32(0)
    if _lib.load().cusync_conv2d_tile_shape(tile, C.byref(m), C.byref(n), C.byref(k)):
        raise ValueError("unknown conv tile id %r" % (tile,))
    return m.value, n.value, k.value


def conv2d_grid(tile, N, H, W, K, R=3, S=3, pad=1, stride=1, split_k=1):
    return _lib.load().cusync_conv2d_grid_split(tile, N, H, W, K, R, S, pad, stride, split_k).tup()


def conv2d_args(stage, N, H, W, Cc, K, x, w, y, tile, R=3, S=3, pad=1, stride=1, epilogue=EPI.NONE, max_workgroups=0,
                split_k=1, workspace=None):
    a = Conv2dArgs()
    a.stage = stage.desc
    a.N, a.H, a.W, a.C, a.K, a.R, a.S, a.pad, a.stride = N, H, W, Cc, K, R, S, pad, stride
    a.x, a.w, a.y = x, w, y
    a.epilogue, a.tile, a.max_workgroups = epilogue, tile, max_workgroups
    a.split_k, a.workspace = split_k, workspace
    return a


def conv2d_workspace_size(N, H, W, Cc, K, tile, split_k, R=3, S=3, pad=1, stride=1):
    a = Conv2dArgs()
    a.N, a.H, a.W, a.C, a.K, a.R, a.S, a.pad, a.stride = N, H, W, Cc, K, R, S, pad, stride
    a.tile, a.split_k = tile, split_k
    return _lib.load().cusync_conv2d_workspace_size(C.byref(a))


def conv2d(stage, N, H, W, Cc, K, x, w, y, tile, stream=None, **kw):
    a = conv2d_args(stage, N, H, W, Cc, K, x, w, y, tile, **kw)
    return _lib.load().cusync_conv2d_run(C.byref(a), stream)


class ConvChain:
    """Handle over cusync_conv_chain_*: `layers` dependent 3x3 convolutions, stream-ordered or one CuSync
    stage per layer (src/ml-bench/volta_conv2d/resnet.cu, vgg.cu)."""

    def __init__(self, N, H, W, Cc, weight_ptrs, sync, tile=-1, opts=-1, relu=True, fused=False, split_k=0):
        """split_k: runs a tile's steps are cut into (the reference's --split_k_slices); 1 = none, 0 = the library picks."""
        self.L = _lib.load()
        self.layers = len(weight_ptrs)
        self.cfg = ConvChainConfig(N, H, W, Cc, self.layers, sync, tile, opts, int(relu), int(fused), split_k)
        arr = (C.c_void_p * self.layers)(*weight_ptrs)
        self.h = self.L.cusync_conv_chain_create(C.byref(self.cfg), arr)
        if not self.h:
            raise RuntimeError("cusync_conv_chain_create failed: " + last_error())

    def run(self, x_ptr, y_ptrs, runs=1, layers=False):
        times = (C.c_double * runs)()
        per = (C.c_double * (runs * self.layers))()
        ys = (C.c_void_p * self.layers)(*y_ptrs)
        check(self.L.cusync_conv_chain_run(self.h, x_ptr, ys, runs, times, per), "cusync_conv_chain_run")
        if layers:
            return list(times), [list(per[r * self.layers:(r + 1) * self.layers]) for r in range(runs)]
        return list(times)

    def tile(self):
        return self.L.cusync_conv_chain_tile(self.h)

    def split(self):
        return self.L.cusync_conv_chain_split(self.h)

    def stage_state(self, which):
        return _read_stage(self.L, self.L.cusync_conv_chain_stage(self.h, which).contents)

    def destroy(self):
        if self.h:
            self.L.cusync_conv_chain_destroy(self.h)
            self.h = None


# ---- attention -------------------------------------------------------------------

def attention_tile_shape():
    m, n, k = C.c_uint32(0), C.c_uint32(0), C.c_uint32(0)
    _lib.load().cusync_attention_tile_shape(C.byref(m), C.byref(n), C.byref(k))
    return m.value, n.value, k.value


def attention_grid(seq, heads, cached_rows=0, kv_split_blocks=0):
    """(heads, row tiles, splits of the key range)."""
    return _lib.load().cusync_attention_grid_split(seq, heads, cached_rows, kv_split_blocks).tup()


def attention_args(stage, seq, heads, qkv, ldqkv, out, ldo, head_dim=128, scale=0.0, causal=True, max_workgroups=0, cached_rows=0,
                   kv_split_blocks=0, workspace=None):
    a = AttentionArgs()
    a.kv_split_blocks, a.workspace = kv_split_blocks, workspace
    a.stage = stage.desc
    a.seq, a.heads, a.head_dim, a.cached_rows = seq, heads, head_dim, cached_rows
    a.qkv, a.ldqkv, a.out, a.ldo = qkv, ldqkv, out, ldo
    a.scale, a.causal, a.max_workgroups = scale, int(causal), max_workgroups
    return a


def attention_workspace_size(seq, heads, cached_rows=0, kv_split_blocks=0):
    a = AttentionArgs()
    a.seq, a.heads, a.cached_rows, a.kv_split_blocks = seq, heads, cached_rows, kv_split_blocks
    return _lib.load().cusync_attention_workspace_size(C.byref(a))


def attention(stage, seq, heads, qkv, ldqkv, out, ldo, stream=None, **kw):
    a = attention_args(stage, seq, heads, qkv, ldqkv, out, ldo, **kw)
    return _lib.load().cusync_attention_run(C.byref(a), stream)


def _read_stage(L, d):
    import numpy as np
    d = type(d).from_buffer_copy(d)      # the descriptor lives inside the chain's handle: keep a copy that outlives it
    g = d.grid
    n = g.x * g.y * g.z
    sems = np.zeros(n, np.uint32)
    order = np.zeros((n, 3), np.uint32)
    tc, sc, ke, to = C.c_uint32(0), C.c_uint32(0), C.c_uint32(0), C.c_uint32(0)
    producer = d.out.kind != POLICY.NOSYNC
    check(L.cusync_stage_read_state(C.byref(d), sems.ctypes.data_as(C.c_void_p) if producer else None,
                                    order.ctypes.data_as(C.c_void_p), C.byref(tc), C.byref(sc),
                                    C.byref(ke), C.byref(to)), "read_state")
    return SimpleNamespace(desc=d, grid=g.tup(), sems=sems, tile_order=order, tile_counter=tc.value,
                           start_counter=sc.value, kernel_executed=ke.value, spin_timeouts=to.value)


class AttnLayer:
    """Handle over cusync_attn_layer_*: X Wqkv -> fused attention -> O Wo, stream-ordered or as three
    CuSync stages (the chain of src/ml-bench/transformer/attention.cu:702-830)."""

    def __init__(self, seq, hidden, heads, sync, wqkv_ptr, wo_ptr, head_dim=128, tile1=-1, tile3=-1, opts=-1, causal=True,
                 cached_rows=0, kv_split_blocks=-1):
        self.L = _lib.load()
        self.cfg = AttnLayerConfig(seq, hidden, heads, head_dim, sync, tile1, tile3, opts, int(causal), cached_rows, kv_split_blocks)
        self.h = self.L.cusync_attn_layer_create(C.byref(self.cfg), wqkv_ptr, wo_ptr)
        if not self.h:
            raise RuntimeError("cusync_attn_layer_create failed: " + last_error())

    def run(self, x_ptr, qkv_ptr, o_ptr, y_ptr, runs=1, stages=False):
        times = (C.c_double * runs)()
        per_stage = (C.c_double * (3 * runs))()
        check(self.L.cusync_attn_layer_run(self.h, x_ptr, qkv_ptr, o_ptr, y_ptr, runs, times, per_stage), "cusync_attn_layer_run")
        if stages:
            return list(times), [list(per_stage[3 * r:3 * r + 3]) for r in range(runs)]
        return list(times)

    def tiles(self):
        a, b = C.c_int(0), C.c_int(0)
        self.L.cusync_attn_layer_tiles(self.h, C.byref(a), C.byref(b))
        return a.value, b.value

    def stage_state(self, which):
        return _read_stage(self.L, self.L.cusync_attn_layer_stage(self.h, which).contents)

    def destroy(self):
        if self.h:
            self.L.cusync_attn_layer_destroy(self.h)
            self.h = None


# ---- cost of the synchronisation itself ---------------------------------------------

def sync_overhead_pair(blocks=1280, threads=128, warmup=10, iters=100):
    """(with_sync_us, without_sync_us) of the reference's sync-overhead example
    (src/examples/sync-overhead/sync-overhead.cu:70-104; its grid is 80*2*(1024/128) = 1280 blocks of 128)."""
    a, b = C.c_double(0), C.c_double(0)
    check(_lib.load().cusync_sync_overhead_pair(blocks, threads, warmup, iters, C.byref(a), C.byref(b)), "sync_overhead_pair")
    return a.value, b.value


def sync_overhead_bare(blocks=1280, threads=128, warmup=10, iters=100):
    """(with_flags_us, without_flags_us) of the same pair with the example's own kernels: a bare flag array, no fences,
    both kernels on one stream (src/examples/sync-overhead/sync-overhead.cu:40-59, 84-101)."""
    a, b = C.c_double(0), C.c_double(0)
    check(_lib.load().cusync_sync_overhead_bare(blocks, threads, warmup, iters, C.byref(a), C.byref(b)), "sync_overhead_bare")
    return a.value, b.value


def probe_mfma_rate(random_data=True, iters=2000, launches=10):
    """(TFLOP/s, shader clock in MHz) the matrix pipes sustain alone, on zero or random register operands."""
    t, f = C.c_double(0), C.c_double(0)
    check(_lib.load().cusync_probe_mfma_rate(1 if random_data else 0, iters, launches, C.byref(t), C.byref(f)), "probe_mfma_rate")
    return t.value, f.value


def sync_overhead_pingpong(partner, rounds=2000):
    """Nanoseconds per post -> wait -> post -> wait round trip between workgroup 0 and workgroup `partner`."""
    t = C.c_double(0)
    check(_lib.load().cusync_sync_overhead_pingpong(partner, rounds, C.byref(t)), "sync_overhead_pingpong")
    return t.value


# ---- MLP chain -------------------------------------------------------------------

class Mlp:
    """Handle over cusync_mlp_* (the reference's libmlp C surface, src/ml-bench/transformer/mlp-lib.cu:555-618)."""

    def __init__(self, model, batch, hidden, inner, sync, w1_ptr, w2_ptr, tile1=-1, tile2=-1, opts=-1, activation=1,
                 split_k1=0, split_k2=0, max_wg1=0, max_wg2=0, one_launch=-1, swiglu_in_gemm2=0, repack_weights=False):
        """one_launch: True / False, or -1 for the library's choice by model and batch size (see choice())."""
        self.L = _lib.load()
        self.cfg = MlpConfig(model, batch, hidden, inner, sync, tile1, tile2, opts, activation, split_k1, split_k2,
                             max_wg1, max_wg2, int(one_launch), int(swiglu_in_gemm2), int(repack_weights))
        self.h = self.L.cusync_mlp_create(C.byref(self.cfg), w1_ptr, w2_ptr)
        if not self.h:
            raise RuntimeError("cusync_mlp_create failed: " + last_error())

    def reload_weights(self):
        """With repack_weights: copies the caller's weights into the handle's padded buffers again."""
        return self.L.cusync_mlp_reload_weights(self.h)

    @classmethod
    def from_db(cls, entry, model, batch, hidden, inner, sync, w1_ptr, w2_ptr, activation=1):
        """Builds the chain from one entry of a tile table in the reference's schema
        (src/ml-bench/transformer/tile_sizes_db.py; cusync_amd/tile_sizes_db.py is written by cusync_amd.tuner)."""
        key = {SYNC.STREAM: "baseline", SYNC.ROW: "rowsync", SYNC.TILE: "tilesync", SYNC.STRIDED: "tilesync"}[sync]
        cfg = entry[key]
        opts = -1
        if key == "tilesync":
            opts = ((OPT.AVOID_CUSTOM_ORDER if cfg.get("AvoidCustomOrder") else 0) |
                    (OPT.AVOID_WAIT_KERNEL if cfg.get("AvoidWaitKernel") else 0) |
                    (OPT.REORDER_TILE_LOADS if cfg.get("ReorderTileLoads") else 0) |
                    (OPT.NO_ATOMIC_ADD if cfg.get("NoAtomicAdd") and sync == SYNC.TILE else 0))
        t1, t2 = entry["TileIds"]
        k1, k2 = cfg["split_ks"]
        return cls(model, batch, hidden, inner, sync, w1_ptr, w2_ptr, tile1=t1, tile2=t2, opts=opts,
                   activation=activation, split_k1=k1, split_k2=k2)

    def run(self, x_ptr, h_ptr, y_ptr, runs=1, split=False):
        times = (C.c_double * runs)()
        if split:
            g1 = (C.c_double * runs)()
            g2 = (C.c_double * runs)()
            check(self.L.cusync_mlp_run_split(self.h, x_ptr, h_ptr, y_ptr, runs, times, g1, g2), "cusync_mlp_run_split")
            return list(times), list(g1), list(g2)
        check(self.L.cusync_mlp_run(self.h, x_ptr, h_ptr, y_ptr, runs, times), "cusync_mlp_run")
        return list(times)

    def choice(self):
        """(tile1, tile2, split_k1, split_k2, one_launch) the tile table gives for this handle's configuration."""
        v = [C.c_int(-1) for _ in range(5)]
        if self.L.cusync_mlp_choice(C.byref(self.cfg), *[C.byref(x) for x in v]) != 0:
            raise RuntimeError("cusync_mlp_choice failed: " + last_error())
        return tuple(x.value for x in v)

    def tiles(self):
        a, b = C.c_int(0), C.c_int(0)
        self.L.cusync_mlp_tiles(self.h, C.byref(a), C.byref(b))
        return a.value, b.value

    def splits(self):
        a, b = C.c_int(0), C.c_int(0)
        self.L.cusync_mlp_splits(self.h, C.byref(a), C.byref(b))
        return a.value, b.value

    def stage_state(self, which):
        return _read_stage(self.L, self.L.cusync_mlp_stage(self.h, which).contents)

    def destroy(self):
        if self.h:
            self.L.cusync_mlp_destroy(self.h)
            self.h = None
