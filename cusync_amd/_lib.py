"""ctypes binding of ``libcusync_amd.so`` (the C ABI in ``include/cusync_amd.h``).

The library is loaded from ``cusync_amd/lib/`` inside the source tree; there is
no fallback: if it has not been built (``python -c "import __graft_entry__ as g;
g.build()"`` or ``make -C cusync_amd/csrc``) loading raises.
"""
import ctypes as C
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_DIR = os.path.join(_HERE, "lib")
LIB_PATH = os.path.join(LIB_DIR, "libcusync_amd.so")
TEST_LIB_PATH = os.path.join(LIB_DIR, "libcusync_stage_tests.so")

u32, i32, vp, sz = C.c_uint32, C.c_int32, C.c_void_p, C.c_size_t


class Dim3(C.Structure):
    _fields_ = [("x", u32), ("y", u32), ("z", u32)]

    def tup(self):
        return (self.x, self.y, self.z)


class PolicyDesc(C.Structure):
    _fields_ = [("kind", i32), ("order", i32), ("tileM", u32), ("tileN", u32),
                ("waitValue", u32), ("postValue", u32), ("gridN", u32), ("stride", u32),
                ("R", u32), ("S", u32), ("H", u32)]


class StageDesc(C.Structure):
    _fields_ = [("grid", Dim3), ("prodGrid", Dim3), ("tileSize", Dim3),
                ("iter", i32), ("opts", i32), ("flags", u32), ("reserved", u32), ("in_", PolicyDesc), ("out", PolicyDesc),
                ("tileOrder", vp), ("tileCounter", vp), ("startCounter", vp), ("xcdTickets", vp),
                ("kernelExecuted", vp), ("spinTimeouts", vp),
                ("tileStatusWrite", vp), ("tileStatusRead", vp)]


class GemmArgs(C.Structure):
    _fields_ = [("stage", StageDesc), ("M", u32), ("N", u32), ("K", u32),
                ("A", vp), ("lda", u32), ("B", vp), ("ldb", u32), ("D", vp), ("ldd", u32),
                ("epilogue", i32), ("a_mode", i32), ("tile", i32), ("split_k", i32),
                ("workspace", vp), ("max_workgroups", i32), ("shared_reduction", i32)]


class Conv2dArgs(C.Structure):
    _fields_ = [("stage", StageDesc), ("N", u32), ("H", u32), ("W", u32), ("C", u32), ("K", u32), ("R", u32), ("S", u32),
                ("pad", u32), ("stride", u32), ("x", vp), ("w", vp), ("y", vp),
                ("epilogue", i32), ("tile", i32), ("max_workgroups", i32), ("split_k", i32), ("workspace", vp)]


class ConvChainConfig(C.Structure):
    _fields_ = [("N", u32), ("H", u32), ("W", u32), ("C", u32), ("layers", u32), ("sync", i32), ("tile", i32),
                ("opts", i32), ("relu", i32), ("fused", i32), ("split_k", i32)]


class AttentionArgs(C.Structure):
    _fields_ = [("stage", StageDesc), ("seq", u32), ("heads", u32), ("head_dim", u32), ("cached_rows", u32), ("qkv", vp), ("ldqkv", u32),
                ("out", vp), ("ldo", u32), ("scale", C.c_float), ("causal", i32), ("max_workgroups", i32),
                ("kv_split_blocks", u32), ("workspace", vp)]


class AttnLayerConfig(C.Structure):
    _fields_ = [("seq", u32), ("hidden", u32), ("heads", u32), ("head_dim", u32), ("sync", i32),
                ("tile1", i32), ("tile3", i32), ("opts", i32), ("causal", i32), ("cached_rows", u32), ("kv_split_blocks", i32)]


class MlpConfig(C.Structure):
    _fields_ = [("model", i32), ("batch", u32), ("hidden", u32), ("inner", u32), ("sync", i32),
                ("tile1", i32), ("tile2", i32), ("opts", i32), ("activation", i32),
                ("split_k1", i32), ("split_k2", i32), ("max_wg1", i32), ("max_wg2", i32), ("one_launch", i32), ("swiglu_in_gemm2", i32), ("repack_weights", i32)]


# every symbol include/cusync_amd.h declares: name -> (restype, argtypes)
SIGNATURES = {
    "cusync_rt_last_error": (C.c_char_p, []),
    "cusync_rt_set_timeline": (C.c_int, [vp, sz]),
    "cusync_rt_device_count": (C.c_int, []),
    "cusync_rt_device_info": (C.c_int, [C.POINTER(C.c_int), C.POINTER(C.c_int), C.POINTER(sz), C.POINTER(sz), C.c_char_p, sz]),
    "cusync_rt_malloc": (C.c_int, [C.POINTER(vp), sz]),
    "cusync_rt_free": (C.c_int, [vp]),
    "cusync_rt_memset": (C.c_int, [vp, C.c_int, sz]),
    "cusync_rt_memcpy_h2d": (C.c_int, [vp, vp, sz]),
    "cusync_rt_memcpy_d2h": (C.c_int, [vp, vp, sz]),
    "cusync_rt_memcpy_d2d": (C.c_int, [vp, vp, sz]),
    "cusync_rt_stream_create": (C.c_int, [C.POINTER(vp)]),
    "cusync_rt_stream_destroy": (C.c_int, [vp]),
    "cusync_rt_stream_sync": (C.c_int, [vp]),
    "cusync_rt_device_sync": (C.c_int, []),
    "cusync_rt_event_create": (C.c_int, [C.POINTER(vp)]),
    "cusync_rt_event_destroy": (C.c_int, [vp]),
    "cusync_rt_event_record": (C.c_int, [vp, vp]),
    "cusync_rt_event_sync": (C.c_int, [vp]),
    "cusync_rt_event_elapsed_us": (C.c_int, [vp, vp, C.POINTER(C.c_double)]),
    "cusync_rt_stream_wait_event": (C.c_int, [vp, vp]),
    "cusync_stage_alloc": (C.c_int, [C.POINTER(StageDesc), vp]),
    "cusync_stage_free": (C.c_int, [C.POINTER(StageDesc)]),
    "cusync_stage_create": (C.c_int, [C.POINTER(StageDesc), C.c_int]),
    "cusync_set_producer_consumer_pair": (C.c_int, [C.POINTER(StageDesc), C.POINTER(StageDesc)]),
    "cusync_invoke_wait_kernel": (C.c_int, [C.POINTER(StageDesc), vp]),
    "cusync_invoke_wait_kernel_after": (C.c_int, [C.POINTER(StageDesc), vp, vp]),
    "cusync_wait_producer_started": (C.c_int, [C.POINTER(StageDesc), u32]),
    "cusync_hold_back": (C.c_int, [C.POINTER(StageDesc), vp]),
    "cusync_wait_kernel": (C.c_int, [vp, u32, vp]),
    "cusync_stage_read_state": (C.c_int, [C.POINTER(StageDesc), vp, vp, C.POINTER(u32), C.POINTER(u32), C.POINTER(u32), C.POINTER(u32)]),
    "cusync_policy_tile_index": (u32, [C.POINTER(PolicyDesc), Dim3, Dim3]),
    "cusync_policy_wait_value": (u32, [C.POINTER(PolicyDesc), Dim3, Dim3]),
    "cusync_policy_post_value": (u32, [C.POINTER(PolicyDesc), Dim3, Dim3]),
    "cusync_policy_is_sync": (C.c_int, [C.POINTER(PolicyDesc), Dim3, Dim3]),
    "cusync_order_block_index": (u32, [C.c_int, Dim3, Dim3]),
    "cusync_order_tile_to_block": (Dim3, [C.c_int, Dim3]),
    "cusync_gemm_tile_shape": (C.c_int, [C.c_int, C.POINTER(u32), C.POINTER(u32), C.POINTER(u32)]),
    "cusync_gemm_grid": (Dim3, [C.c_int, u32, u32, C.c_int]),
    "cusync_gemm_can_implement": (C.c_int, [C.POINTER(GemmArgs)]),
    "cusync_gemm_workspace_size": (sz, [C.POINTER(GemmArgs)]),
    "cusync_gemm_max_resident": (C.c_int, [C.c_int]),
    "cusync_gemm_fills_device": (C.c_int, [C.POINTER(GemmArgs)]),
    "cusync_gemm_chain_run": (C.c_int, [C.POINTER(GemmArgs), C.c_int, vp]),
    "cusync_gemm_run": (C.c_int, [C.POINTER(GemmArgs), vp]),
    "cusync_gemm_run_static_workspace": (C.c_int, [C.POINTER(GemmArgs), vp]),
    "cusync_conv2d_tile_shape": (C.c_int, [C.c_int, C.POINTER(u32), C.POINTER(u32), C.POINTER(u32)]),
    "cusync_conv2d_grid": (Dim3, [C.c_int, u32, u32, u32, u32, u32, u32, u32, u32]),
    "cusync_conv2d_grid_split": (Dim3, [C.c_int, u32, u32, u32, u32, u32, u32, u32, u32, C.c_int]),
    "cusync_conv2d_workspace_size": (sz, [C.POINTER(Conv2dArgs)]),
    "cusync_conv2d_can_implement": (C.c_int, [C.POINTER(Conv2dArgs)]),
    "cusync_conv2d_max_resident": (C.c_int, [C.c_int]),
    "cusync_conv2d_run": (C.c_int, [C.POINTER(Conv2dArgs), vp]),
    "cusync_conv_chain_create": (vp, [C.POINTER(ConvChainConfig), C.POINTER(vp)]),
    "cusync_conv_chain_destroy": (None, [vp]),
    "cusync_conv_chain_run": (C.c_int, [vp, vp, C.POINTER(vp), C.c_int, C.POINTER(C.c_double), C.POINTER(C.c_double)]),
    "cusync_conv_chain_stage": (C.POINTER(StageDesc), [vp, u32]),
    "cusync_conv_chain_tile": (C.c_int, [vp]),
    "cusync_conv_chain_split": (C.c_int, [vp]),
    "cusync_attention_tile_shape": (C.c_int, [C.POINTER(u32), C.POINTER(u32), C.POINTER(u32)]),
    "cusync_attention_grid": (Dim3, [u32, u32]),
    "cusync_attention_grid_split": (Dim3, [u32, u32, u32, u32]),
    "cusync_attention_workspace_size": (sz, [C.POINTER(AttentionArgs)]),
    "cusync_attention_can_implement": (C.c_int, [C.POINTER(AttentionArgs)]),
    "cusync_attention_max_resident": (C.c_int, []),
    "cusync_attention_run": (C.c_int, [C.POINTER(AttentionArgs), vp]),
    "cusync_attn_layer_create": (vp, [C.POINTER(AttnLayerConfig), vp, vp]),
    "cusync_attn_layer_destroy": (None, [vp]),
    "cusync_attn_layer_run": (C.c_int, [vp, vp, vp, vp, vp, C.c_int, C.POINTER(C.c_double), C.POINTER(C.c_double)]),
    "cusync_attn_layer_stage": (C.POINTER(StageDesc), [vp, C.c_int]),
    "cusync_attn_layer_tiles": (C.c_int, [vp, C.POINTER(C.c_int), C.POINTER(C.c_int)]),
    "cusync_sync_overhead_pair": (C.c_int, [u32, u32, C.c_int, C.c_int, C.POINTER(C.c_double), C.POINTER(C.c_double)]),
    "cusync_sync_overhead_bare": (C.c_int, [u32, u32, C.c_int, C.c_int, C.POINTER(C.c_double), C.POINTER(C.c_double)]),
    "cusync_sync_overhead_pingpong": (C.c_int, [u32, u32, C.POINTER(C.c_double)]),
    "cusync_probe_mfma_rate": (C.c_int, [C.c_int, u32, C.c_int, C.POINTER(C.c_double), C.POINTER(C.c_double)]),
    "cusync_mlp_create": (vp, [C.POINTER(MlpConfig), vp, vp]),
    "cusync_mlp_destroy": (None, [vp]),
    "cusync_mlp_reload_weights": (C.c_int, [vp]),
    "cusync_mlp_run": (C.c_int, [vp, vp, vp, vp, C.c_int, C.POINTER(C.c_double)]),
    "cusync_mlp_run_split": (C.c_int, [vp, vp, vp, vp, C.c_int, C.POINTER(C.c_double), C.POINTER(C.c_double), C.POINTER(C.c_double)]),
    "cusync_mlp_stage": (C.POINTER(StageDesc), [vp, C.c_int]),
    "cusync_mlp_tiles": (C.c_int, [vp, C.POINTER(C.c_int), C.POINTER(C.c_int)]),
    "cusync_mlp_splits": (C.c_int, [vp, C.POINTER(C.c_int), C.POINTER(C.c_int)]),
    "cusync_mlp_choice": (C.c_int, [C.POINTER(MlpConfig)] + [C.POINTER(C.c_int)] * 5),
}

_lib = None


def load():
    """Load the C-ABI library and attach prototypes.  Raises if it is not built."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise RuntimeError(
            "cusync_amd: %s is missing — the HIP library has not been built "
            "(run `make -C cusync_amd/csrc` or __graft_entry__.build()). "
            "There is no CPU fallback." % LIB_PATH)
    # PyTorch ships a HIP runtime of its own.  Whichever copy is loaded first serves the whole process, and the
    # tensors handed to this library come from PyTorch's: let it load first (measured the other way round: the
    # occupancy query answers 0 workgroups per CU for every kernel that needs more than 64 KB of LDS).
    try:
        import torch  # noqa: F401
    except ImportError:
        pass
    L = C.CDLL(LIB_PATH, mode=C.RTLD_GLOBAL)
    for name, (res, args) in SIGNATURES.items():
        f = getattr(L, name)          # AttributeError if the symbol is not exported
        f.restype = res
        f.argtypes = args
    _lib = L
    return L


def load_stage_tests():
    load()
    if not os.path.exists(TEST_LIB_PATH):
        raise RuntimeError("cusync_amd: %s is missing — build it first" % TEST_LIB_PATH)
    return C.CDLL(TEST_LIB_PATH)
