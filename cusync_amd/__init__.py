"""cusync_amd — MI355X-native CuSync.

The product is the C-ABI library ``libcusync_amd.so`` (``include/cusync_amd.h``)
and the C++ headers in ``include/cusync/``.  This Python package is a thin
ctypes front end used by the tests and the benchmark; device memory is owned by
the caller (torch tensors in the tests) and passed as raw pointers.
"""
from . import _lib
from .api import (  # noqa: F401
    ERR, OPT, ORDER, POLICY, EPI, TILE, CONV_TILE, SYNC, MODEL,
    CuSyncError, check, policy_desc, no_sync, row_sync, tile_sync, strided_sync,
    conv2d_tile_sync, consecutive_sync, Stage, set_producer_consumer_pair,
    gemm_grid, tile_shape, gemm, conv2d, conv2d_grid, conv2d_tile_shape, ConvChain, attention, attention_grid, attention_tile_shape, AttnLayer, Mlp, sync_overhead_pair, sync_overhead_pingpong, last_error, device_info,
)

__all__ = ["_lib", "Stage", "Mlp", "gemm"]
