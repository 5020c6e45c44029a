"""ctypes binding of libhsa_gfx950.so (the C ABI declared in include/hsa_gfx950.h).

There is no CPU or PyTorch fallback behind these calls: if the shared library has
not been built, importing the ops raises.
"""
from __future__ import annotations

import ctypes
import os
from ctypes import c_int, c_int64, c_void_p, c_char_p

import torch

HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(HERE, "libhsa_gfx950.so")

HSA_F32, HSA_F16, HSA_BF16 = 0, 1, 2
ATTN_AUTO, ATTN_GATHER, ATTN_TILE = 0, 1, 2
_ALGO = {"auto": ATTN_AUTO, "gather": ATTN_GATHER, "tile": ATTN_TILE}
_DTYPE = {torch.float32: HSA_F32, torch.float16: HSA_F16, torch.bfloat16: HSA_BF16}

_lib = None


class HsaError(RuntimeError):
    pass


def _declare(lib):
    P, I, I64 = c_void_p, c_int, c_int64
    lib.hsa_abi_version.restype = I
    lib.hsa_last_error.restype = c_char_p
    lib.hsa_attn_fwd.argtypes = [P, P, P, P, P, P, P] + [I] * 10 + [P]
    lib.hsa_attn_fwd.restype = I
    lib.hsa_attn_fwd_timed.argtypes = [P, P, P, P, P, P, P] + [I] * 10 + [P, P, P]
    lib.hsa_attn_fwd_timed.restype = I
    lib.hsa_cross_update_level_tune.argtypes = [I, ctypes.c_long]
    lib.hsa_cross_update_level_tune.restype = I
    lib.hsa_attn_bwd_tables.argtypes = [P] * 11 + [ctypes.c_size_t] + [I] * 9 + [P]
    lib.hsa_attn_bwd_tables.restype = I
    lib.hsa_attn_bwd_saved_tune.argtypes = [I]
    lib.hsa_attn_bwd_saved_tune.restype = I
    lib.hsa_attn_tile_tune.argtypes = [I] * 4
    lib.hsa_attn_tile_tune.restype = I
    lib.hsa_attn_fwd_uses_tile.argtypes = [I] * 9
    lib.hsa_attn_fwd_uses_tile.restype = I
    lib.hsa_build_parents_fwd.argtypes = [P] * 7 + [I] * 4 + [I64] * 6 + [I, P]
    lib.hsa_build_parents_fwd.restype = I
    lib.hsa_build_parents_strided_fwd.argtypes = [P] * 7 + [I] * 4 + [P, P, I, P]
    lib.hsa_build_parents_strided_fwd.restype = I
    lib.hsa_cross_update_top_tune.argtypes = [I]
    lib.hsa_cross_update_top_tune.restype = I
    lib.hsa_cross_update_level_rows.argtypes = [I, I, I, I]
    lib.hsa_cross_update_level_rows.restype = I
    lib.hsa_cross_update_top_rows.argtypes = [I, I, I]
    lib.hsa_cross_update_top_rows.restype = I
    lib.hsa_cross_update_pack_weights.argtypes = [P, P, P, I, I, I, P]
    lib.hsa_cross_update_pack_weights.restype = I
    lib.hsa_cross_update_top_fwd.argtypes = [P] * 4 + [I] * 4 + [I64] * 5 + [I, P]
    lib.hsa_cross_update_top_fwd.restype = I
    lib.hsa_build_tree_fwd.argtypes = [P] * 7 + [I] * 4 + [I64] * 7 + [I, P]
    lib.hsa_build_tree_fwd.restype = I
    lib.hsa_build_tree_tune.argtypes = [I, I]
    lib.hsa_build_tree_tune.restype = I
    lib.hsa_topology_host.argtypes = [I, I, P, P, P]
    lib.hsa_topology_host.restype = I
    lib.hsa_topology_device.argtypes = [I, I, P, P, P, P]
    lib.hsa_topology_device.restype = I
    lib.hsa_span_input_y.argtypes = [P, P, I, I, I, I, P]
    lib.hsa_span_input_y.restype = I
    lib.hsa_build_parents_bwd.argtypes = [P] * 11 + [I] * 5 + [P]
    lib.hsa_build_parents_bwd.restype = I
    lib.hsa_build_parents_strided_bwd.argtypes = [P] * 11 + [I] * 4 + [P, P, I, P]
    lib.hsa_build_parents_strided_bwd.restype = I
    lib.hsa_attn_fwd_lse.argtypes = [P] * 5 + [I] * 9 + [P]
    lib.hsa_attn_fwd_lse.restype = I
    lib.hsa_attn_bwd_saved_workspace_bytes.argtypes = [I] * 9
    lib.hsa_attn_bwd_saved_workspace_bytes.restype = ctypes.c_size_t
    lib.hsa_attn_bwd_saved.argtypes = [P] * 10 + [ctypes.c_size_t] + [I] * 9 + [P]
    lib.hsa_attn_bwd_saved.restype = I
    lib.hsa_attn_bwd_workspace_bytes.argtypes = [I] * 9
    lib.hsa_attn_bwd_workspace_bytes.restype = ctypes.c_size_t
    lib.hsa_attn_bwd.argtypes = [P] * 8 + [ctypes.c_size_t] + [I] * 10 + [P]
    lib.hsa_attn_bwd.restype = I
    lib.hsa_attn_bwd_static_capacity.argtypes = []
    lib.hsa_attn_bwd_static_capacity.restype = ctypes.c_size_t
    lib.hsa_attn_bwd_static.argtypes = [P] * 7 + [I] * 10 + [P]
    lib.hsa_attn_bwd_static.restype = I
    lib.hsa_span_input_y_bwd.argtypes = [P, P, I, I, I, I, P]
    lib.hsa_span_input_y_bwd.restype = I


def lib():
    """The loaded library; raises if it has not been built."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise HsaError(
                "libhsa_gfx950.so is missing (%s). Build it first: "
                "python -m sparseattention_amd._build" % LIB_PATH)
        handle = ctypes.CDLL(LIB_PATH)
        _declare(handle)
        _lib = handle
    return _lib


def check(rc: int, what: str):
    if rc != 0:
        msg = lib().hsa_last_error().decode("utf-8", "replace")
        raise HsaError("%s failed (%d): %s" % (what, rc, msg))


def dtype_code(t: torch.Tensor) -> int:
    try:
        return _DTYPE[t.dtype]
    except KeyError:
        raise AssertionError("unsupported dtype %s (float32, float16, bfloat16 only)" % t.dtype)


def algo_code(name: str) -> int:
    return _ALGO[name]


def ptr(t):
    return None if t is None else c_void_p(t.data_ptr())


def require_gpu(*tensors):
    for t in tensors:
        if t is not None and not t.is_cuda:
            raise HsaError("this op runs on the GPU only; got a %s tensor" % t.device)


_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)


def stream_of(t: torch.Tensor):
    """The current HIP stream of the tensor's device as a raw handle."""
    if _raw_stream is not None:
        return c_void_p(_raw_stream(t.device.index))
    return c_void_p(torch.cuda.current_stream(t.device).cuda_stream)


class _SameDevice:
    def __enter__(self):
        return None

    def __exit__(self, *exc):
        return False


_SAME_DEVICE = _SameDevice()


def on_device(t: torch.Tensor):
    """Context that makes the tensor's device the current one for the launches inside; free when
    it already is."""
    if t.device.index == torch.cuda.current_device():
        return _SAME_DEVICE
    return torch.cuda.device(t.device)
