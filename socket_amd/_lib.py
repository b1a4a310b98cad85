"""ctypes binding of libsocket_hip.so (the C ABI declared in include/socket_hip.h).

There is no CPU route: importing works anywhere (so the package can be
inspected and the library's exports checked without a GPU), but the library
must be present, and any compute call needs a HIP device.  A missing library
raises at first use with the build command to run.
"""
from __future__ import annotations

import ctypes
import os
from ctypes import c_char_p, c_float, c_int, c_int64, c_size_t, c_void_p, POINTER

import torch

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libsocket_hip.so")

SOCKET_OK = 0
SOCKET_ERR_NULL = -1
SOCKET_ERR_SHAPE = -2
SOCKET_ERR_UNSUPPORTED = -3
SOCKET_ERR_ALIGN = -4
SOCKET_ERR_WORKSPACE = -5
SOCKET_ERR_LAUNCH = -6

SOCKET_F32, SOCKET_BF16, SOCKET_F16 = 0, 1, 2
SOCKET_TOPK_MAX_M = 16384

_DTYPE_ENUM = {torch.float32: SOCKET_F32, torch.bfloat16: SOCKET_BF16, torch.float16: SOCKET_F16}

_P, _I, _L, _Z = c_void_p, c_int, c_int64, c_size_t

# name -> (restype, argtypes); one entry per declaration in include/socket_hip.h
SIGNATURES = {
    "socket_abi_version": (_I, []),
    "socket_status_string": (c_char_p, [_I]),
    "socket_device_query": (_I, [POINTER(c_int), POINTER(c_int)]),
    "socket_words_per_key": (_I, [_I, _I]),
    "socket_permute_planes": (_I, [_P, _I, _I, _I, _I, _P, _P]),
    "socket_hash_keys": (_I, [_P, _P, _I, _L, _L, _L, _L, _L, _L, _P, _P, _P, _P, _I,
                              _I, _I, _I, _I, _I, _I, _L, _P]),
    "socket_unpack_codes": (_I, [_P, _P, _I, _I, _I, _I, _I, _I, _L, _L, _L, _L, _L, _P]),
    "socket_pack_codes": (_I, [_P, _L, _L, _L, _L, _P, _I, _I, _I, _I, _I, _I, _L, _P]),
    "socket_score_range_parts": (_I, [_I, _I, _I, _I, _I, _I, _I, _I]),
    "socket_score_packed": (_I, [_P, _I, _P, _P, _P, _P, _P, _I, _I, _I, _I, _I, _I, _I, _I, _L, _L, _I, _P]),
    "socket_soft_hash_collision": (_I, [_P, _P, _P, _P, _P, _I, _I, _I, _I, _I, _P]),
    "socket_soft_hash_score_f16": (_I, [_P, _P, _P, _P, _P, _I, _I, _I, _I, _I, _P]),
    "socket_score_plan_query": (_I, [_I, _I, _I, _I, _I, _I, _I, _I, _I, POINTER(c_int), POINTER(c_int),
                                     POINTER(c_int), POINTER(c_float)]),
    "socket_score_shape_cost": (_I, [_I, _I, _I, _I, _I, _I, _I, _I, _I, _I, _I, _I, POINTER(c_int), POINTER(c_int),
                                     POINTER(c_float)]),
    "socket_group_shape": (_I, [_I, _I, POINTER(c_int), POINTER(c_int)]),
    "socket_score_prefers_grouped": (_I, [_I, _I, _I, _I, _I, _I, _I, _I]),
    "socket_score_range_parts_grouped": (_I, [_I, _I, _I, _I, _I, _I, _I, _I]),
    "socket_score_persistent_serves": (_I, [_I, _I, _I, _I, _I, _I, _I, _I]),
    "socket_group_q_probs": (_I, [_P, _I, _P, _I, _I, _I, _I, _I, _P]),
    "socket_score_packed_grouped": (_I, [_P, _I, _P, _P, _P, _P, _P, _I, _I, _I, _I, _I, _I, _I, _I, _L, _L, _I, _P]),
    "socket_soft_hash_grouped": (_I, [_P, _I, _L, _L, _P, _P, _P, _I, _I, _I, _I, _I, _I, _I, _I, c_float, c_float, _P]),
    "socket_soft_hash": (_I, [_P, _I, _L, _L, _P, _P, _P, _I, _I, _I, _I, _I, _I, _I, _I, c_float, c_float, _P]),
    "socket_select_workspace_bytes": (_Z, [_I, _I, _I, _I]),
    "socket_select_workspace_zero_bytes": (_Z, [_I, _I, _I, _I]),
    "socket_select_list": (_I, [_P, _L, _P, _P, _P, _I, _I, _I, _I, _I, _I, _I, _I, _P, _L, _I, _P, _P, _Z, _P]),
    "socket_rope_append": (_I, [_P, _I, _L, _P, _I, _L, _P, _I, _P, _P, _P, _L, _L, _L, _P, _P, _P, _I, _I, _I, _I,
                                _L, _P]),
    "socket_decode_prologue": (_I, [_P, _I, _L, _P, _I, _L, _P, _I, _P, _P, _P, _L, _L, _L, _P, _P, _P, _P, _P, _P, _P,
                                    _I, _I, _I, _I, _I, _I, _I, _I, _I, _L, c_float, c_float, _P]),
    "socket_add_rmsnorm": (_I, [_P, _P, _P, _P, _P, _I, _L, _I, c_float, _P]),
    "socket_silu_mul": (_I, [_P, _P, _P, _I, _L, _P]),
    "socket_gemv_bf16": (_I, [_P, _L, _P, _P, _P, _L, _I, _I, _I, _P]),
    "socket_norm_gemv_bf16": (_I, [_P, _P, _P, c_float, _P, _P, _P, _P, _I, _I, _I, _P]),
    "socket_attend_stage1": (_I, [_P, _P, _P, _I, _L, _L, _L, _L, _L, _L, _L, _L,
                                  _P, _L, _L, _P, _L, _L, _P, _P,
                                  _I, _I, _I, _I, _I, _I, _I, _I, _P]),
    "socket_attend_stage2": (_I, [_P, _P, _P, _L, _L, _P, _I, _L, _L, _I, _I, _I, _I, _I, _P]),
    "socket_sparse_attention_block_seq": (_I, [_I, _I, _I]),
    "socket_sparse_attention_workspace_bytes": (_Z, [_I, _I, _I, _I]),
    "socket_sparse_attention": (_I, [_P, _P, _P, _I, _L, _L, _L, _L, _L, _L, _L, _L,
                                     _P, _L, _L, _P, _L, _L, _P, _L, _L, _P, _Z,
                                     _I, _I, _I, _I, _I, _I, _P]),
    "socket_static_scratch_bytes": (_Z, []),
    "socket_static_scratch_init": (_I, []),
    "socket_sparse_attention_static": (_I, [_P, _P, _P, _I, _L, _L, _L, _L, _L, _L, _L, _L,
                                            _P, _L, _L, _P, _L, _L, _P, _L, _L,
                                            _I, _I, _I, _I, _I, _I, _P]),
    "socket_dense_decode_workspace_bytes": (_Z, [_I, _I, _I, _I]),
    "socket_dense_decode": (_I, [_P, _P, _P, _I, _L, _L, _L, _L, _L, _L, _L, _L,
                                 _P, _P, _L, _L, _P, _Z, _I, _I, _I, _I, _I, _P]),
    "socket_block_sparse_attention": (_I, [_P, _P, _P, _I] + [_L] * 9 + [_P, _P, _P] + [_L] * 3 + [_I] * 8 + [_P]),
}

_lib = None


class SocketHipError(RuntimeError):
    """A libsocket_hip entry point returned a non-zero status."""

    def __init__(self, fn: str, status: int, text: str):
        super().__init__(f"{fn} failed with status {status}: {text}")
        self.status = status


def lib() -> ctypes.CDLL:
    """The loaded library with argument types set; raises if it is not built."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise RuntimeError(
                f"{LIB_PATH} is missing: build it with `python -m socket_amd.build` "
                "(hipcc, gfx950). There is no fallback path."
            )
        handle = ctypes.CDLL(LIB_PATH)
        for name, (res, args) in SIGNATURES.items():
            fn = getattr(handle, name)
            fn.restype = res
            fn.argtypes = args
        if handle.socket_abi_version() != 4:
            raise RuntimeError("libsocket_hip.so ABI version mismatch; rebuild it")
        _lib = handle
    return _lib


def check(fn: str, status: int) -> None:
    if status != SOCKET_OK:
        text = lib().socket_status_string(status).decode()
        raise SocketHipError(fn, status, text)


def dtype_enum(dt: torch.dtype) -> int:
    try:
        return _DTYPE_ENUM[dt]
    except KeyError:
        raise RuntimeError(f"unsupported dtype {dt}: expected float32, bfloat16 or float16") from None


def ptr(t) -> c_void_p:
    return c_void_p(0 if t is None else t.data_ptr())


def stream_ptr(device=None) -> c_void_p:
    """The HIP stream torch is currently issuing work on, as the reference's
    kernels (Triton and load_inline launches) do."""
    return c_void_p(torch.cuda.current_stream(device).cuda_stream)


def require_device(*tensors) -> None:
    for t in tensors:
        if t is not None and not t.is_cuda:
            raise AssertionError("expected a tensor on the HIP device")
