"""ctypes binding of libpaged_attn.so (the C ABI declared in include/paged_attn.h).

torch is imported first on purpose: the library links the HIP runtime by soname
and must share the one instance torch has already loaded, so that device
pointers and stream handles mean the same thing on both sides.
"""
from __future__ import annotations

import ctypes
import os
import threading

import torch  # noqa: F401  (loads the HIP runtime this library binds to)

from .build import LIB_PATH

_lock = threading.Lock()
_lib = None

c_int, c_float, c_void_p, c_size_t = ctypes.c_int, ctypes.c_float, ctypes.c_void_p, ctypes.c_size_t



class QTransformStruct(ctypes.Structure):
    """`pa_q_transform` of include/paged_attn.h."""
    _fields_ = [("norm_weight", c_void_p), ("rope_cos", c_void_p), ("rope_sin", c_void_p),
                ("rope_max_pos", c_int), ("norm_eps", c_float)]


class NewKvStruct(ctypes.Structure):
    """`pa_new_kv` of include/paged_attn.h."""
    _fields_ = [("xk", c_void_p), ("xv", c_void_p), ("k_norm_weight", c_void_p), ("query_lens", c_void_p)]


class OutProjStruct(ctypes.Structure):
    """`pa_out_proj` of include/paged_attn.h."""
    _fields_ = [("o_weight", c_void_p), ("o_bias", c_void_p), ("out", c_void_p), ("N", c_int)]


SIGNATURES = {
    "pa_version": (c_int, []),
    "pa_last_error": (ctypes.c_char_p, []),
    "pa_decode_workspace_bytes": (c_size_t, [c_int] * 5),
    "pa_decode_workspace_bytes_for": (c_size_t, [c_int] * 9),
    "pa_decode": (c_int, [c_void_p] * 9 + [c_size_t] + [c_int] * 8 + [c_float] + [c_int] * 3 + [c_void_p, c_int, c_void_p, c_void_p]),
    "pa_decode_noalloc": (c_int, [c_void_p] * 8 + [c_int] * 8 + [c_float] + [c_int] * 3 + [c_void_p, c_int, c_void_p, c_void_p]),
    "pa_verify_workspace_bytes": (c_size_t, [c_int] * 4),
    "pa_verify": (c_int, [c_void_p] * 10 + [c_size_t] + [c_int] * 9 + [c_float, c_int, c_void_p, c_int, c_void_p, c_void_p]),
    "pa_prefill_workspace_bytes": (c_size_t, [c_int] * 7),
    "pa_prefill": (c_int, [c_void_p] * 9 + [c_int] * 9 + [c_float, c_int, c_int, c_void_p, c_int, c_void_p, c_size_t, c_void_p, c_void_p]),
    "pa_blocksparse_prefill": (c_int, [c_void_p] * 4 + [c_int] * 8 + [c_float, c_int, c_void_p]),
    "pa_o_proj": (c_int, [c_void_p] * 4 + [c_int] * 4 + [c_void_p]),
    "pa_o_proj_ws": (c_int, [c_void_p] * 5 + [c_size_t] + [c_int] * 4 + [c_void_p]),
    "pa_o_proj_workspace_bytes": (c_size_t, [c_int] * 3),
    "pa_decode_step_workspace_bytes": (c_size_t, [c_int] * 10),
    "pa_decode_step": (c_int, [c_void_p] * 11 + [c_size_t] + [c_int] * 8 + [c_float] + [c_int] * 3 + [c_void_p, c_int, c_void_p, c_void_p]),
    "pa_verify_step_workspace_bytes": (c_size_t, [c_int] * 5),
    "pa_verify_step": (c_int, [c_void_p] * 11 + [c_size_t] + [c_int] * 9 + [c_float, c_int, c_void_p, c_int, c_void_p, c_void_p]),
    "pa_gather_kv": (c_int, [c_void_p] * 4 + [c_int] * 8 + [c_void_p]),
    "pa_kv_write": (c_int, [c_void_p] * 9 + [c_int] * 8 + [c_void_p]),
    "pa_qk_norm_rope_kv_write": (c_int, [c_void_p] * 6 + [c_float] + [c_void_p] * 2 + [c_int] + [c_void_p] * 7 + [c_int] * 9 + [c_void_p]),
    "pa_debug_set": (c_int, [c_int, c_int]),
    "pa_profile_enable": (c_int, [c_int]),
    "pa_profile_collect": (c_int, [ctypes.POINTER(c_float), c_int]),
    "pa_profile_empty_launch": (c_int, [c_void_p]),
}


class PagedAttnLibraryError(RuntimeError):
    """The native library is missing or failed to load (no fallback exists)."""


def load():
    """Load the shared library once.  Raises if it has not been built."""
    global _lib
    with _lock:
        if _lib is not None:
            return _lib
        if not os.path.exists(LIB_PATH):
            raise PagedAttnLibraryError(
                f"{LIB_PATH} not found: build it with `python -m nkipy_amd.build` "
                "(there is no CPU or PyTorch fallback for these ops)")
        try:
            lib = ctypes.CDLL(LIB_PATH)
        except OSError as e:  # pragma: no cover - depends on the machine
            raise PagedAttnLibraryError(f"cannot load {LIB_PATH}: {e}") from e
        for name, (res, args) in SIGNATURES.items():
            fn = getattr(lib, name)
            fn.restype = res
            fn.argtypes = args
        _lib = lib
        return _lib


def last_error() -> str:
    return load().pa_last_error().decode("utf-8", "replace")
