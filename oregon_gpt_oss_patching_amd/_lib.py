"""ctypes binding of include/gptoss_attn.h.

The library is the product: if libgptoss_attn.so is missing or cannot be loaded
this module raises; there is no fallback implementation.
"""
from __future__ import annotations

import ctypes
import os
from typing import Optional

_HERE = os.path.dirname(os.path.abspath(__file__))
LIBRARY = os.path.join(_HERE, "libgptoss_attn.so")

ABI_VERSION = 4
DTYPE_BF16 = 0
DTYPE_FP32 = 1

EXPORTS = (
    "gptoss_attn_version",
    "gptoss_attn_status_string",
    "gptoss_attn_validate",
    "gptoss_attn_workspace_bytes",
    "gptoss_attn_fwd",
    "gptoss_attn_bwd_preprocess",
    "gptoss_attn_bwd_dkdv",
    "gptoss_attn_bwd_dq",
    "gptoss_attn_bwd",
    "gptoss_attn_bwd_static",
    "gptoss_attn_static_scratch_bytes",
    "gptoss_attn_mfma_rate_probe",
    "gptoss_attn_stream_probe",
)


class Strides(ctypes.Structure):
    _fields_ = [("b", ctypes.c_int64), ("h", ctypes.c_int64), ("s", ctypes.c_int64)]


class Params(ctypes.Structure):
    """Mirror of `gptoss_attn_params`; field order and types must match the header."""

    _fields_ = [
        ("struct_size", ctypes.c_uint32),
        ("dtype", ctypes.c_int32),
        ("B", ctypes.c_int32), ("H", ctypes.c_int32), ("G", ctypes.c_int32),
        ("Sq", ctypes.c_int32), ("Skv", ctypes.c_int32), ("D", ctypes.c_int32),
        ("window", ctypes.c_int32),
        ("q_offset", ctypes.c_int32),
        ("scale", ctypes.c_float),
        ("reserved0", ctypes.c_int32),
        ("q", ctypes.c_void_p), ("k", ctypes.c_void_p), ("v", ctypes.c_void_p),
        ("sinks", ctypes.c_void_p),
        ("seqlens", ctypes.c_void_p),
        ("doc_start", ctypes.c_void_p),
        ("o", ctypes.c_void_p),
        ("lse", ctypes.c_void_p),
        ("d_o", ctypes.c_void_p),
        ("dq", ctypes.c_void_p), ("dk", ctypes.c_void_p), ("dv", ctypes.c_void_p),
        ("dsinks", ctypes.c_void_p),
        ("delta", ctypes.c_void_p),
        ("q_stride", Strides), ("k_stride", Strides), ("v_stride", Strides), ("o_stride", Strides),
        ("do_stride", Strides), ("dq_stride", Strides), ("dk_stride", Strides), ("dv_stride", Strides),
        ("q_offset_dev", ctypes.c_void_p),
    ]


class GptossAttnError(RuntimeError):
    def __init__(self, fn: str, status: int, text: str):
        super().__init__(f"{fn} failed with status {status}: {text}")
        self.status = status


_lib: Optional[ctypes.CDLL] = None


def load() -> ctypes.CDLL:
    """Loads libgptoss_attn.so (once).  Raises if it has not been built."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIBRARY):
            raise RuntimeError(
                f"{LIBRARY} is missing: build it with `python -m oregon_gpt_oss_patching_amd.build` "
                "(hipcc, gfx950). There is no fallback attention path.")
        lib = ctypes.CDLL(LIBRARY)
        lib.gptoss_attn_version.restype = ctypes.c_int
        lib.gptoss_attn_version.argtypes = []
        lib.gptoss_attn_status_string.restype = ctypes.c_char_p
        lib.gptoss_attn_status_string.argtypes = [ctypes.c_int]
        lib.gptoss_attn_validate.restype = ctypes.c_int
        lib.gptoss_attn_validate.argtypes = [ctypes.POINTER(Params), ctypes.c_int]
        lib.gptoss_attn_workspace_bytes.restype = ctypes.c_size_t
        lib.gptoss_attn_workspace_bytes.argtypes = [ctypes.POINTER(Params)]
        lib.gptoss_attn_static_scratch_bytes.restype = ctypes.c_size_t
        lib.gptoss_attn_static_scratch_bytes.argtypes = []
        lib.gptoss_attn_mfma_rate_probe.restype = ctypes.c_int64
        lib.gptoss_attn_mfma_rate_probe.argtypes = [ctypes.c_void_p, ctypes.c_size_t, ctypes.c_int, ctypes.c_void_p,
                                                    ctypes.c_size_t, ctypes.c_void_p]
        lib.gptoss_attn_stream_probe.restype = ctypes.c_int64
        lib.gptoss_attn_stream_probe.argtypes = [ctypes.c_int, ctypes.c_int, ctypes.c_int, ctypes.c_void_p, ctypes.c_size_t,
                                                 ctypes.c_void_p]
        for name in ("gptoss_attn_fwd", "gptoss_attn_bwd_preprocess", "gptoss_attn_bwd_dkdv",
                     "gptoss_attn_bwd_dq", "gptoss_attn_bwd", "gptoss_attn_bwd_static"):
            fn = getattr(lib, name)
            fn.restype = ctypes.c_int
            fn.argtypes = [ctypes.POINTER(Params), ctypes.c_void_p]
        if lib.gptoss_attn_version() != ABI_VERSION:
            raise RuntimeError("libgptoss_attn.so ABI version mismatch; rebuild the library")
        _lib = lib
    return _lib


def status_string(status: int) -> str:
    return load().gptoss_attn_status_string(int(status)).decode()


def call(name: str, params: Params, stream: int = 0) -> None:
    """Calls an entry point and raises GptossAttnError on a non-zero status."""
    rc = getattr(load(), name)(ctypes.byref(params), ctypes.c_void_p(stream))
    if rc != 0:
        raise GptossAttnError(name, rc, status_string(rc))


def new_params() -> Params:
    p = Params()
    p.struct_size = ctypes.sizeof(Params)
    return p
