"""ctypes front end for attn_tiled.c (the C restatement of the reference's tiled
kernels).  Test infrastructure only; see the header of attn_tiled.c."""
from __future__ import annotations

import ctypes
import os
import subprocess
from typing import Optional, Sequence

import torch

_HERE = os.path.dirname(os.path.abspath(__file__))
_SO = os.path.join(_HERE, "liboracle_attn.so")
_lib = None


def build(force: bool = False) -> str:
    """Compile attn_tiled.c with the Makefile beside it."""
    if force and os.path.exists(_SO):
        os.remove(_SO)
    subprocess.run(["make", "-C", _HERE, "-s"], check=True)
    return _SO


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(_SO):
            build()
        _lib = ctypes.CDLL(_SO)
        for name in ("oracle_attn_fwd", "oracle_attn_bwd_delta", "oracle_attn_bwd"):
            getattr(_lib, name).restype = ctypes.c_int
    return _lib


def _fp(t: Optional[torch.Tensor]):
    if t is None:
        return ctypes.c_void_p(0)
    assert t.dtype == torch.float32 and t.is_contiguous() and t.device.type == "cpu"
    return ctypes.c_void_p(t.data_ptr())


def _ip(seqlens: Optional[Sequence[int]]):
    if seqlens is None:
        return None, ctypes.c_void_p(0)
    arr = (ctypes.c_int * len(seqlens))(*[int(x) for x in seqlens])
    return arr, ctypes.cast(arr, ctypes.c_void_p)


def tiled_fwd(q, k, v, sinks, scale, window=None, q_offset=0, seqlens=None, doc_start=None):
    """q (B,H,Sq,D), k/v (B,G,Skv,D) fp32 -> (o (B,Sq,H,D), lse (B,H,Sq))."""
    q, k, v = (t.detach().float().contiguous() for t in (q, k, v))
    s = None if sinks is None else sinks.detach().float().contiguous()
    b, h, sq, d = q.shape
    g, skv = k.shape[1], k.shape[2]
    o = torch.empty(b, sq, h, d)
    lse = torch.empty(b, h, sq)
    keep, sl = _ip(seqlens)
    keep2, dsp = _ip(None if doc_start is None else torch.as_tensor(doc_start).reshape(-1).tolist())
    rc = lib().oracle_attn_fwd(_fp(q), _fp(k), _fp(v), _fp(s), _fp(o), _fp(lse),
                               b, h, g, sq, skv, d, ctypes.c_float(scale),
                               int(window or 0), int(q_offset), sl, dsp)
    if rc:
        raise RuntimeError(f"oracle_attn_fwd rc={rc}")
    return o, lse


def tiled_bwd(q, k, v, sinks, o, lse, d_o, scale, window=None, q_offset=0, seqlens=None, doc_start=None):
    """Returns (dq, dk, dv, dsinks, delta); o and d_o are (B,Sq,H,D)."""
    q, k, v, o, lse, d_o = (t.detach().float().contiguous() for t in (q, k, v, o, lse, d_o))
    s = None if sinks is None else sinks.detach().float().contiguous()
    b, h, sq, d = q.shape
    g, skv = k.shape[1], k.shape[2]
    delta = torch.empty(b, h, sq)
    rc = lib().oracle_attn_bwd_delta(_fp(o), _fp(d_o), _fp(delta), b, h, sq, d)
    if rc:
        raise RuntimeError(f"oracle_attn_bwd_delta rc={rc}")
    dq, dk, dv = torch.empty_like(q), torch.empty_like(k), torch.empty_like(v)
    dsinks = torch.empty(h)
    keep, sl = _ip(seqlens)
    keep2, dsp = _ip(None if doc_start is None else torch.as_tensor(doc_start).reshape(-1).tolist())
    rc = lib().oracle_attn_bwd(_fp(q), _fp(k), _fp(v), _fp(s), _fp(lse), _fp(delta), _fp(d_o),
                               _fp(dq), _fp(dk), _fp(dv), _fp(dsinks),
                               b, h, g, sq, skv, d, ctypes.c_float(scale),
                               int(window or 0), int(q_offset), sl, dsp)
    if rc:
        raise RuntimeError(f"oracle_attn_bwd rc={rc}")
    return dq, dk, dv, dsinks, delta
