"""Drop-in for the reference's `attention_kernel.py`, backed by hand-written
gfx950 HIP kernels instead of Triton.

Same public names and call conventions as the reference module:

* `attention(q, k, v, sinks, sm_scale, bandwidth, start_q)` -- positional, like
  `_attention.apply` (attention_kernel.py:220-347).  q is (B, H, S, D), k and v
  are (B, G, S_kv, D), the result is (B, S, H, D).
* `triton_flash_attention(module, query, key, value, attention_mask, scaling,
  dropout=0.0, **kwargs) -> (attn_output, None)` -- the Hugging Face attention
  interface (attention_kernel.py:348-358).  The name is kept so that
  `modeling_gpt_oss.eager_attention_forward = triton_flash_attention` keeps
  working; there is no Triton underneath.

Differences from the reference, none of which change a result it can produce:
no padding copies of q/k/v (rows are bounds-checked in the kernels), O is written
directly in (B, S, H, D) and dO read directly from it (no transpose copies,
attention_kernel.py:272,290), dK/dV/dSinks are produced without atomics and need
no zero-fill, `sinks=None` works in backward (the reference raises at :344), and
an optional `seqlens` (right-padding lengths) is accepted.
"""
from __future__ import annotations

from typing import Optional, Tuple

import torch

from . import _lib

__all__ = ["attention", "triton_flash_attention", "hip_flash_attention", "attention_forward", "attention_backward",
           "doc_start_from_position_ids", "OP_NAMESPACE"]

_DTYPES = {torch.bfloat16: _lib.DTYPE_BF16, torch.float32: _lib.DTYPE_FP32}

# When True the Hugging Face adapter masks across documents of packed rows (from the
# `position_ids` it is handed).  False reproduces the reference, which ignores position ids.
RESPECT_PACKING = False


def _strides_bhs(t: torch.Tensor, layout: str):
    """(b, h, s) element strides of a 4-D tensor given as 'bhsd' or 'bshd'."""
    st = t.stride()
    if layout == "bhsd":
        return st[0], st[1], st[2]
    return st[0], st[2], st[1]


_MAX_SEQ_STRIDE = 1 << 24   # elements; the library refuses larger sequence strides (ERR_STRIDE)


def _row_contiguous(t: torch.Tensor, seq_dim: int = 2) -> torch.Tensor:
    """The kernels need unit stride along head_dim, 16-byte aligned rows and a sequence stride
    of at least head_dim and at most 2^24 elements; anything else is copied."""
    if (t.stride(-1) != 1 or any((s * t.element_size()) % 16 for s in t.stride()[:-1]) or t.data_ptr() % 16
            or not (t.shape[-1] <= t.stride(seq_dim) <= _MAX_SEQ_STRIDE)):
        return t.contiguous()
    return t


def _set(st, triple):
    st.b, st.h, st.s = (int(x) for x in triple)


def _check_inputs(q, k, v, sinks, allow_cast=False):
    if not (q.is_cuda and k.is_cuda and v.is_cuda):
        raise RuntimeError("gptoss attention runs on the GPU only (HIP kernels); got a CPU tensor")
    ok_dtypes = tuple(_DTYPES) + ((torch.float16,) if allow_cast else ())
    if q.dtype not in ok_dtypes or k.dtype != q.dtype or v.dtype != q.dtype:
        raise RuntimeError(f"unsupported dtypes {q.dtype}/{k.dtype}/{v.dtype}: "
                           "q, k, v must all be bfloat16 or all be float32")
    if q.dim() != 4 or k.dim() != 4 or v.dim() != 4:
        raise RuntimeError("q must be (B,H,S,D) and k, v (B,G,S_kv,D)")
    if k.shape != v.shape or q.shape[0] != k.shape[0] or q.shape[3] != k.shape[3]:
        raise RuntimeError(f"shape mismatch: q {tuple(q.shape)}, k {tuple(k.shape)}, v {tuple(v.shape)}")
    if sinks is not None:
        if sinks.numel() != q.shape[1]:
            raise RuntimeError("sinks must hold one logit per query head")
        _require_on(q, "sinks", sinks)
    _require_on(q, "k", k)
    _require_on(q, "v", v)


def _require_on(q, name, t):
    """Every tensor reaches the kernels as a raw device pointer, so it has to live on q's GPU."""
    if not torch.is_tensor(t) or t.device != q.device:
        where = t.device if torch.is_tensor(t) else type(t).__name__
        raise RuntimeError(f"{name} is on {where} but q is on {q.device}: every tensor must be on q's GPU")


def _check_saved(q, o, lse, d_o):
    """The backward's extra tensors go to the kernels as raw pointers: refuse anything that is not
    on q's GPU or not in the layout the kernels address, before any launch."""
    b, h, sq, d = q.shape
    for name, t in (("o", o), ("lse", lse), ("d_o", d_o)):
        _require_on(q, name, t)
    for name, t in (("o", o), ("d_o", d_o)):
        if t.dtype != q.dtype:
            raise RuntimeError(f"{name} has dtype {t.dtype}, expected q's dtype {q.dtype}")
        if tuple(t.shape) != (b, sq, h, d):
            raise RuntimeError(f"{name} must be (B, S, H, D) = {(b, sq, h, d)}, got {tuple(t.shape)}")
    if lse.dtype != torch.float32:
        raise RuntimeError(f"lse must be float32, got {lse.dtype}")
    if tuple(lse.shape) != (b, h, sq):
        raise RuntimeError(f"lse must be (B, H, S) = {(b, h, sq)}, got {tuple(lse.shape)}")


def _base_params(q, k, v, sinks32, seqlens, scale, window, q_offset, doc_start=None, q_offset_dev=None):
    p = _lib.new_params()
    b, h, sq, d = q.shape
    g, skv = k.shape[1], k.shape[2]
    p.dtype = _DTYPES[q.dtype]
    p.B, p.H, p.G, p.Sq, p.Skv, p.D = b, h, g, sq, skv, d
    p.window = int(window or 0)
    p.q_offset = int(q_offset or 0)
    p.scale = float(scale)
    p.q, p.k, p.v = q.data_ptr(), k.data_ptr(), v.data_ptr()
    p.sinks = sinks32.data_ptr() if sinks32 is not None else None
    p.seqlens = seqlens.data_ptr() if seqlens is not None else None
    p.doc_start = doc_start.data_ptr() if doc_start is not None else None
    p.q_offset_dev = q_offset_dev.data_ptr() if q_offset_dev is not None else None
    _set(p.q_stride, _strides_bhs(q, "bhsd"))
    _set(p.k_stride, _strides_bhs(k, "bhsd"))
    _set(p.v_stride, _strides_bhs(v, "bhsd"))
    return p


def _stream(t: torch.Tensor) -> int:
    return torch.cuda.current_stream(t.device).cuda_stream


def _prep_seqlens(seqlens, device, batch):
    if seqlens is None:
        return None
    sl = torch.as_tensor(seqlens, device=device).to(torch.int32).contiguous()
    if sl.numel() != batch:
        raise RuntimeError("seqlens must hold one length per batch row")
    return sl


def _prep_q_offset_dev(q_offset_dev, q):
    """One int32 on q's device holding the position of query row 0, or None.  No host read."""
    if q_offset_dev is None:
        return None
    t = q_offset_dev
    if not torch.is_tensor(t) or t.device != q.device or t.numel() != 1 or t.dtype.is_floating_point:
        raise RuntimeError("q_offset_dev must be a one-element integer tensor on the same device as q")
    return t.reshape(1).to(torch.int32).contiguous()


def _prep_doc_start(doc_start, q):
    if doc_start is None:
        return None
    ds = torch.as_tensor(doc_start, device=q.device).to(torch.int32).contiguous()
    if ds.shape != (q.shape[0], q.shape[2]):
        raise RuntimeError("doc_start must be (B, S): the first token index of each query's document")
    return ds


def doc_start_from_position_ids(position_ids: torch.Tensor) -> torch.Tensor:
    """(B, S) int32 document-start index per token of packed rows, from position ids that restart
    at every document (the convention transformers detects packing by, masking_utils.py:728-757):
    a new document begins wherever the position does not follow its predecessor by one."""
    pos = position_ids
    b, s = pos.shape
    idx = torch.arange(s, device=pos.device).view(1, s).expand(b, s)
    new_doc = torch.ones_like(pos, dtype=torch.bool)
    new_doc[:, 1:] = (pos[:, 1:] - pos[:, :-1]) != 1
    starts = torch.where(new_doc, idx, torch.zeros_like(idx))
    return torch.cummax(starts, dim=1).values.to(torch.int32)


def attention_forward(q, k, v, sinks, sm_scale, window=None, q_offset=0, seqlens=None, doc_start=None,
                      q_offset_dev=None):
    """Runs the forward kernel.  Returns (o (B,S,H,D), lse (B,H,S) fp32).
    q_offset_dev: optional one-element integer tensor on the device that holds the query offset
    (the reference's `start_q` tensor); the kernels read it, the host never does."""
    _check_inputs(q, k, v, sinks)
    q, k, v = _row_contiguous(q), _row_contiguous(k), _row_contiguous(v)
    b, h, sq, d = q.shape
    sinks32 = None if sinks is None else sinks.detach().to(torch.float32).contiguous()
    sl = _prep_seqlens(seqlens, q.device, b)
    ds = _prep_doc_start(doc_start, q)
    qod = _prep_q_offset_dev(q_offset_dev, q)
    o = torch.empty((b, sq, h, d), dtype=q.dtype, device=q.device)
    lse = torch.empty((b, h, sq), dtype=torch.float32, device=q.device)
    with torch.cuda.device(q.device):
        p = _base_params(q, k, v, sinks32, sl, sm_scale, window, q_offset, ds, qod)
        p.o, p.lse = o.data_ptr(), lse.data_ptr()
        _set(p.o_stride, _strides_bhs(o, "bshd"))
        _lib.call("gptoss_attn_fwd", p, _stream(q))
    return o, lse


def attention_backward(q, k, v, sinks, o, lse, d_o, sm_scale, window=None, q_offset=0, seqlens=None,
                       need_dsinks=True, doc_start=None, split=False, q_offset_dev=None):
    """Runs the backward: `gptoss_attn_bwd`, or with `split=True` the three separate entry points
    (preprocess, dK/dV, dQ), which give the same bits.  o and d_o are (B,S,H,D).
    Returns (dq, dk, dv, dsinks_fp32_or_None)."""
    _check_inputs(q, k, v, sinks)
    _check_saved(q, o, lse, d_o)
    q, k, v = _row_contiguous(q), _row_contiguous(k), _row_contiguous(v)
    o, d_o = _row_contiguous(o, 1), _row_contiguous(d_o, 1)
    lse = lse.contiguous()
    b, h, sq, d = q.shape
    sinks32 = None if sinks is None else sinks.detach().to(torch.float32).contiguous()
    sl = _prep_seqlens(seqlens, q.device, b)
    ds = _prep_doc_start(doc_start, q)
    qod = _prep_q_offset_dev(q_offset_dev, q)
    dq = torch.empty((b, h, sq, d), dtype=q.dtype, device=q.device)
    dk = torch.empty(k.shape, dtype=k.dtype, device=q.device)
    dv = torch.empty(v.shape, dtype=v.dtype, device=q.device)
    dsinks = torch.empty((h,), dtype=torch.float32, device=q.device) if need_dsinks else None
    with torch.cuda.device(q.device):
        p = _base_params(q, k, v, sinks32, sl, sm_scale, window, q_offset, ds, qod)
        # scratch: [-delta; lse*log2e], then the dK/dV partial sums of split key blocks (short sequences)
        delta = torch.empty((_lib.load().gptoss_attn_workspace_bytes(p) // 4,), dtype=torch.float32, device=q.device)
        p.o, p.lse = o.data_ptr(), lse.data_ptr()
        _set(p.o_stride, _strides_bhs(o, "bshd"))
        p.d_o = d_o.data_ptr()
        _set(p.do_stride, _strides_bhs(d_o, "bshd"))
        p.dq, p.dk, p.dv = dq.data_ptr(), dk.data_ptr(), dv.data_ptr()
        _set(p.dq_stride, _strides_bhs(dq, "bhsd"))
        _set(p.dk_stride, _strides_bhs(dk, "bhsd"))
        _set(p.dv_stride, _strides_bhs(dv, "bhsd"))
        p.delta = delta.data_ptr()
        p.dsinks = dsinks.data_ptr() if dsinks is not None else None
        for name in (("gptoss_attn_bwd_preprocess", "gptoss_attn_bwd_dkdv", "gptoss_attn_bwd_dq") if split
                     else ("gptoss_attn_bwd",)):
            _lib.call(name, p, _stream(q))
    return dq, dk, dv, dsinks


# ---- torch custom ops --------------------------------------------------------------------
# The two library calls are registered as opaque PyTorch operators, `gptoss_attn::fwd` and
# `gptoss_attn::bwd`, with shape-only ("fake") implementations, so that tracing tools
# (torch.compile, FakeTensorMode, activation-checkpoint replay) see one node per call and never
# look inside.  The autograd.Function below calls through them.
OP_NAMESPACE = "gptoss_attn"


@torch.library.custom_op(f"{OP_NAMESPACE}::fwd", mutates_args=(), device_types="cuda")
def _op_fwd(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, sinks: Optional[torch.Tensor], sm_scale: float,
            window: int, q_offset: int, seqlens: Optional[torch.Tensor],
            doc_start: Optional[torch.Tensor],
            q_offset_dev: Optional[torch.Tensor] = None) -> Tuple[torch.Tensor, torch.Tensor]:
    return attention_forward(q, k, v, sinks, sm_scale, window, q_offset, seqlens, doc_start, q_offset_dev)


@_op_fwd.register_fake
def _op_fwd_fake(q, k, v, sinks, sm_scale, window, q_offset, seqlens, doc_start, q_offset_dev=None):
    b, h, sq, d = q.shape
    return q.new_empty((b, sq, h, d)), q.new_empty((b, h, sq), dtype=torch.float32)


@torch.library.custom_op(f"{OP_NAMESPACE}::bwd", mutates_args=(), device_types="cuda")
def _op_bwd(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, sinks: Optional[torch.Tensor], o: torch.Tensor,
            lse: torch.Tensor, d_o: torch.Tensor, sm_scale: float, window: int, q_offset: int,
            seqlens: Optional[torch.Tensor], doc_start: Optional[torch.Tensor],
            need_dsinks: bool,
            q_offset_dev: Optional[torch.Tensor] = None) -> Tuple[torch.Tensor, torch.Tensor, torch.Tensor, torch.Tensor]:
    dq, dk, dv, dsinks = attention_backward(q, k, v, sinks, o, lse, d_o, sm_scale, window, q_offset, seqlens,
                                            need_dsinks=need_dsinks, doc_start=doc_start, q_offset_dev=q_offset_dev)
    if dsinks is None:      # an operator cannot return None: an empty tensor stands for "not requested"
        dsinks = torch.empty((0,), dtype=torch.float32, device=q.device)
    return dq, dk, dv, dsinks


@_op_bwd.register_fake
def _op_bwd_fake(q, k, v, sinks, o, lse, d_o, sm_scale, window, q_offset, seqlens, doc_start, need_dsinks,
                 q_offset_dev=None):
    return (torch.empty_like(q, memory_format=torch.contiguous_format),
            torch.empty_like(k, memory_format=torch.contiguous_format),
            torch.empty_like(v, memory_format=torch.contiguous_format),
            q.new_empty((q.shape[1] if need_dsinks else 0,), dtype=torch.float32))


class _attention(torch.autograd.Function):
    """Same argument list and gradient tuple as the reference's `_attention`
    (attention_kernel.py:220-344), plus optional trailing `seqlens` and `doc_start`.

    bfloat16 tensors take the tuned bf16-MFMA kernels and float32 tensors the float32 kernels
    (exact to float32 rounding, not tuned for speed).  float16 tensors are accepted for
    convenience: they are rounded to bfloat16 on the way in and the results cast back."""

    @staticmethod
    def forward(ctx, q, k, v, sinks, sm_scale, bandwidth, start_q, seqlens=None, doc_start=None):
        _check_inputs(q, k, v, sinks, allow_cast=True)
        ctx.in_dtypes = (q.dtype, k.dtype, v.dtype)
        if q.dtype == torch.float16:
            q, k, v = (t.to(torch.bfloat16) for t in (q, k, v))
        # a start_q tensor that lives on the device stays there: the kernels read it (as the
        # reference's do, attention_kernel.py:44-47), the host does not wait for it
        q_offset, q_offset_dev = 0, None
        if torch.is_tensor(start_q) and start_q.is_cuda:
            q_offset_dev = _prep_q_offset_dev(start_q, q)
        elif start_q is not None:
            q_offset = int(start_q.item()) if torch.is_tensor(start_q) else int(start_q)
        seqlens = _prep_seqlens(seqlens, q.device, q.shape[0])
        doc_start = _prep_doc_start(doc_start, q)
        window = int(bandwidth or 0)
        sinks_in = None if sinks is None else sinks.detach()
        o, lse = _op_fwd(q, k, v, sinks_in, float(sm_scale), window, q_offset, seqlens, doc_start, q_offset_dev)
        ctx.save_for_backward(q, k, v, sinks, o, lse, seqlens, doc_start, q_offset_dev)
        ctx.sm_scale = float(sm_scale)
        ctx.window = window
        ctx.q_offset = q_offset
        return o.to(ctx.in_dtypes[0])

    @staticmethod
    def backward(ctx, do):
        q, k, v, sinks, o, lse, seqlens, doc_start, q_offset_dev = ctx.saved_tensors
        need_ds = sinks is not None and ctx.needs_input_grad[3]
        sinks_in = None if sinks is None else sinks.detach()
        dq, dk, dv, dsinks = _op_bwd(q, k, v, sinks_in, o, lse, do.to(q.dtype), ctx.sm_scale, ctx.window,
                                     ctx.q_offset, seqlens, doc_start, need_ds, q_offset_dev)
        dsinks = dsinks.to(sinks.dtype).view_as(sinks) if need_ds else None
        qd, kd, vd = ctx.in_dtypes
        return dq.to(qd), dk.to(kd), dv.to(vd), dsinks, None, None, None, None, None


attention = _attention.apply


def hip_flash_attention(
    module,
    query: torch.Tensor,
    key: torch.Tensor,
    value: torch.Tensor,
    attention_mask: Optional[torch.Tensor],
    scaling: float,
    dropout: float = 0.0,
    **kwargs,
):
    """Hugging Face attention-interface adapter (attention_kernel.py:348-358).

    Like the reference it ignores `attention_mask` and `dropout`: causality and the
    sliding window come from `module.sliding_window`, the sink logits from
    `module.sinks`.  A caller with right-padded batches may pass `seqlens=` in
    kwargs, or hand a 1-D integer tensor of valid lengths over as `attention_mask`.  Rows
    packed from several documents attend across documents, as in the reference, unless the
    caller passes `doc_start=` (see `doc_start_from_position_ids`) or packing awareness was
    switched on with `patch_flash_attention(respect_packing=True)`, in which case the
    `position_ids` the model passes along are used."""
    doc_start = kwargs.get("doc_start")
    if doc_start is None and RESPECT_PACKING and kwargs.get("position_ids") is not None:
        pos = kwargs["position_ids"]
        if pos.dim() == 2 and pos.shape[0] == query.shape[0] and pos.shape[1] == query.shape[2] == key.shape[2]:
            doc_start = doc_start_from_position_ids(pos)
    seqlens = kwargs.get("seqlens")
    if (seqlens is None and torch.is_tensor(attention_mask) and attention_mask.dim() == 1
            and not attention_mask.dtype.is_floating_point):
        # valid lengths handed over in place of the dense mask (see sft_bench.mask_free_attention_mask)
        seqlens = attention_mask
    out = attention(query, key, value, module.sinks, scaling, module.sliding_window, None, seqlens, doc_start)
    return out, None


# The reference's public name, kept so existing patch code keeps working.
triton_flash_attention = hip_flash_attention
