"""CPU oracle for GPT-OSS attention: the eager math, restated in plain torch.

TEST INFRASTRUCTURE ONLY.  Nothing in the shipped package imports this module;
it exists so that tests, the smoke check and the benchmark's CPU-baseline leg
have something independent to compare the HIP kernels with.

What is restated, and where it comes from:

* ``eager_attention``   -- the function the reference monkeypatches away,
  ``transformers/models/gpt_oss/modeling_gpt_oss.py:235-263`` (transformers
  5.15.0): repeat K/V over the GQA group (``:203-212``), ``QK^T * scaling``,
  additive mask, concatenate the per-head sink logit as one extra column,
  subtract the row max, softmax, drop the sink column, ``@ V``, transpose to
  (B, S, H, D).
* ``allowed_mask``      -- the index predicates ``kv <= q``
  (``transformers/masking_utils.py:76-80``) and ``kv > q - window``
  (``:92-100``), which are the same predicates the reference kernel evaluates
  per element (``attention_kernel.py:68,71``), plus right-padding key/query
  validity for padded batches.
* ``logsumexp_rows``    -- the per-row statistic the reference forward stores,
  ``M = m + log(l + exp(sink - m))`` (``attention_kernel.py:93-98``).

Gradients are not restated: they come from ``torch.autograd`` differentiating
``eager_attention``, which is what differentiates the original eager function
during training.

Pinning (see tests/test_oracle_*.py): golden vectors written by the installed
``transformers`` eager function (tests/golden/), the sink -> -inf limit against
``torch.nn.functional.scaled_dot_product_attention``, a pure-Python triple loop
on tiny shapes, fp64 ``gradcheck``, and softmax invariants.
"""
from __future__ import annotations

from typing import Optional, Sequence

import torch


def allowed_mask(
    sq: int,
    skv: int,
    window: Optional[int],
    q_offset: int = 0,
    seqlens: Optional[Sequence[int]] = None,
    batch: int = 1,
    doc_start: Optional[torch.Tensor] = None,
) -> torch.Tensor:
    """Boolean (B, 1, Sq, Skv) mask, True where query row i may see key j.

    Row i sits at absolute position ``q_offset + i``.  A key is visible when
    ``j <= pos`` (masking_utils.py:80) and, for a sliding layer,
    ``j > pos - window`` (masking_utils.py:98).  ``window`` of None or 0 means a
    full-causal layer, which is how the reference treats a falsy BANDWIDTH
    (attention_kernel.py:60-63).  With ``seqlens`` (right padding), keys at or
    beyond the row's valid length are hidden and so is every key for a padded
    query row.  With ``doc_start`` (B, Sq) -- for packed rows, the index of the
    first token of the document each query belongs to -- keys before it are
    hidden, which for a causal mask is exactly transformers' same-document
    predicate (masking_utils.py:182-190).
    """
    i = torch.arange(sq).view(sq, 1) + q_offset
    j = torch.arange(skv).view(1, skv)
    ok = j <= i
    if window:
        ok = ok & (j > i - window)
    ok = ok.view(1, 1, sq, skv).expand(batch, 1, sq, skv)
    if seqlens is not None:
        lens = torch.as_tensor(list(seqlens), dtype=torch.long).view(batch, 1, 1, 1)
        kvalid = torch.arange(skv).view(1, 1, 1, skv) < lens
        qvalid = (torch.arange(sq).view(1, 1, sq, 1) + q_offset) < lens
        ok = ok & kvalid & qvalid
    if doc_start is not None:
        ds = torch.as_tensor(doc_start).to(torch.long).view(batch, 1, sq, 1)
        ok = ok & (torch.arange(skv).view(1, 1, 1, skv) >= ds)
    return ok


def repeat_kv(x: torch.Tensor, n_rep: int) -> torch.Tensor:
    """(B, G, S, D) -> (B, G*n_rep, S, D); query head h reads KV head h // n_rep
    (modeling_gpt_oss.py:203-212; attention_kernel.py:36)."""
    return x.repeat_interleave(n_rep, dim=1)


def eager_attention(
    q: torch.Tensor,
    k: torch.Tensor,
    v: torch.Tensor,
    sinks: Optional[torch.Tensor],
    scale: float,
    window: Optional[int] = None,
    q_offset: int = 0,
    seqlens: Optional[Sequence[int]] = None,
    doc_start: Optional[torch.Tensor] = None,
) -> torch.Tensor:
    """Eager attention with a sink column; returns (B, Sq, H, D).

    q: (B, H, Sq, D); k, v: (B, G, Skv, D); sinks: (H,) or None.  ``None``
    means a sink logit of 0 -- that is what the reference kernel does
    (attention_kernel.py:39-42) -- not "no sink".
    Computation runs in the dtype of ``q`` (use fp32/fp64 inputs).
    Masked logits are set to -inf rather than to a large negative number so
    that a fully masked row (a padded query) leaves only the sink column and
    therefore produces an exactly zero output row.
    """
    b, h, sq, d = q.shape
    g, skv = k.shape[1], k.shape[2]
    r = h // g
    kk = repeat_kv(k, r)
    vv = repeat_kv(v, r)
    logits = torch.matmul(q, kk.transpose(2, 3)) * scale
    ok = allowed_mask(sq, skv, window, q_offset, seqlens, b, doc_start).to(q.device)
    logits = logits.masked_fill(~ok, float("-inf"))
    if sinks is None:
        sink_col = torch.zeros(1, h, 1, 1, dtype=q.dtype, device=q.device)
    else:
        sink_col = sinks.to(q.dtype).view(1, h, 1, 1)
    combined = torch.cat([logits, sink_col.expand(b, h, sq, 1)], dim=-1)
    combined = combined - combined.max(dim=-1, keepdim=True).values
    probs = torch.softmax(combined, dim=-1)
    out = torch.matmul(probs[..., :-1], vv)
    return out.transpose(1, 2).contiguous()


def logsumexp_rows(
    q: torch.Tensor,
    k: torch.Tensor,
    sinks: Optional[torch.Tensor],
    scale: float,
    window: Optional[int] = None,
    q_offset: int = 0,
    seqlens: Optional[Sequence[int]] = None,
    doc_start: Optional[torch.Tensor] = None,
) -> torch.Tensor:
    """(B, H, Sq) natural-log logsumexp over the visible logits and the sink,
    the quantity the reference stores as M (attention_kernel.py:93-98)."""
    b, h, sq, d = q.shape
    g, skv = k.shape[1], k.shape[2]
    kk = repeat_kv(k, h // g)
    logits = torch.matmul(q, kk.transpose(2, 3)) * scale
    ok = allowed_mask(sq, skv, window, q_offset, seqlens, b, doc_start).to(q.device)
    logits = logits.masked_fill(~ok, float("-inf"))
    if sinks is None:
        sink_col = torch.zeros(1, h, 1, 1, dtype=q.dtype, device=q.device)
    else:
        sink_col = sinks.to(q.dtype).view(1, h, 1, 1)
    combined = torch.cat([logits, sink_col.expand(b, h, sq, 1)], dim=-1)
    return torch.logsumexp(combined, dim=-1)


def eager_attention_grads(
    q: torch.Tensor,
    k: torch.Tensor,
    v: torch.Tensor,
    sinks: torch.Tensor,
    d_out: torch.Tensor,
    scale: float,
    window: Optional[int] = None,
    q_offset: int = 0,
    seqlens: Optional[Sequence[int]] = None,
    doc_start: Optional[torch.Tensor] = None,
):
    """Forward + autograd backward.  ``d_out`` is (B, Sq, H, D), the layout in
    which the gradient reaches the op (attention_kernel.py:290).  Returns
    ``(out, dq, dk, dv, dsinks)``."""
    q = q.detach().clone().requires_grad_(True)
    k = k.detach().clone().requires_grad_(True)
    v = v.detach().clone().requires_grad_(True)
    s = sinks.detach().clone().requires_grad_(True)
    out = eager_attention(q, k, v, s, scale, window, q_offset, seqlens, doc_start)
    dq, dk, dv, ds = torch.autograd.grad(out, (q, k, v, s), d_out)
    return out.detach(), dq, dk, dv, ds


def make_inputs(
    seed: int,
    b: int,
    h: int,
    g: int,
    sq: int,
    d: int,
    dtype: torch.dtype = torch.float32,
    skv: Optional[int] = None,
):
    """Seeded synthetic inputs, drawn on the CPU in fp32 in the fixed order
    Q, K, V, sinks, dO ~ N(0,1) and rounded to ``dtype``.  CPU ``randn`` with a
    fixed generator seed is platform independent, so the same call reproduces
    the same tensors on the GPU box."""
    skv = sq if skv is None else skv
    gen = torch.Generator(device="cpu").manual_seed(seed)
    q = torch.randn(b, h, sq, d, generator=gen).to(dtype)
    k = torch.randn(b, g, skv, d, generator=gen).to(dtype)
    v = torch.randn(b, g, skv, d, generator=gen).to(dtype)
    sinks = torch.randn(h, generator=gen).to(dtype)
    d_out = torch.randn(b, sq, h, d, generator=gen).to(dtype)
    return q, k, v, sinks, d_out


def pair_count(s: int, window: Optional[int]) -> int:
    """Visible (query, key) pairs per head for a length-``s`` row:
    s(s+1)/2 for full causal, W*s - W(W-1)/2 for a window W <= s."""
    if not window or window >= s:
        return s * (s + 1) // 2
    return window * s - window * (window - 1) // 2


def attention_flops(b: int, h: int, d: int, pairs: int):
    """Algorithmic FLOPs: 2 GEMMs forward, 5 backward, 2*D flops per pair each."""
    unit = 2 * d * pairs * b * h
    return {"fwd": 2 * unit, "bwd": 5 * unit, "total": 7 * unit}


def doc_start_from_lengths(doc_lens: Sequence[Sequence[int]], s: int) -> torch.Tensor:
    """(B, S) int32 document-start index per token for rows packed from documents of the
    given lengths (each row's lengths must sum to ``s``)."""
    rows = []
    for lens in doc_lens:
        assert sum(lens) == s
        starts, pos = [], 0
        for n in lens:
            starts += [pos] * n
            pos += n
        rows.append(starts)
    return torch.tensor(rows, dtype=torch.int32)
