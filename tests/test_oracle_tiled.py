"""Pins oracle/attn_tiled.c (the C restatement of the reference's tiled kernels)
against oracle/eager_ref.py and against the transformers golden vectors."""
import os

import numpy as np
import pytest
import torch

from oracle import eager_ref as E
from oracle import tiled as T

SCALE = 0.125

CASES = [
    # S, window, seqlens, q_offset, Skv
    (100, None, None, 0, None),
    (130, 32, None, 0, None),
    (200, 128, None, 0, None),
    (96, 17, [50, 96], 0, None),
    (70, None, [1, 70], 0, None),
    (40, None, None, 24, 64),
    (40, 16, None, 24, 64),
]


@pytest.mark.parametrize("s,w,sl,qo,skv", CASES)
def test_tiled_matches_eager(s, w, sl, qo, skv):
    b = len(sl) if sl else 1
    q, k, v, sinks, d_out = E.make_inputs(21, b, 8, 2, s, 64, skv=skv)
    dbl = [t.double() for t in (q, k, v, sinks, d_out)]
    out, dq, dk, dv, ds = E.eager_attention_grads(*dbl, SCALE, w, qo, sl)
    lse = E.logsumexp_rows(dbl[0], dbl[1], dbl[3], SCALE, w, qo, sl)
    o2, lse2 = T.tiled_fwd(q, k, v, sinks, SCALE, w, qo, sl)
    dq2, dk2, dv2, ds2, delta = T.tiled_bwd(q, k, v, sinks, o2, lse2, d_out, SCALE, w, qo, sl)
    for name, a, b_ in (("o", out, o2), ("lse", lse, lse2), ("dq", dq, dq2), ("dk", dk, dk2),
                        ("dv", dv, dv2), ("ds", ds, ds2)):
        assert torch.allclose(a.float(), b_, atol=3e-6, rtol=1e-5), (name, float((a.float() - b_).abs().max()))
    assert torch.allclose(delta, (out * dbl[4]).sum(-1).permute(0, 2, 1).float(), atol=3e-6)


def test_tiled_matches_transformers_golden(golden_dir):
    z = np.load(os.path.join(golden_dir, "tiny_win8.npz"))
    q, k, v, sinks, d_out = E.make_inputs(int(z["seed"]), 1, 8, 2, 64, 64)
    o, lse = T.tiled_fwd(q, k, v, sinks, SCALE, 8)
    dq, dk, dv, ds, _ = T.tiled_bwd(q, k, v, sinks, o, lse, d_out, SCALE, 8)
    for name, mine in (("out", o), ("dq", dq), ("dk", dk), ("dv", dv), ("dsinks", ds)):
        assert np.allclose(mine.numpy(), z[name], rtol=1e-4, atol=2e-5), name


def test_null_sinks_is_zero_logit():
    q, k, v, _, _ = E.make_inputs(22, 1, 4, 2, 30, 64)
    a, la = T.tiled_fwd(q, k, v, None, SCALE)
    b_, lb = T.tiled_fwd(q, k, v, torch.zeros(4), SCALE)
    assert torch.equal(a, b_) and torch.equal(la, lb)


def test_padded_rows_are_inert():
    q, k, v, sinks, d_out = E.make_inputs(23, 2, 4, 2, 40, 64)
    sl = [13, 40]
    o, lse = T.tiled_fwd(q, k, v, sinks, SCALE, None, 0, sl)
    assert torch.all(o[0, 13:] == 0)
    assert torch.allclose(lse[0, :, 13:], sinks.view(-1, 1).expand(4, 27))
    dq, dk, dv, ds, _ = T.tiled_bwd(q, k, v, sinks, o, lse, d_out, SCALE, None, 0, sl)
    assert torch.all(dq[0, :, 13:] == 0) and torch.all(dk[0, :, 13:] == 0) and torch.all(dv[0, :, 13:] == 0)


def test_tiled_packed_rows_match_eager_and_golden(golden_dir):
    z = np.load(os.path.join(golden_dir, "tiny_packed_win8.npz"))
    ds = E.doc_start_from_lengths(z["doc_lens"].tolist(), 64)
    q, k, v, sinks, d_out = E.make_inputs(int(z["seed"]), 1, 8, 2, 64, 64)
    o, lse = T.tiled_fwd(q, k, v, sinks, SCALE, 8, 0, None, ds)
    dq, dk, dv, dsk, _ = T.tiled_bwd(q, k, v, sinks, o, lse, d_out, SCALE, 8, 0, None, ds)
    for name, mine in (("out", o), ("dq", dq), ("dk", dk), ("dv", dv), ("dsinks", dsk)):
        assert np.allclose(mine.numpy(), z[name], rtol=1e-4, atol=2e-5), name
    # a larger ragged packed case against the eager oracle
    ds = E.doc_start_from_lengths([[70, 3, 127], [200]], 200)
    q, k, v, sinks, d_out = E.make_inputs(24, 2, 8, 2, 200, 64)
    ref = E.eager_attention_grads(*(t.double() for t in (q, k, v, sinks, d_out)), SCALE, None, 0, None, ds)
    o, lse = T.tiled_fwd(q, k, v, sinks, SCALE, None, 0, None, ds)
    got = (o,) + T.tiled_bwd(q, k, v, sinks, o, lse, d_out, SCALE, None, 0, None, ds)[:4]
    for a, b_ in zip(ref, got):
        assert torch.allclose(a.float(), b_, atol=3e-6, rtol=1e-5)


def test_three_bf16_terms_carry_an_fp32_number():
    """The dK/dV kernels take lse / scale and -delta as three bf16 terms each (hi = bf16(x), mid = bf16(x - hi),
    lo = bf16(x - hi - mid), csrc/attn_common.h split_row_stats) and let the matrix pipe add them up in fp32.
    The claim the kernels rest on, checked here in torch's own bf16 arithmetic (round to nearest even, as the
    device's conversion): both residuals are exact in fp32 and the three terms add up to x exactly, for the
    whole range the statistics live in (logsumexp / scale up to a few thousand, delta of either sign, tiny values)."""
    import torch
    gen = torch.Generator().manual_seed(5)
    mags = torch.tensor([1e-6, 1e-3, 0.1, 1.0, 17.0, 300.0, 4096.0, 1.0e5])
    x = (torch.randn(8, 20000, generator=gen) * mags.view(8, 1)).reshape(-1).float()
    x = torch.cat([x, torch.tensor([0.0, -0.0, 1.0, -1.0, 255.5, 65535.99, 2.0 ** -20, 3.0e38 / 2 ** 40])])
    hi = x.to(torch.bfloat16).float()
    r1 = x - hi
    assert torch.equal(r1.double(), x.double() - hi.double())          # the first residual is exact
    mid = r1.to(torch.bfloat16).float()
    r2 = r1 - mid
    assert torch.equal(r2.double(), r1.double() - mid.double())        # so is the second
    lo = r2.to(torch.bfloat16).float()
    assert torch.equal(lo, r2)                                         # and it fits 8 mantissa bits: nothing is left
    assert torch.equal((hi + mid) + lo, x) and torch.equal((lo + mid) + hi, x)
