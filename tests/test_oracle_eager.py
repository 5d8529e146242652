"""Pins oracle/eager_ref.py: golden vectors from the installed transformers eager
function, library special cases, brute force, gradcheck and softmax invariants.
Each check is chosen so that a plausible slip (dropped sink term, wrong window
edge, wrong head mapping, transposed output) fails at least one of them."""
import math
import os

import numpy as np
import pytest
import torch
import torch.nn.functional as F

from oracle import eager_ref as E

SCALE = 0.125


def _load(golden_dir, name):
    z = np.load(os.path.join(golden_dir, f"{name}.npz"))
    sl = z["seqlens"].tolist() or None
    return z, int(z["seed"]), int(z["B"]), int(z["H"]), int(z["G"]), int(z["S"]), int(z["D"]), int(z["window"]) or None, sl


@pytest.mark.parametrize("name", ["tiny_full", "tiny_win8", "tiny_pad_full", "tiny_pad_win8"])
def test_golden_full_tensors(golden_dir, name):
    z, seed, b, h, g, s, d, w, sl = _load(golden_dir, name)
    q, k, v, sinks, d_out = E.make_inputs(seed, b, h, g, s, d)
    if sl is not None:
        qvalid = (torch.arange(s).view(1, s) < torch.tensor(sl).view(b, 1)).view(b, s, 1, 1)
        d_out = d_out * qvalid
    out, dq, dk, dv, ds = E.eager_attention_grads(q, k, v, sinks, d_out, SCALE, w, 0, sl)
    gold_out = torch.from_numpy(z["out"])
    if sl is not None:
        # transformers lets padded query rows attend valid keys; the op defines them as zero
        assert torch.all(out[~qvalid.expand_as(out)] == 0)
        out = out * qvalid
        gold_out = gold_out * qvalid
    for name_, mine, gold in (("out", out, gold_out), ("dq", dq, z["dq"]), ("dk", dk, z["dk"]),
                              ("dv", dv, z["dv"]), ("dsinks", ds, z["dsinks"])):
        gold = torch.as_tensor(gold)
        assert torch.allclose(mine, gold, rtol=1e-4, atol=2e-5), (name_, float((mine - gold).abs().max()))
    if sl is not None:
        for bi, L in enumerate(sl):
            assert torch.all(dq[bi, :, L:] == 0) and torch.all(dk[bi, :, L:] == 0) and torch.all(dv[bi, :, L:] == 0)


@pytest.mark.parametrize("name", ["cfg1_full", "cfg1_win32"])
def test_golden_config1_samples(golden_dir, name):
    z, seed, b, h, g, s, d, w, sl = _load(golden_dir, name)
    q, k, v, sinks, d_out = E.make_inputs(seed, b, h, g, s, d)
    out, dq, dk, dv, ds = E.eager_attention_grads(q, k, v, sinks, d_out, SCALE, w)
    for n, t in (("out", out), ("dq", dq), ("dk", dk), ("dv", dv)):
        flat = t.reshape(-1)
        idx = torch.arange(0, flat.numel(), max(1, flat.numel() // 1024))[:1024]
        assert np.allclose(flat[idx].numpy(), z[f"{n}_sample"], rtol=1e-4, atol=2e-5), n
        assert math.isclose(float(t.double().norm()), float(z[f"{n}_norm"]), rel_tol=1e-5), n
    assert np.allclose(ds.numpy(), z["dsinks"], rtol=1e-4, atol=2e-5)


@pytest.mark.parametrize("window", [None, 5, 64])
def test_sink_to_minus_inf_is_sdpa(window):
    """With the sink logit at -1e4 the extra column vanishes and the op is plain
    masked GQA attention, which torch ships."""
    q, k, v, _, _ = E.make_inputs(3, 2, 8, 2, 40, 64)
    sinks = torch.full((8,), -1e4)
    out = E.eager_attention(q, k, v, sinks, SCALE, window)
    mask = E.allowed_mask(40, 40, window, batch=2)
    ref = F.scaled_dot_product_attention(q, k, v, attn_mask=mask, scale=SCALE, enable_gqa=True)
    assert torch.allclose(out, ref.transpose(1, 2), atol=2e-6)


def test_sink_renormalisation_identity():
    """O_sink = O_nosink * exp(lse_nosink - logaddexp(lse_nosink, sink))."""
    q, k, v, sinks, _ = E.make_inputs(4, 1, 4, 2, 33, 64, torch.float64)
    out = E.eager_attention(q, k, v, sinks, SCALE, 7)
    nosink = torch.full_like(sinks, -1e4)
    o0 = E.eager_attention(q, k, v, nosink, SCALE, 7)
    lse0 = E.logsumexp_rows(q, k, nosink, SCALE, 7)
    lse1 = torch.logaddexp(lse0, sinks.view(1, -1, 1))
    assert torch.allclose(lse1, E.logsumexp_rows(q, k, sinks, SCALE, 7), atol=1e-12)
    factor = torch.exp(lse0 - lse1).permute(0, 2, 1).unsqueeze(-1)
    assert torch.allclose(out, o0 * factor, atol=1e-12)


def test_brute_force_loops():
    """Pure-Python triple loop on a tiny case, written from the definition."""
    b, h, g, s, d, w = 1, 4, 2, 9, 4, 3
    q, k, v, sinks, _ = E.make_inputs(5, b, h, g, s, d, torch.float64)
    out = E.eager_attention(q, k, v, sinks, 0.5, w)
    lse = E.logsumexp_rows(q, k, sinks, 0.5, w)
    for hh in range(h):
        kvh = hh // (h // g)
        for i in range(s):
            js = [j for j in range(s) if j <= i and j > i - w]
            assert len(js) == min(i + 1, w)
            logits = [0.5 * sum(float(q[0, hh, i, e]) * float(k[0, kvh, j, e]) for e in range(d)) for j in js]
            z = sum(math.exp(x) for x in logits) + math.exp(float(sinks[hh]))
            assert math.isclose(math.log(z), float(lse[0, hh, i]), rel_tol=1e-12, abs_tol=1e-12)
            for e in range(d):
                acc = sum(math.exp(x) / z * float(v[0, kvh, j, e]) for x, j in zip(logits, js))
                assert math.isclose(acc, float(out[0, i, hh, e]), rel_tol=1e-10, abs_tol=1e-12)


def test_window_one_and_first_row_closed_form():
    """W=1: O_i = sigmoid(s_ii - sink) v_i; row 0 of any layer obeys the same form."""
    q, k, v, sinks, _ = E.make_inputs(6, 1, 4, 4, 12, 64, torch.float64)
    out = E.eager_attention(q, k, v, sinks, SCALE, 1)
    sii = (q * k).sum(-1) * SCALE                      # (1,H,S) since G == H
    gate = torch.sigmoid(sii - sinks.view(1, -1, 1))
    assert torch.allclose(out, (gate.unsqueeze(-1) * v).transpose(1, 2), atol=1e-12)
    full = E.eager_attention(q, k, v, sinks, SCALE, None)
    assert torch.allclose(full[:, 0], out[:, 0], atol=1e-12)


def test_window_ge_seq_is_full_causal():
    q, k, v, sinks, _ = E.make_inputs(7, 1, 8, 2, 50, 64)
    a = E.eager_attention(q, k, v, sinks, SCALE, None)
    for w in (50, 51, 4096):
        assert torch.equal(a, E.eager_attention(q, k, v, sinks, SCALE, w))
    assert not torch.allclose(a, E.eager_attention(q, k, v, sinks, SCALE, 49))


def test_gqa_equals_mha_on_repeated_kv():
    q, k, v, sinks, d_out = E.make_inputs(8, 1, 8, 2, 20, 64, torch.float64)
    out, dq, dk, dv, ds = E.eager_attention_grads(q, k, v, sinks, d_out, SCALE, 6)
    kk, vv = k.repeat_interleave(4, 1), v.repeat_interleave(4, 1)
    out2, dq2, dk2, dv2, ds2 = E.eager_attention_grads(q, kk, vv, sinks, d_out, SCALE, 6)
    assert torch.allclose(out, out2, atol=1e-12) and torch.allclose(dq, dq2, atol=1e-12)
    assert torch.allclose(dk, dk2.view(1, 2, 4, 20, 64).sum(2), atol=1e-12)
    assert torch.allclose(dv, dv2.view(1, 2, 4, 20, 64).sum(2), atol=1e-12)
    assert torch.allclose(ds, ds2, atol=1e-12)


def test_dsinks_closed_form_and_jacobian_row_sum():
    """dSinks_h = -sum_i exp(sink-M_i) (dO_i . O_i); sum_j dS_ij + dSink_i = 0."""
    q, k, v, sinks, d_out = E.make_inputs(9, 2, 4, 2, 24, 64, torch.float64)
    out, dq, dk, dv, ds = E.eager_attention_grads(q, k, v, sinks, d_out, SCALE, 10)
    lse = E.logsumexp_rows(q, k, sinks, SCALE, 10)
    delta = (out * d_out).sum(-1).permute(0, 2, 1)                     # (B,H,S)
    closed = -(torch.exp(sinks.view(1, -1, 1) - lse) * delta).sum((0, 2))
    assert torch.allclose(ds, closed, atol=1e-12)


def test_gradcheck_fp64():
    q, k, v, sinks, _ = E.make_inputs(10, 1, 4, 2, 6, 4, torch.float64)
    args = [t.requires_grad_(True) for t in (q, k, v, sinks)]
    assert torch.autograd.gradcheck(lambda a, b_, c, s_: E.eager_attention(a, b_, c, s_, 0.5, 3), args, atol=1e-7)


def test_none_sinks_means_zero_logit():
    q, k, v, _, _ = E.make_inputs(11, 1, 4, 2, 10, 64)
    assert torch.equal(E.eager_attention(q, k, v, None, SCALE), E.eager_attention(q, k, v, torch.zeros(4), SCALE))


def test_q_offset_matches_suffix_of_longer_sequence():
    """Sq < Skv with q_offset: the rows equal the last rows of the square problem."""
    q, k, v, sinks, _ = E.make_inputs(12, 1, 4, 2, 30, 64)
    for w in (None, 7):
        full = E.eager_attention(q, k, v, sinks, SCALE, w)
        part = E.eager_attention(q[:, :, 18:], k, v, sinks, SCALE, w, q_offset=18)
        assert torch.allclose(full[:, 18:], part, atol=1e-6)


def test_pair_count_and_flops():
    assert E.pair_count(16384, None) == 134225920 and E.pair_count(16384, 128) == 2089024
    assert E.pair_count(4096, 128) == 516160 and E.pair_count(256, 32) == 7696
    assert E.allowed_mask(256, 256, 32).sum().item() == 7696
    f = E.attention_flops(1, 64, 64, E.pair_count(16384, None))
    assert abs(f["total"] - 7.697e12) / 7.697e12 < 1e-3


@pytest.mark.parametrize("name", ["tiny_packed_full", "tiny_packed_win8"])
def test_golden_packed_sequences(golden_dir, name):
    """Packed rows: transformers builds the same-document mask from position ids; the oracle
    takes the equivalent document-start index per token."""
    z, seed, b, h, g, s, d, w, sl = _load(golden_dir, name)
    ds = E.doc_start_from_lengths(z["doc_lens"].tolist(), s)
    q, k, v, sinks, d_out = E.make_inputs(seed, b, h, g, s, d)
    got = E.eager_attention_grads(q, k, v, sinks, d_out, SCALE, w, 0, None, ds)
    for name_, mine, gold in zip(("out", "dq", "dk", "dv", "dsinks"), got, (z["out"], z["dq"], z["dk"], z["dv"], z["dsinks"])):
        gold = torch.as_tensor(gold)
        assert torch.allclose(mine, gold, rtol=1e-4, atol=2e-5), (name_, float((mine - gold).abs().max()))
    # and it differs from the unpacked result, so the fixture does exercise the document mask
    plain = E.eager_attention(q, k, v, sinks, SCALE, w)
    assert not torch.allclose(plain, got[0], atol=1e-3)


def test_packed_row_equals_separate_documents():
    """Each document of a packed row attends as if it were alone."""
    lens = [7, 12, 5]
    q, k, v, sinks, _ = E.make_inputs(13, 1, 4, 2, 24, 64, torch.float64)
    ds = E.doc_start_from_lengths([lens], 24)
    for w in (None, 4):
        packed = E.eager_attention(q, k, v, sinks, SCALE, w, doc_start=ds)
        pos = 0
        for n in lens:
            alone = E.eager_attention(q[:, :, pos:pos + n], k[:, :, pos:pos + n], v[:, :, pos:pos + n], sinks, SCALE, w)
            assert torch.allclose(packed[:, pos:pos + n], alone, atol=1e-12)
            pos += n
