"""Seeded sweep over irregular problems: odd group sizes (3 or 5 query heads per KV head), row
lengths that are not multiples of any tile, windows on either side of the tile sizes, decode-style
offsets with more keys than queries, right-padded and packed rows, shifted sink logits, tensors
delivered as transposed views.  Both tensor dtypes.

What is compared, per case (bf16 tolerances as in test_gpu_parity, fp32 as in test_gpu_float32):
  * forward: O and lse against the eager oracle on the same inputs;
  * backward: dQ, dK, dV, dSinks against the tiled oracle's backward evaluated from the SAME saved
    O and lse the kernels were given.  The backward is a function of (q, k, v, sinks, O, lse, dO)
    (attention_kernel.py:264, :276-344 work from the saved bf16 O as well); stated this way the
    comparison is well conditioned for every case of the sweep.  End to end (against autograd through
    the eager oracle) delta = rowsum(dO * O) taken from a bf16-rounded O loses all relative accuracy
    in dQ when every row keeps a single key with probability ~1 (window 1, sink logit far below),
    and in a dSinks that is the cancelling sum of a few rows; test_gpu_parity holds the end-to-end
    comparisons on well-conditioned problems.
"""
import random

import pytest
import torch

from oracle import eager_ref as E
from oracle import tiled as T

import test_gpu_float32 as TF
import test_gpu_parity as TP

pytestmark = pytest.mark.gpu

DEV = "cuda"
N_CASES = 96


def draw_case(case):
    rng = random.Random(7919 * case + 13)
    r = rng.choice([1, 2, 3, 4, 5, 8])
    g = rng.choice([1, 2, 3, 8]) if r < 8 else rng.choice([1, 2, 8])
    b = rng.choice([1, 1, 2, 3])
    sq = rng.randint(1, rng.choice([70, 200, 600] if r * g * b > 16 else [70, 200, 600, 1500]))
    mode = rng.choice(["plain", "plain", "offset", "padded", "packed"])
    q_offset, skv, seqlens, lens = 0, sq, None, None
    if mode == "offset":
        q_offset = rng.randint(1, 200)
        skv = sq + q_offset + rng.choice([0, 0, rng.randint(1, 70)])
    w = rng.choice([None, None, 1, 2, 17, 64, 127, 128, 129, rng.randint(1, sq + 64)])
    dt = torch.float32 if rng.random() < 0.25 else torch.bfloat16
    shift = rng.choice([-8.0, 4.0]) if rng.random() < 0.3 else 0.0
    if mode == "padded":
        seqlens = [rng.randint(1, sq) for _ in range(b)]
        seqlens[rng.randrange(b)] = sq
    if mode == "packed":
        lens = []
        for _ in range(b):
            cuts = sorted(set(rng.randint(1, sq - 1) for _ in range(rng.randint(0, min(6, sq - 1))))) if sq > 1 else []
            lens.append([hi - lo for lo, hi in zip([0] + cuts, cuts + [sq])])
    views = (rng.random() < 0.5, rng.random() < 0.3)
    return dict(b=b, h=r * g, g=g, sq=sq, skv=skv, w=w, q_offset=q_offset, seqlens=seqlens, lens=lens, dt=dt,
                shift=shift, views=views)


@pytest.mark.parametrize("case", range(N_CASES))
def test_random_problem(case):
    import oregon_gpt_oss_patching_amd as A
    c = draw_case(case)
    b, sq, w, q_offset, seqlens, dt = c["b"], c["sq"], c["w"], c["q_offset"], c["seqlens"], c["dt"]
    q, k, v, sinks, d_out = E.make_inputs(5000 + case, b, c["h"], c["g"], sq, 64, dt, skv=c["skv"])
    sinks = (sinks + c["shift"]).to(dt)
    if seqlens is not None:
        d_out = TP.mask_dout(d_out, seqlens)
    ds = E.doc_start_from_lengths(c["lens"], sq) if c["lens"] is not None else None
    qd, kd, vd, sd, dod = (t.to(DEV) for t in (q, k, v, sinks, d_out))
    if c["views"][0]:       # value as the model delivers it: a transposed view of (B, S, G, D)
        vd = vd.transpose(1, 2).contiguous().transpose(1, 2)
    if c["views"][1]:
        qd = qd.transpose(1, 2).contiguous().transpose(1, 2)
        kd = kd.transpose(1, 2).contiguous().transpose(1, 2)
    dsd = ds.to(DEV) if ds is not None else None
    print(c, flush=True)
    o, lse = A.attention_forward(qd, kd, vd, sd, TP.SCALE, w, q_offset, seqlens, dsd)
    dq, dk, dv, dsk = A.attention_backward(qd, kd, vd, sd, o, lse, dod, TP.SCALE, w, q_offset, seqlens, doc_start=dsd)
    torch.cuda.synchronize()
    o, lse, dq, dk, dv, dsk = (t.cpu() for t in (o, lse, dq, dk, dv, dsk))

    wide = torch.float64 if dt == torch.float32 else torch.float32
    f = [t.to(wide) for t in (q, k, v, sinks, d_out)]
    ro = E.eager_attention(f[0], f[1], f[2], f[3], TP.SCALE, w, q_offset, seqlens, ds)
    rlse = E.logsumexp_rows(f[0], f[1], f[3], TP.SCALE, w, q_offset, seqlens, ds)
    tdq, tdk, tdv, tds, _ = T.tiled_bwd(q, k, v, sinks, o, lse, d_out, TP.SCALE, w, q_offset, seqlens, ds)
    if dt == torch.float32:
        TF.compare([o, lse, dq, dk, dv, dsk], [ro, rlse, tdq.double(), tdk.double(), tdv.double(), tds.double()])
    else:
        TP.compare_all((o, lse, dq, dk, dv, dsk), (ro, rlse, tdq, tdk, tdv, tds))
