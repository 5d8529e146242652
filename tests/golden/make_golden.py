"""Writes tests/golden/*.npz: outputs of the installed `transformers`
GPT-OSS eager attention (the function the reference monkeypatches away,
patching.py:4-7) on seeded inputs, so that the CPU oracle in oracle/ can be
pinned against the real thing without shipping it.

Run once, in the authoring container (needs `transformers`; nothing is fetched):

    python tests/golden/make_golden.py

The fixtures hold inputs' seed recipe and the expected outputs only.  The mask is
built by transformers' own `eager_mask` from its own mask functions, i.e. the
same additive finfo.min mask the model would hand to eager attention, including
the 2-D padding mask for the padded-batch cases and the same-document mask that
transformers derives from restarting position ids for the packed cases.
"""
import os
import sys
from types import SimpleNamespace

import numpy as np
import torch

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))

from oracle.eager_ref import make_inputs  # noqa: E402  (seed recipe only)

# packed rows: document lengths per batch row (position ids restart at each document)
PACKED = {"tiny_packed_full": [[20, 30, 14]], "tiny_packed_win8": [[5, 41, 18]]}

CASES = [
    # name, seed, B, H, G, S, D, window, seqlens
    ("tiny_full", 11, 1, 8, 2, 64, 64, None, None),
    ("tiny_win8", 12, 1, 8, 2, 64, 64, 8, None),
    ("tiny_pad_full", 13, 2, 8, 2, 48, 64, None, [48, 29]),
    ("tiny_pad_win8", 14, 2, 8, 2, 48, 64, 8, [17, 48]),
    ("tiny_packed_full", 15, 1, 8, 2, 64, 64, None, None),
    ("tiny_packed_win8", 16, 1, 8, 2, 64, 64, 8, None),
    ("cfg1_full", 1, 1, 8, 2, 256, 64, None, None),
    ("cfg1_win32", 1, 1, 8, 2, 256, 64, 32, None),
]


def run_case(seed, b, h, g, s, d, window, seqlens, doc_lens=None):
    from transformers import masking_utils as mu
    from transformers.models.gpt_oss import modeling_gpt_oss as mg

    q, k, v, sinks, d_out = make_inputs(seed, b, h, g, s, d, torch.float32)
    fn = mu.causal_mask_function if window is None else mu.sliding_window_causal_mask_function(window)
    if doc_lens is not None:
        # transformers' own packed-sequence detection from position ids (masking_utils.py:728-757)
        pos = torch.tensor([[p for n in lens for p in range(n)] for lens in doc_lens])
        packed = mu.find_packed_sequence_indices(pos)
        fn = mu.and_masks(fn, mu.packed_sequence_mask_function(packed))
    pad2d = None
    if seqlens is not None:
        pad2d = torch.arange(s).view(1, s) < torch.tensor(seqlens).view(b, 1)
    mask = mu.eager_mask(batch_size=b, q_length=s, kv_length=s, mask_function=fn,
                         attention_mask=pad2d, dtype=torch.float32)
    if seqlens is not None:
        # the op treats padded QUERY rows as seeing nothing; eager would let them
        # attend valid keys, so the comparison zeroes their incoming gradient.
        qvalid = pad2d.view(b, s, 1, 1).to(d_out.dtype)
        d_out = d_out * qvalid
    q.requires_grad_(True); k.requires_grad_(True); v.requires_grad_(True)
    sinks = sinks.clone().requires_grad_(True)
    module = SimpleNamespace(sinks=sinks, num_key_value_groups=h // g, training=False)
    out, _ = mg.eager_attention_forward(module, q, k, v, mask, 1.0 / 8.0)
    dq, dk, dv, ds = torch.autograd.grad(out, (q, k, v, sinks), d_out)
    return out.detach(), dq, dk, dv, ds


def main():
    for name, seed, b, h, g, s, d, window, seqlens in CASES:
        out, dq, dk, dv, ds = run_case(seed, b, h, g, s, d, window, seqlens, PACKED.get(name))
        meta = dict(seed=seed, B=b, H=h, G=g, S=s, D=d, window=window or 0,
                    seqlens=np.array(seqlens if seqlens else [], dtype=np.int32),
                    doc_lens=np.array(PACKED.get(name, []), dtype=np.int32))
        if s > 64:
            # config-1 size: keep norms and a fixed strided sample, not full tensors
            def samp(t):
                flat = t.reshape(-1)
                idx = torch.arange(0, flat.numel(), max(1, flat.numel() // 1024))[:1024]
                return flat[idx].numpy()
            arrs = {f"{n}_sample": samp(t) for n, t in
                    (("out", out), ("dq", dq), ("dk", dk), ("dv", dv))}
            arrs.update({f"{n}_norm": np.array(float(t.double().norm())) for n, t in
                         (("out", out), ("dq", dq), ("dk", dk), ("dv", dv))})
            arrs["dsinks"] = ds.numpy()
        else:
            arrs = dict(out=out.numpy(), dq=dq.numpy(), dk=dk.numpy(), dv=dv.numpy(), dsinks=ds.numpy())
        np.savez_compressed(os.path.join(HERE, f"{name}.npz"), **meta, **arrs)
        print("wrote", name, {k2: getattr(v2, "shape", None) for k2, v2 in arrs.items()})


if __name__ == "__main__":
    main()
