"""gptoss_attn_bwd_static -- the backward that allocates nothing and brings its own scratch --
against gptoss_attn_bwd on the same inputs, through the C ABI: two calls in a row on one GPU,
the second on a smaller problem, so that what the first call left in the shared array is there
when the second one runs.  Bit-for-bit where gptoss_attn_bwd takes the same sums (dQ, dSinks; dK / dV
of long full-causal rows); at the bf16 tolerance of the parity tests where it adds fp32 partial sums
that the no-alloc variant has no room for (key blocks of short rows cut into slices, seam tiles
between the chunks of a sliding-window layer)."""
import ctypes

import pytest
import torch

from oracle import eager_ref as E

pytestmark = pytest.mark.gpu

SCALE = 0.125
DEV = "cuda"


def _backward_both(b, h, g, s, window, seed, dtype=torch.bfloat16, lens=None):
    from oregon_gpt_oss_patching_amd import _lib
    from oregon_gpt_oss_patching_amd import attention_kernel as ak
    lib = _lib.load()
    q, k, v, sinks, d_out = E.make_inputs(seed, b, h, g, s, 64, dtype)
    if lens is not None:
        qvalid = (torch.arange(s).view(1, s) < torch.tensor(lens).view(b, 1)).view(b, s, 1, 1)
        d_out = d_out * qvalid
    q, k, v, sinks, d_out = (t.to(DEV) for t in (q, k, v, sinks, d_out))
    sl = None if lens is None else torch.tensor(lens, dtype=torch.int32, device=DEV)
    o, lse = ak.attention_forward(q, k, v, sinks, SCALE, window, 0, lens)
    s32 = sinks.float().contiguous()
    stream = torch.cuda.current_stream().cuda_stream
    results = []
    for name in ("gptoss_attn_bwd", "gptoss_attn_bwd_static"):
        p = ak._base_params(q, k, v, s32, sl, SCALE, window, 0)
        p.o, p.lse, p.d_o = o.data_ptr(), lse.data_ptr(), d_out.data_ptr()
        ak._set(p.o_stride, ak._strides_bhs(o, "bshd"))
        ak._set(p.do_stride, ak._strides_bhs(d_out, "bshd"))
        # outputs start as NaN patterns: an element the call does not write shows up
        dq = torch.full_like(q, float("nan"))
        dk = torch.full_like(k, float("nan"))
        dv = torch.full_like(v, float("nan"))
        ds = torch.full((h,), float("nan"), dtype=torch.float32, device=DEV)
        p.dq, p.dk, p.dv, p.dsinks = dq.data_ptr(), dk.data_ptr(), dv.data_ptr(), ds.data_ptr()
        ak._set(p.dq_stride, ak._strides_bhs(dq, "bhsd"))
        ak._set(p.dk_stride, ak._strides_bhs(dk, "bhsd"))
        ak._set(p.dv_stride, ak._strides_bhs(dv, "bhsd"))
        parts_cut = False
        if name == "gptoss_attn_bwd":
            need = lib.gptoss_attn_workspace_bytes(ctypes.byref(p))
            parts_cut = need > (8 + 16) * b * h * s + 16      # more than the row statistics: partial sums
            delta = torch.empty((need // 4,), dtype=torch.float32, device=DEV)
            p.delta = delta.data_ptr()
        else:
            p.delta = None                      # the caller brings no scratch at all
        _lib.call(name, p, stream)
        torch.cuda.synchronize()
        results.append((dq, dk, dv, ds))
        if name == "gptoss_attn_bwd":
            cut = parts_cut
    return results[0], results[1], cut


def _compare(ref, got, cut):
    for name, r, t in zip(("dq", "dk", "dv", "dsinks"), ref, got):
        assert torch.isfinite(t).all(), name
        if cut and name in ("dk", "dv"):
            err = (t.float() - r.float()).abs()
            assert bool((err <= 2e-2 + 2.0 ** -8 * r.float().abs()).all()), (name, float(err.max()))
            assert float((t.double() - r.double()).norm() / r.double().norm()) <= 1e-2, name
        else:
            assert torch.equal(t, r), name


@pytest.mark.parametrize("window", [128, None])
def test_static_scratch_backward_matches_workspace_backward(window):
    from oregon_gpt_oss_patching_amd import _lib
    lib = _lib.load()
    assert lib.gptoss_attn_static_scratch_bytes() == 48 << 20
    print(f"no-alloc backward, window={window}: first call B=2 H=64 G=8 S=2048", flush=True)
    ref, got, cut = _backward_both(2, 64, 8, 2048, window, 11)
    _compare(ref, got, cut)
    print(f"no-alloc backward, window={window}: second call B=1 H=8 G=2 S=333 (smaller)", flush=True)
    ref, got, cut = _backward_both(1, 8, 2, 333, window, 12)
    _compare(ref, got, cut)


@pytest.mark.parametrize("b,h,g,s,window,dtype,lens", [
    (2, 8, 2, 300, None, torch.float32, None),           # float32 tensors: preprocess + dK/dV + dQ on the built-in scratch
    (2, 8, 2, 300, 64, torch.float32, [300, 1]),
    (2, 16, 4, 1300, 128, torch.bfloat16, [1300, 1]),    # padded rows in the window kernel's walk past its chunk:
    (2, 16, 4, 1300, 128, torch.bfloat16, [64, 1300]),   # whole chunks and their neighbour tiles lie in the padding
    (2, 16, 4, 1300, 128, torch.bfloat16, [1299, 129]),
    (1, 17, 1, 200, 128, torch.bfloat16, None),          # 17 query heads per KV head: dQ + dK/dV kernels, static scratch
    (1, 4, 4, 200, 128, torch.bfloat16, None),           # one query head per KV head: the same fallback
    (2, 17, 1, 200, None, torch.bfloat16, [200, 77]),
    (1, 64, 8, 16384, None, torch.bfloat16, None),       # the headline layer: 64-key dK/dV kernel, 24 of the 48 MiB in use
    (9, 8, 8, 1024, None, torch.bfloat16, [1024, 1000, 960, 7, 64, 65, 512, 513, 1]),   # the same kernel with padded rows
])
def test_static_scratch_backward_other_routes(b, h, g, s, window, dtype, lens):
    """The routes the two-call test above does not take, each against gptoss_attn_bwd: float32 tensors,
    right-padded rows in the single-pass window kernel's no-seam walk (every workgroup walks two query
    tiles past its chunk and drops the dK/dV of the two tiles before it), and group sizes the
    single-pass kernel does not take.  Padded positions must be exactly zero."""
    print(f"no-alloc backward: B={b} H={h} G={g} S={s} W={window} {dtype} lens={lens}", flush=True)
    ref, got, cut = _backward_both(b, h, g, s, window, 13, dtype, lens)
    single_pass = dtype == torch.bfloat16 and window is not None and window <= 128 and 2 <= h // g <= 16
    _compare(ref, got, cut or single_pass)
    if lens is not None:
        for i, n in enumerate(lens):
            if n < s:
                for t in got[:3]:
                    assert float(t[i, :, n:].abs().max()) == 0.0


def test_static_scratch_refuses_what_does_not_fit():
    """24 bytes of row statistics per row beyond the built-in array: refused on the host, nothing launched."""
    from oregon_gpt_oss_patching_amd import _lib
    from oregon_gpt_oss_patching_amd import attention_kernel as ak
    b, h, g, s = 1, 64, 8, 16384
    q = torch.empty(b, h, s, 64, dtype=torch.bfloat16, device=DEV)
    k = torch.empty(b, g, s, 64, dtype=torch.bfloat16, device=DEV)
    p = ak._base_params(q, k, k, None, None, SCALE, 0, 0)
    for f in ("o", "d_o", "dq"):
        setattr(p, f, q.data_ptr())
    p.lse = q.data_ptr()
    p.dk = p.dv = k.data_ptr()
    for f in ("o_stride", "do_stride"):
        ak._set(getattr(p, f), ak._strides_bhs(q.transpose(1, 2), "bshd"))
    for f in ("dq_stride",):
        ak._set(getattr(p, f), ak._strides_bhs(q, "bhsd"))
    for f in ("dk_stride", "dv_stride"):
        ak._set(getattr(p, f), ak._strides_bhs(k, "bhsd"))
    p.B = 3                                           # 3 * 64 * 16384 rows: 75 MB of statistics
    p.q_stride.b = p.k_stride.b = p.v_stride.b = 0
    with pytest.raises(_lib.GptossAttnError) as ei:
        _lib.call("gptoss_attn_bwd_static", p, 0)
    assert ei.value.status == -10
