"""The Python drop-in surface on the GPU: autograd.Function, the Hugging Face
adapter with tensors laid out as GptOssAttention.forward delivers them, output
layout, and the patched model path."""
from types import SimpleNamespace

import pytest
import torch

from oracle import eager_ref as E

pytestmark = pytest.mark.gpu
SCALE = 0.125
DEV = "cuda"


def rel_l2(a, b):
    return float((a.double() - b.double()).norm() / (b.double().norm() + 1e-30))


def test_autograd_function_matches_oracle():
    import oregon_gpt_oss_patching_amd as A
    for w in (None, 32):
        q, k, v, sinks, d_out = E.make_inputs(5, 2, 8, 2, 192, 64, torch.bfloat16)
        ref = E.eager_attention_grads(q.float(), k.float(), v.float(), sinks.float(), d_out.float(), SCALE, w)
        qd, kd, vd, sd = (t.to(DEV).requires_grad_(True) for t in (q, k, v, sinks))
        out = A.attention(qd, kd, vd, sd, SCALE, w, None)
        assert out.shape == (2, 192, 8, 64) and out.is_contiguous()
        out.backward(d_out.to(DEV))
        assert sd.grad.dtype == sd.dtype and sd.grad.shape == sd.shape
        for g, r in zip((out, qd.grad, kd.grad, vd.grad, sd.grad), ref):
            assert rel_l2(g.detach().float().cpu(), r) < 1e-2


def test_hf_adapter_with_model_layouts():
    """q, k contiguous (B,H,S,D); v a transposed view of (B,S,G,D); sinks a bf16
    Parameter; attention_mask given but ignored; output (B,S,H,D) contiguous."""
    import oregon_gpt_oss_patching_amd as A
    b, h, g, s = 2, 16, 4, 160
    q, k, v, sinks, d_out = E.make_inputs(6, b, h, g, s, 64, torch.bfloat16)
    ref = E.eager_attention_grads(q.float(), k.float(), v.float(), sinks.float(), d_out.float(), SCALE, 128)
    qd, kd = q.to(DEV).requires_grad_(True), k.to(DEV).requires_grad_(True)
    v_bsgd = v.transpose(1, 2).contiguous().to(DEV).requires_grad_(True)
    vd = v_bsgd.transpose(1, 2)
    assert not vd.is_contiguous()
    module = SimpleNamespace(sinks=torch.nn.Parameter(sinks.to(DEV)), sliding_window=128, training=True)
    mask = torch.zeros(b, 1, s, s, device=DEV, dtype=torch.bfloat16)
    out, weights = A.triton_flash_attention(module, qd, kd, vd, mask, SCALE, dropout=0.0, sliding_window=128, s_aux=module.sinks)
    assert weights is None and out.shape == (b, s, h, 64) and out.is_contiguous()
    out.reshape(b, s, -1).backward(d_out.to(DEV).reshape(b, s, -1))
    got = (out, qd.grad, kd.grad, v_bsgd.grad.transpose(1, 2), module.sinks.grad)
    for gt, r in zip(got, ref):
        assert rel_l2(gt.detach().float().cpu(), r) < 1e-2


def test_frozen_sinks_skip_dsinks():
    import oregon_gpt_oss_patching_amd as A
    q, k, v, sinks, d_out = E.make_inputs(7, 1, 8, 2, 64, 64, torch.bfloat16)
    qd, kd, vd = (t.to(DEV).requires_grad_(True) for t in (q, k, v))
    sd = sinks.to(DEV)      # requires_grad False, as under LoRA
    out = A.attention(qd, kd, vd, sd, SCALE, None, None)
    out.backward(d_out.to(DEV))
    assert sd.grad is None and qd.grad is not None


def test_gradient_checkpoint_recompute_is_stable():
    import torch.utils.checkpoint as cp
    import oregon_gpt_oss_patching_amd as A
    q, k, v, sinks, d_out = E.make_inputs(8, 1, 8, 2, 128, 64, torch.bfloat16)
    qd, kd, vd, sd = (t.to(DEV).requires_grad_(True) for t in (q, k, v, sinks))
    out = cp.checkpoint(lambda a, b_, c, s_: A.attention(a, b_, c, s_, SCALE, 32, None), qd, kd, vd, sd, use_reentrant=False)
    out.backward(d_out.to(DEV))
    g1 = [t.grad.clone() for t in (qd, kd, vd, sd)]
    for t in (qd, kd, vd, sd):
        t.grad = None
    A.attention(qd, kd, vd, sd, SCALE, 32, None).backward(d_out.to(DEV))
    for a, t in zip(g1, (qd, kd, vd, sd)):
        assert torch.equal(a, t.grad)


def test_patched_gpt_oss_layer_matches_eager():
    """patch_flash_attention() swaps the function GptOssAttention calls; a 2-layer
    GPT-OSS-shaped model (one sliding, one full layer) must give, patched, a loss
    and gradients at least as close to an fp32 eager run as the unpatched bf16 run is."""
    from transformers import GptOssConfig, GptOssForCausalLM
    from oregon_gpt_oss_patching_amd import patching
    cfg = GptOssConfig(vocab_size=512, hidden_size=256, intermediate_size=256, num_hidden_layers=2,
                       num_attention_heads=16, num_key_value_heads=4, head_dim=64, num_local_experts=2,
                       num_experts_per_tok=2, sliding_window=32, max_position_embeddings=512,
                       layer_types=["sliding_attention", "full_attention"], attn_implementation="eager")
    # top-k == number of experts: routing stays continuous, so bf16-level differences in the
    # attention output cannot flip an expert choice and turn into an O(1) gradient change
    torch.manual_seed(0)
    model = GptOssForCausalLM(cfg).to(DEV, torch.bfloat16)
    with torch.no_grad():
        for name, prm in model.named_parameters():
            if name.endswith("sinks"):
                prm.copy_(torch.randn_like(prm))
    ids = torch.randint(0, 512, (2, 200), device=DEV)

    def run(m):
        m.zero_grad(set_to_none=True)
        out = m(input_ids=ids, labels=ids)
        out.loss.backward()
        grads = {n: p.grad.detach().float().clone() for n, p in m.named_parameters() if p.grad is not None}
        return float(out.loss.detach()), grads

    # ground truth: the same weights in fp32 through the unpatched eager path
    import copy
    loss_t, g_t = run(copy.deepcopy(model).float())
    loss_e, g_e = run(model)                      # bf16 eager (softmax in bf16)
    patching.patch_flash_attention()
    try:
        loss_p, g_p = run(model)                  # bf16 with the HIP kernels
    finally:
        patching.unpatch_flash_attention()
    assert abs(loss_p - loss_t) < 2e-2 * max(1.0, abs(loss_t)), (loss_t, loss_e, loss_p)
    # the patched gradients must be about as close to the fp32 truth as bf16 eager is
    # (both runs carry the bf16 noise of every other layer, hence the factor 2)
    for n in g_t:
        if g_t[n].norm() > 1e-6:
            err_e, err_p = rel_l2(g_e[n], g_t[n]), rel_l2(g_p[n], g_t[n])
            # dSinks is a heavily cancelling sum over rows of exp(sink-lse) * (dO . O) taken from
            # the bf16-rounded O; where it nearly cancels (tiny gradient) the rounding noise of
            # either bf16 path is a visible fraction of it, so sinks get a wider band.
            bound = max(4.0 * err_e, 0.25) if n.endswith("sinks") else max(2.0 * err_e, 5e-2)
            assert err_p < bound, (n, err_p, err_e)


def _tiny_lora_model():
    from oregon_gpt_oss_patching_amd import sft_bench
    model = sft_bench.build_model(layers=2, hidden=256, heads=16, kv_heads=4, experts=2, top_k=2, vocab=512,
                                  window=32, device=DEV)
    params = sft_bench.add_lora(model, r=8, alpha=16.0)
    return sft_bench, model, params


def test_lora_decoder_step_patched_vs_eager():
    """The training harness on a 2-layer S=512 cut: loss and LoRA gradient norm of one
    step agree between the eager and the patched model (bf16 tolerance)."""
    from oregon_gpt_oss_patching_amd import patching
    sft_bench, model, params = _tiny_lora_model()
    assert all("lora_" in n for n, p in model.named_parameters() if p.requires_grad)
    ids = torch.randint(0, 512, (2, 512), device=DEV)
    # make the adapters non-trivial so q/k/v/o gradients flow through both factors
    with torch.no_grad():
        for n, p in model.named_parameters():
            if "lora_b" in n:
                p.copy_(0.02 * torch.randn_like(p))

    def step(mask=None):
        model.zero_grad(set_to_none=True)
        out = model(input_ids=ids, labels=ids, attention_mask=mask)
        out.loss.backward()
        gn = torch.sqrt(sum((p.grad.float() ** 2).sum() for p in params))
        return float(out.loss.detach()), float(gn)

    loss_e, gn_e = step()
    patching.patch_flash_attention()
    try:
        loss_p, gn_p = step()
        loss_m, gn_m = step(sft_bench.mask_free_attention_mask(None))      # no dense masks built
    finally:
        patching.unpatch_flash_attention()
    assert abs(loss_p - loss_e) < 2e-2 * abs(loss_e), (loss_e, loss_p)
    assert abs(gn_p - gn_e) < 5e-2 * gn_e, (gn_e, gn_p)
    assert loss_m == loss_p and gn_m == gn_p        # the kernels never read the dense masks


def test_mask_free_padding_path_matches_masked_model():
    """A right-padded batch: valid lengths passed in place of the dense masks give the same
    loss on valid tokens as the stock eager model given the 2-D padding mask."""
    from oregon_gpt_oss_patching_amd import patching
    sft_bench, model, params = _tiny_lora_model()
    b, s = 2, 256
    ids = torch.randint(0, 512, (b, s), device=DEV)
    lens = torch.tensor([256, 97], device=DEV)
    pad = (torch.arange(s, device=DEV).view(1, s) < lens.view(b, 1))
    labels = ids.masked_fill(~pad, -100)
    model.eval()
    with torch.no_grad():
        loss_e = float(model(input_ids=ids, labels=labels, attention_mask=pad.long()).loss)
        patching.patch_flash_attention()
        try:
            loss_p = float(model(input_ids=ids, labels=labels,
                                 attention_mask=sft_bench.mask_free_attention_mask(pad)).loss)
        finally:
            patching.unpatch_flash_attention()
    assert abs(loss_p - loss_e) < 2e-2 * abs(loss_e), (loss_e, loss_p)


def test_float16_tensors_are_accepted_at_bf16_accuracy():
    """float16 tensors are rounded to bfloat16 on the way in and the results cast back."""
    import oregon_gpt_oss_patching_amd as A
    q, k, v, sinks, d_out = E.make_inputs(1, 1, 8, 2, 256, 64, torch.float16)
    for w in (None, 32):
        ref = E.eager_attention_grads(q.float(), k.float(), v.float(), sinks.float(), d_out.float(), SCALE, w)
        qd, kd, vd, sd = (t.to(DEV).requires_grad_(True) for t in (q, k, v, sinks))
        out = A.attention(qd, kd, vd, sd, SCALE, w, None)
        assert out.dtype == torch.float16
        out.backward(d_out.to(DEV))
        for g, r in zip((out, qd.grad, kd.grad, vd.grad, sd.grad), ref):
            assert g.dtype == torch.float16
            assert rel_l2(g.detach().float().cpu(), r) < 1e-2


def test_custom_ops_are_registered_and_match_the_direct_calls():
    """`gptoss_attn::fwd` / `gptoss_attn::bwd` are what the autograd.Function runs; they must equal
    the direct library calls bit for bit, and their shape-only implementations must agree with
    the real ones (torch.library.opcheck)."""
    import oregon_gpt_oss_patching_amd as A
    q, k, v, sinks, d_out = (t.to(DEV) for t in E.make_inputs(9, 1, 8, 2, 130, 64, torch.bfloat16))
    o, lse = torch.ops.gptoss_attn.fwd(q, k, v, sinks, SCALE, 32, 0, None, None)
    o2, lse2 = A.attention_forward(q, k, v, sinks, SCALE, 32)
    assert torch.equal(o, o2) and torch.equal(lse, lse2)
    got = torch.ops.gptoss_attn.bwd(q, k, v, sinks, o, lse, d_out, SCALE, 32, 0, None, None, True)
    ref = A.attention_backward(q, k, v, sinks, o, lse, d_out, SCALE, 32)
    for g, r in zip(got, ref):
        assert torch.equal(g, r)
    assert torch.ops.gptoss_attn.bwd(q, k, v, sinks, o, lse, d_out, SCALE, 32, 0, None, None, False)[3].numel() == 0
    torch.library.opcheck(torch.ops.gptoss_attn.fwd.default, (q, k, v, sinks, SCALE, 32, 0, None, None),
                          test_utils=("test_schema", "test_faketensor"))
    torch.library.opcheck(torch.ops.gptoss_attn.bwd.default, (q, k, v, sinks, o, lse, d_out, SCALE, 32, 0, None, None, True),
                          test_utils=("test_schema", "test_faketensor"))


@pytest.mark.parametrize("window", [None, 128])
def test_torch_compile_traces_the_custom_ops(window):
    """torch.compile (dynamo + AOT autograd, backend "aot_eager", fullgraph) over attention(): the two
    library calls are opaque custom operators with shape-only implementations, so the traced
    program calls them unchanged and forward and gradients have the bits of the eager call."""
    import oregon_gpt_oss_patching_amd as A
    q, k, v, sinks, d_out = E.make_inputs(14, 2, 16, 2, 384, 64, torch.bfloat16)
    d_out = d_out.to(DEV)

    def fn(q_, k_, v_, s_):
        return A.attention(q_, k_, v_, s_, SCALE, window, None)

    eager_in = [t.to(DEV).requires_grad_(True) for t in (q, k, v, sinks)]
    out_e = fn(*eager_in)
    out_e.backward(d_out)
    torch._dynamo.reset()
    compiled = torch.compile(fn, backend="aot_eager", fullgraph=True)
    comp_in = [t.to(DEV).requires_grad_(True) for t in (q, k, v, sinks)]
    out_c = compiled(*comp_in)
    out_c.backward(d_out)
    torch.cuda.synchronize()
    assert torch.equal(out_c, out_e)
    for a, b in zip(comp_in, eager_in):
        assert torch.equal(a.grad, b.grad)


def test_packed_rows_through_the_patched_model():
    """Packed rows (position ids restarting inside a row).  The stock GPT-OSS eager path of this
    transformers version does not pass position ids to its mask builder, so, like the reference,
    it lets documents see each other; the default patch must match it.  With
    respect_packing=True the patched model must instead match the eager model given
    transformers' own same-document masks."""
    from transformers import masking_utils as mu
    from oregon_gpt_oss_patching_amd import patching
    sft_bench, model, params = _tiny_lora_model()
    s = 192
    ids = torch.randint(0, 512, (1, s), device=DEV)
    lens = [50, 100, 42]
    pos = torch.tensor([[p for n in lens for p in range(n)]], device=DEV)
    packed = mu.find_packed_sequence_indices(pos.cpu())
    doc = mu.packed_sequence_mask_function(packed)
    masks = {
        "full_attention": mu.eager_mask(1, s, s, mask_function=mu.and_masks(mu.causal_mask_function, doc),
                                        dtype=torch.bfloat16).to(DEV),
        "sliding_attention": mu.eager_mask(1, s, s, mask_function=mu.and_masks(
            mu.sliding_window_causal_mask_function(model.config.sliding_window), doc), dtype=torch.bfloat16).to(DEV),
    }
    free = sft_bench.mask_free_attention_mask(None)
    model.eval()
    with torch.no_grad():
        ref_leaky = model(input_ids=ids, position_ids=pos).logits.float().cpu()
        ref_docs = model(input_ids=ids, position_ids=pos, attention_mask=masks).logits.float().cpu()
        patching.patch_flash_attention(respect_packing=True)
        try:
            got_docs = model(input_ids=ids, position_ids=pos, attention_mask=free).logits.float().cpu()
        finally:
            patching.unpatch_flash_attention()
        patching.patch_flash_attention()
        try:
            got_leaky = model(input_ids=ids, position_ids=pos, attention_mask=free).logits.float().cpu()
        finally:
            patching.unpatch_flash_attention()
    assert rel_l2(ref_docs[:, 60:], ref_leaky[:, 60:]) > 0.1          # the two semantics really differ
    assert rel_l2(got_leaky, ref_leaky) < 3e-2
    assert rel_l2(got_docs, ref_docs) < 3e-2


def test_hip_graph_capture_and_replay_match_eager_launches():
    """The library allocates nothing and never synchronises, so forward + backward can be
    captured in a HIP graph.  Three replays, with eager work and synchronisations in between,
    must reproduce the eager launches bit for bit (the kernels are deterministic)."""
    import oregon_gpt_oss_patching_amd as A
    q, k, v, sinks, d_out = (t.to("cuda") for t in E.make_inputs(321, 1, 16, 4, 384, 64, torch.bfloat16))
    for window in (None, 128):
        o_ref, lse_ref = A.attention_forward(q, k, v, sinks, 0.125, window)
        ref = (o_ref, lse_ref) + tuple(A.attention_backward(q, k, v, sinks, o_ref, lse_ref, d_out, 0.125, window))
        torch.cuda.synchronize()
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):                      # warm-up on the capture stream
            o, lse = A.attention_forward(q, k, v, sinks, 0.125, window)
            A.attention_backward(q, k, v, sinks, o, lse, d_out, 0.125, window)
        torch.cuda.current_stream().wait_stream(side)
        torch.cuda.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            o, lse = A.attention_forward(q, k, v, sinks, 0.125, window)
            outs = (o, lse) + tuple(A.attention_backward(q, k, v, sinks, o, lse, d_out, 0.125, window))
        for _ in range(3):
            for t in outs:
                t.fill_(float("nan"))                      # eager work between the replays
            torch.cuda.synchronize()
            graph.replay()
            torch.cuda.synchronize()
            for got, want in zip(outs, ref):
                assert torch.equal(got, want)


def test_hip_graph_replays_follow_a_query_offset_in_device_memory():
    """A start position that lives in device memory is read by the kernels at run time, so one
    captured graph serves different offsets: between replays only the int32 on the device changes
    (the reference's kernels read their start_q tensor the same way, attention_kernel.py:44-47).
    Every replay must equal the eager call with that offset passed by value."""
    import oregon_gpt_oss_patching_amd as A
    q, k, v, sinks, d_out = (t.to("cuda") for t in E.make_inputs(322, 1, 8, 2, 48, 64, torch.bfloat16, skv=160))
    off = torch.zeros(1, dtype=torch.int32, device="cuda")
    for window in (None, 32):
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):                      # warm-up on the capture stream
            o, lse = A.attention_forward(q, k, v, sinks, 0.125, window, q_offset_dev=off)
            A.attention_backward(q, k, v, sinks, o, lse, d_out, 0.125, window, q_offset_dev=off)
        torch.cuda.current_stream().wait_stream(side)
        torch.cuda.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            o, lse = A.attention_forward(q, k, v, sinks, 0.125, window, q_offset_dev=off)
            outs = (o, lse) + tuple(A.attention_backward(q, k, v, sinks, o, lse, d_out, 0.125, window, q_offset_dev=off))
        for start in (112, 0, 57):
            off.fill_(start)
            for t in outs:
                t.fill_(float("nan"))
            torch.cuda.synchronize()
            graph.replay()
            torch.cuda.synchronize()
            o_ref, lse_ref = A.attention_forward(q, k, v, sinks, 0.125, window, start)
            ref = (o_ref, lse_ref) + tuple(A.attention_backward(q, k, v, sinks, o_ref, lse_ref, d_out, 0.125, window, start))
            for got, want in zip(outs, ref):
                assert torch.equal(got, want), start


def test_mfma_rate_probe_runs_and_counts_its_mfmas():
    """The measurement aid bench.py uses: launches, returns the number of MFMA instructions it executes
    (two workgroups of four wavefronts per compute unit, 16 MFMAs per pass) and leaves finite sums."""
    import ctypes
    from oregon_gpt_oss_patching_amd import _lib
    lib = _lib.load()
    cus = torch.cuda.get_device_properties(0).multi_processor_count
    ops = torch.randn(4096, device="cuda").to(torch.bfloat16)
    sink = torch.full((512 * cus,), float("nan"), dtype=torch.float32, device="cuda")
    n = lib.gptoss_attn_mfma_rate_probe(ops.data_ptr(), ops.numel() * 2, 50, sink.data_ptr(), sink.numel(),
                                        torch.cuda.current_stream().cuda_stream)
    torch.cuda.synchronize()
    assert n == 2 * cus * 4 * 50 * 16
    assert bool(torch.isfinite(sink).all())
    assert lib.gptoss_attn_mfma_rate_probe(ops.data_ptr(), ops.numel() * 2, 50, sink.data_ptr(), 100, None) < 0   # sink too small


def test_stream_probe_runs_every_mix_and_counts_its_mfmas():
    """Every synthetic instruction stream launches at 1, 2 and 3 wavefronts per SIMD, returns the number of MFMAs it
    executes (48 per pass and wavefront, one workgroup per compute unit) and leaves the same finite number in every
    thread's sink slot (its operands are zero: 0 for the MFMA-only stream, a count of exp2(0) terms for the others);
    a sink that is too small is refused."""
    from oregon_gpt_oss_patching_amd import _lib
    lib = _lib.load()
    cus = torch.cuda.get_device_properties(0).multi_processor_count
    sink = torch.full((768 * cus,), float("nan"), dtype=torch.float32, device=DEV)
    for mix in range(6):
        for waves in (1, 2, 3):
            sink.fill_(float("nan"))
            n = lib.gptoss_attn_stream_probe(mix, waves, 7, sink.data_ptr(), sink.numel(), torch.cuda.current_stream().cuda_stream)
            torch.cuda.synchronize()
            assert n == cus * 4 * waves * 7 * 48, (mix, waves, n)
            got = sink[:256 * waves * cus]
            assert torch.isfinite(got).all() and (got == got[0]).all() and (mix != 0 or got[0] == 0), (mix, waves, got[0].item())
            assert torch.isnan(sink[256 * waves * cus:]).all()           # nothing written past the launch's own threads
    assert lib.gptoss_attn_stream_probe(0, 3, 7, sink.data_ptr(), 100, None) < 0
