"""Training-throughput harness for a truncated GPT-OSS-shaped decoder with LoRA.

This is the counterpart of the reference's `sft.py` launcher for the part of it
that can run offline: the reference loads `openai/gpt-oss-20b` and a dataset by
name through TRL/PEFT (sft.py:30-50, configs/sft_lora.yaml), none of which is
available without a network.  Here the same model CLASS (Hugging Face
`GptOssForCausalLM`, `attn_implementation="eager"` as in configs/sft_lora.yaml:3)
is built from a local config with random bf16 weights, wrapped with a small LoRA
adapter on q/k/v/o, fed uniform random token ids, and trained for a few steps
twice: once with the stock eager attention and once with
`patch_flash_attention()` applied -- the comparison the reference's throughput
figure makes (README.md:20-22).

    python -m oregon_gpt_oss_patching_amd.sft_bench            # 4 layers, S=8192, B=1, LoRA r=16
    python -m oregon_gpt_oss_patching_amd.sft_bench --layers 2 --seq 512 --experts 4

Prints one JSON line with tokens/s for both paths.
"""
from __future__ import annotations

import argparse
import json
import math
import time

import torch
from torch import nn


class LoRALinear(nn.Module):
    """y = W x + b + (alpha / r) * B(A x); W, b frozen (what peft's LoRA does for a Linear)."""

    def __init__(self, base: nn.Linear, r: int, alpha: float):
        super().__init__()
        self.base = base
        for p in self.base.parameters():
            p.requires_grad_(False)
        self.lora_a = nn.Parameter(torch.empty(r, base.in_features, dtype=base.weight.dtype, device=base.weight.device))
        self.lora_b = nn.Parameter(torch.zeros(base.out_features, r, dtype=base.weight.dtype, device=base.weight.device))
        nn.init.kaiming_uniform_(self.lora_a, a=math.sqrt(5))
        self.scaling = alpha / r

    def forward(self, x):
        return self.base(x) + (x @ self.lora_a.t() @ self.lora_b.t()) * self.scaling


def add_lora(model: nn.Module, r: int = 16, alpha: float = 32.0, targets=("q_proj", "k_proj", "v_proj", "o_proj")):
    """Freezes every parameter and wraps the attention projections with LoRA adapters."""
    for p in model.parameters():
        p.requires_grad_(False)
    for module in list(model.modules()):
        for name in targets:
            child = getattr(module, name, None)
            if isinstance(child, nn.Linear):
                setattr(module, name, LoRALinear(child, r, alpha))
    return [p for p in model.parameters() if p.requires_grad]


def build_model(layers=4, hidden=2880, heads=64, kv_heads=8, head_dim=64, experts=32, top_k=4,
                vocab=201088, window=128, dtype=torch.bfloat16, device="cuda", seed=5):
    from transformers import GptOssConfig, GptOssForCausalLM

    cfg = GptOssConfig(
        vocab_size=vocab, hidden_size=hidden, intermediate_size=hidden, num_hidden_layers=layers,
        num_attention_heads=heads, num_key_value_heads=kv_heads, head_dim=head_dim,
        num_local_experts=experts, num_experts_per_tok=top_k, sliding_window=window,
        layer_types=["sliding_attention" if i % 2 == 0 else "full_attention" for i in range(layers)],
        attn_implementation="eager", use_cache=False)
    torch.manual_seed(seed)
    with torch.device(device):
        model = GptOssForCausalLM(cfg).to(dtype)
    with torch.no_grad():
        for name, p in model.named_parameters():
            if name.endswith("sinks"):
                p.copy_(torch.randn_like(p))
    return model


def mask_free_attention_mask(padding_mask=None):
    """`attention_mask=` value that stops `GptOssModel.forward` from materialising its two
    dense (B,1,S,S) masks (modeling_gpt_oss.py:467-477), which the flash kernels never read.
    With a 2-D right-padding mask the per-row valid lengths travel in its place; only valid
    while `patch_flash_attention()` is in effect."""
    seqlens = None
    if padding_mask is not None:
        seqlens = padding_mask.to(torch.int32).sum(dim=1).to(torch.int32)
    return {"full_attention": seqlens, "sliding_attention": seqlens}


def train_steps(model, params, ids, steps, warmup, grad_checkpointing, attention_mask=None):
    opt = torch.optim.AdamW(params, lr=2e-4)
    if grad_checkpointing:
        model.gradient_checkpointing_enable()
        model.enable_input_require_grads()
    model.train()
    losses = []

    def one():
        opt.zero_grad(set_to_none=True)
        out = model(input_ids=ids, labels=ids, attention_mask=attention_mask)
        out.loss.backward()
        opt.step()
        return out.loss.detach()

    for _ in range(warmup):
        one()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps):
        losses.append(one())
    torch.cuda.synchronize()
    dt = (time.perf_counter() - t0) / steps
    return dt, [float(x) for x in losses]


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--layers", type=int, default=4)
    ap.add_argument("--seq", type=int, default=8192)
    ap.add_argument("--batch", type=int, default=1)
    ap.add_argument("--experts", type=int, default=32)
    ap.add_argument("--vocab", type=int, default=201088)
    ap.add_argument("--lora-r", type=int, default=16)
    ap.add_argument("--steps", type=int, default=3)
    ap.add_argument("--warmup", type=int, default=1)
    ap.add_argument("--no-grad-checkpointing", action="store_true",
                    help="the reference trains with gradient_checkpointing: true (configs/sft_lora.yaml:13)")
    ap.add_argument("--skip-eager", action="store_true")
    ap.add_argument("--keep-dense-masks", action="store_true",
                    help="let the model build its dense S x S masks in the patched run too")
    args = ap.parse_args()

    from . import patching

    dev = "cuda"
    model = build_model(layers=args.layers, experts=args.experts, vocab=args.vocab, device=dev)
    params = add_lora(model, r=args.lora_r, alpha=2.0 * args.lora_r)
    gen = torch.Generator(device="cpu").manual_seed(5)
    ids = torch.randint(0, args.vocab, (args.batch, args.seq), generator=gen).to(dev)
    ckpt = not args.no_grad_checkpointing
    tokens = args.batch * args.seq
    out = {"config": {"workload": f"truncated GPT-OSS decoder + LoRA r={args.lora_r} on q/k/v/o, {args.layers} layers, "
                                  f"hidden 2880, 64q/8kv hd64, {args.experts} experts top-4, vocab {args.vocab}, "
                                  f"B={args.batch} S={args.seq}, bf16 random init, AdamW step, "
                                  f"gradient checkpointing {'on' if ckpt else 'off'}"},
           "data": "synthetic", "steps": args.steps, "warmup": args.warmup}
    state = {k: v.detach().clone() for k, v in model.state_dict().items() if "lora_" in k}
    if not args.skip_eager:
        dt, losses = train_steps(model, params, ids, args.steps, args.warmup, ckpt)
        out["eager"] = {"tokens_per_s": round(tokens / dt, 1), "ms_per_step": round(dt * 1e3, 2), "loss": losses}
        model.load_state_dict(state, strict=False)      # same starting point for the second run
    patching.patch_flash_attention()
    try:
        mask = None if args.keep_dense_masks else mask_free_attention_mask(None)
        dt, losses = train_steps(model, params, ids, args.steps, args.warmup, ckpt, attention_mask=mask)
    finally:
        patching.unpatch_flash_attention()
    out["patched"] = {"tokens_per_s": round(tokens / dt, 1), "ms_per_step": round(dt * 1e3, 2), "loss": losses,
                      "dense_masks": bool(args.keep_dense_masks)}
    if "eager" in out:
        out["speedup"] = round(out["patched"]["tokens_per_s"] / out["eager"]["tokens_per_s"], 3)
    print(json.dumps(out))


if __name__ == "__main__":
    main()
