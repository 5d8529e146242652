"""Drop-in for the reference's `patching.py` (patching.py:1-10): swaps Hugging
Face's GPT-OSS eager attention for the HIP flash attention and back.

The model must be loaded with `attn_implementation="eager"`: the attention layer
looks the eager function up as a module global at call time, which is what makes
the assignment below take effect.
"""
from transformers.models.gpt_oss import modeling_gpt_oss

from .attention_kernel import triton_flash_attention

_original_eager_attention_forward = modeling_gpt_oss.eager_attention_forward


def patch_flash_attention():
    modeling_gpt_oss.eager_attention_forward = triton_flash_attention


def unpatch_flash_attention():
    modeling_gpt_oss.eager_attention_forward = _original_eager_attention_forward
