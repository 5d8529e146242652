"""Drop-in for the reference's `patching.py` (patching.py:1-10): swaps Hugging
Face's GPT-OSS eager attention for the HIP flash attention and back.

The model must be loaded with `attn_implementation="eager"`: the attention layer
looks the eager function up as a module global at call time, which is what makes
the assignment below take effect.
"""
from transformers.models.gpt_oss import modeling_gpt_oss

from . import attention_kernel
from .attention_kernel import triton_flash_attention

_original_eager_attention_forward = modeling_gpt_oss.eager_attention_forward


def patch_flash_attention(respect_packing: bool = False):
    """`respect_packing=True` additionally keeps the documents of a packed row (position ids
    restarting inside the row) from attending to each other (transformers' same-document mask,
    masking_utils.py:182-190,728-757); the default reproduces the reference, which treats the
    row as one causal sequence."""
    attention_kernel.RESPECT_PACKING = bool(respect_packing)
    modeling_gpt_oss.eager_attention_forward = triton_flash_attention


def unpatch_flash_attention():
    attention_kernel.RESPECT_PACKING = False
    modeling_gpt_oss.eager_attention_forward = _original_eager_attention_forward
