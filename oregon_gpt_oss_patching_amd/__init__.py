"""MI355X-native flash attention (forward + backward) for the GPT-OSS attention
variant, with the Python surface of nlp-uoregon/oregon_gpt_oss_patching.

    from oregon_gpt_oss_patching_amd import triton_flash_attention
    from oregon_gpt_oss_patching_amd.patching import patch_flash_attention
"""
from .attention_kernel import (  # noqa: F401
    attention,
    attention_backward,
    attention_forward,
    doc_start_from_position_ids,
    hip_flash_attention,
    triton_flash_attention,
)

__all__ = ["attention", "attention_forward", "attention_backward", "doc_start_from_position_ids",
           "hip_flash_attention", "triton_flash_attention"]
