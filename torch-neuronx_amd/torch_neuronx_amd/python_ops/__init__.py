"""Operator layer: the reference's fused-attention entry points, served by the HIP library."""

from .native_multi_head_attn_mid import native_multi_head_attn_mid  # noqa: F401
from .scaled_dot_product_fused_attention import (  # noqa: F401
    scaled_dot_product_efficient_attention,
    scaled_dot_product_efficient_attention_backward,
    scaled_dot_product_flash_attention,
    scaled_dot_product_flash_attention_backward,
    scaled_dot_product_fused_attention_overrideable,
    scaled_dot_product_fused_attention_overrideable_backward,
)
