"""MI355X-native fused scaled-dot-product attention behind the torch-neuronx operator surface.

Importing the package loads ``libmi355_sdpa.so`` lazily (first op call) and registers the ATen
attention ops for ROCm GPU tensors unless ``TORCH_NEURONX_AMD_REGISTER=0``.
"""

import os as _os

from . import _lib, kernels, mask_patterns, ops, python_ops, registration  # noqa: F401
from .kernels import (  # noqa: F401
    scaled_dot_product_attention_backward_kernel,
    scaled_dot_product_attention_kernel,
    sdpa_decode_fp8kv,
)
from .ops import decode_fp8kv, sdpa_backward, sdpa_forward  # noqa: F401
from .python_ops import native_multi_head_attn_mid  # noqa: F401
from .registration import register, registered_ops, route_functional, unregister  # noqa: F401

if _os.environ.get("TORCH_NEURONX_AMD_REGISTER", "1").lower() not in ("0", "false", "off", "no"):
    register()
    if _os.environ.get("TORCH_NEURONX_AMD_ROUTE_FUNCTIONAL", "0").lower() in ("1", "true", "on", "yes"):
        route_functional(True)

__all__ = [
    "sdpa_forward", "sdpa_backward", "decode_fp8kv", "ops", "kernels", "python_ops", "registration",
    "register", "unregister", "registered_ops", "route_functional", "scaled_dot_product_attention_kernel",
    "scaled_dot_product_attention_backward_kernel", "sdpa_decode_fp8kv", "native_multi_head_attn_mid",
]
