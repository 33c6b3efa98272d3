"""MI355X-native fused scaled-dot-product attention behind the torch-neuronx operator surface."""

from . import _lib, ops  # noqa: F401
from .ops import decode_fp8kv, sdpa_backward, sdpa_forward  # noqa: F401

__all__ = ["sdpa_forward", "sdpa_backward", "decode_fp8kv", "ops"]
