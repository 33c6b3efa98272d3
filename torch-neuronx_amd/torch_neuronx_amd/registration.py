"""torch.library registrations: the ATen attention ops for ROCm (dispatch key CUDA) are served
by this package.

* ``aten::_scaled_dot_product_fused_attention_overrideable`` (+ ``_backward``): the pair the
  reference registers for its device (torch_neuronx/python_ops/__init__.py:89-104).  Upstream has
  no GPU kernel for it, so this registration overrides nothing.
* ``aten::_scaled_dot_product_flash_attention`` (+ ``_backward``) and
  ``aten::_scaled_dot_product_efficient_attention`` (+ ``_backward``): what
  ``F.scaled_dot_product_attention`` calls for GPU tensors (its backend choice for this device
  type is a compiled-in table, not the dispatcher), so they are what makes the plain functional
  API land in these kernels.  They replace the stock kernels; set
  ``TORCH_NEURONX_AMD_OVERRIDE_ATEN=0`` before import to leave those two pairs alone.
* ``aten::_fused_sdp_choice``: reachable through ``torch._fused_sdp_choice``; rules of
  torch_neuronx/csrc/aten/SdpBackendSelection.cpp:14-68.

Upstream's autograd formulas for these ops call the matching ``_backward`` op, so no
autograd.Function is needed.
"""

from __future__ import annotations

import os
import warnings

import torch

from . import python_ops as po
from .python_ops import scaled_dot_product_fused_attention as impl

_lib_handle = None
_registered = []


def _flag(name: str, default: str = "1") -> bool:
    return os.environ.get(name, default).lower() not in ("0", "false", "off", "no")


def register(override_aten: bool | None = None) -> list:
    """Install the kernels (idempotent).  Returns the names of the ops registered."""
    global _lib_handle
    if _lib_handle is not None:
        return list(_registered)
    if override_aten is None:
        override_aten = _flag("TORCH_NEURONX_AMD_OVERRIDE_ATEN")
    lib = torch.library.Library("aten", "IMPL")
    table = [
        ("_scaled_dot_product_fused_attention_overrideable", po.scaled_dot_product_fused_attention_overrideable),
        ("_scaled_dot_product_fused_attention_overrideable_backward",
         po.scaled_dot_product_fused_attention_overrideable_backward),
    ]
    if override_aten:
        table += [
            ("_scaled_dot_product_flash_attention", po.scaled_dot_product_flash_attention),
            ("_scaled_dot_product_flash_attention_backward", po.scaled_dot_product_flash_attention_backward),
            ("_scaled_dot_product_efficient_attention", po.scaled_dot_product_efficient_attention),
            ("_scaled_dot_product_efficient_attention_backward",
             po.scaled_dot_product_efficient_attention_backward),
            ("_fused_sdp_choice", impl.fused_sdp_choice),
        ]
    with warnings.catch_warnings():
        warnings.simplefilter("ignore")  # "overriding a previously registered kernel" is the point
        for name, fn in table:
            lib.impl(name, fn, "CUDA")
            _registered.append(name)
    _lib_handle = lib
    return list(_registered)


def unregister() -> None:
    """Remove the registrations (the stock kernels come back)."""
    global _lib_handle
    if _lib_handle is not None:
        _lib_handle._destroy()
        _lib_handle = None
        _registered.clear()


def registered_ops() -> list:
    return list(_registered)
