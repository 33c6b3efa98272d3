"""Kernel-level custom ops with the reference's fused-attention call signature.

``mi355_kernels::scaled_dot_product_attention_kernel`` and
``mi355_kernels::scaled_dot_product_attention_backward_kernel`` take exactly the arguments of
``nki_kernels::scaled_dot_product_attention_kernel``
(torch_neuronx/python_ops/nki_kernels/scaled_dot_product_attention.py:9-41) and
``nki_kernels::scaled_dot_product_attention_backward_kernel``
(torch_neuronx/python_ops/nki_kernels/scaled_dot_product_attention_backward.py:9-51): inputs in
``(B, H, S, D)`` layout, K/V at ``Hkv`` heads (the GQA ratio is implied by the shapes),
``dropout_p`` / ``seed`` accepted and ignored, the log-sum-exp written into the caller's ``lse``
buffer when training.  ``mi355_kernels::sdpa_decode_fp8kv`` has no reference counterpart.
"""

from __future__ import annotations

from typing import Optional, Tuple

import torch

from . import ops


@torch.library.custom_op("mi355_kernels::scaled_dot_product_attention_kernel", mutates_args={"lse"})
def _scaled_dot_product_attention_kernel(
    q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, is_causal: bool, dropout_p: float,
    scale: Optional[float], training: bool, seed: Optional[int], lse: Optional[torch.Tensor],
) -> torch.Tensor:
    out, lse_ret = ops.sdpa_forward(q, k, v, is_causal=is_causal, scale=scale, need_lse=training)
    if training and lse is not None:
        B, H, L = lse_ret.shape
        if lse.dim() == 4:  # the tiled (B, H, 128, L // 128) form: row t * 128 + p sits at [p, t]
            if L % 128 != 0 or tuple(lse.shape) != (B, H, 128, L // 128):
                raise ValueError(f"a tiled lse buffer must have shape {(B, H, 128, L // 128)} with L divisible by 128, "
                                 f"got {tuple(lse.shape)}")
            lse.copy_(lse_ret.reshape(B, H, L // 128, 128).transpose(-1, -2))
        elif tuple(lse.shape) == (B, H, L):
            lse.copy_(lse_ret)
        else:
            raise ValueError(f"lse buffer must have shape {(B, H, L)} or the tiled {(B, H, 128, 'L // 128')}, "
                             f"got {tuple(lse.shape)}")
    return out


@_scaled_dot_product_attention_kernel.register_fake
def _(q, k, v, is_causal, dropout_p, scale, training, seed, lse):
    return q.new_empty((q.shape[0], q.shape[1], q.shape[2], v.shape[3]))


def scaled_dot_product_attention_kernel(q, k, v, is_causal=False, dropout_p=0.0, scale=None, training=False,
                                        seed=None, lse=None):
    """Fused attention forward; ``dropout_p`` and ``seed`` are accepted for compatibility and not
    consumed.  With ``training=True`` the log-sum-exp is copied into ``lse``."""
    return _scaled_dot_product_attention_kernel(q, k, v, is_causal, dropout_p, scale, training, seed, lse)


@torch.library.custom_op("mi355_kernels::scaled_dot_product_attention_backward_kernel", mutates_args=())
def scaled_dot_product_attention_backward_kernel(
    grad_out: torch.Tensor, q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, out: torch.Tensor,
    lse: torch.Tensor, is_causal: bool = False, dropout_p: float = 0.0, scale: Optional[float] = None,
    seed: Optional[int] = None,
) -> Tuple[torch.Tensor, torch.Tensor, torch.Tensor]:
    B, H, L, _ = q.shape
    if lse.dim() == 4:  # the reference's tiled (B, H, 128, L // 128) form
        if L % 128 != 0 or tuple(lse.shape) != (B, H, 128, L // 128):
            raise ValueError("a tiled lse needs a query length divisible by 128 and shape (B, H, 128, L // 128)")
        lse = lse.transpose(-1, -2).reshape(B, H, L)
    dq, dk, dv, _ = ops.sdpa_backward(grad_out, q, k, v, out, lse, is_causal=is_causal, scale=scale)
    return dq, dk, dv


@scaled_dot_product_attention_backward_kernel.register_fake
def _(grad_out, q, k, v, out, lse, is_causal=False, dropout_p=0.0, scale=None, seed=None):
    return torch.empty_like(q), torch.empty_like(k), torch.empty_like(v)


@torch.library.custom_op("mi355_kernels::sdpa_decode_fp8kv", mutates_args=())
def sdpa_decode_fp8kv(
    q: torch.Tensor, k_fp8: torch.Tensor, v_fp8: torch.Tensor, k_scale: torch.Tensor, v_scale: torch.Tensor,
    kv_lens: Optional[torch.Tensor] = None, scale: Optional[float] = None,
) -> Tuple[torch.Tensor, torch.Tensor]:
    """Decode-step attention over an fp8 e4m3 cache: ``(out, lse)``."""
    return ops.decode_fp8kv(q, k_fp8, v_fp8, k_scale, v_scale, kv_lens, scale)


@sdpa_decode_fp8kv.register_fake
def _(q, k_fp8, v_fp8, k_scale, v_scale, kv_lens=None, scale=None):
    return torch.empty_like(q), q.new_empty(q.shape[:3], dtype=torch.float32)
