"""Middle stage of native multi-head attention: attention on ``[B, H, D, S]`` operands.

Mirrors ``NativeMultiHeadAttnMidOp`` of the reference
(``torch_neuronx/python_ops/native_multi_head_attn_mid.py:112-153`` for the kernel call,
``torch_neuronx/python_ops/torch_mlir/ops/native_multi_head_attn_mid.py:58-116`` for the general
form with ``H_kv`` key/value heads and its own value width): the operands arrive with the
sequence as the LAST dimension, the result leaves as ``[B, H_q, S_q, D_v]``.  The fused kernels
read head-dim-contiguous rows, so each operand is brought into that layout by one transposing
device copy (HBM-bound); the attention runs
in the same HIP kernels as every other entry point.
"""

from __future__ import annotations

import torch

from .. import ops

_EMPTY_MSG = ("Attention operations do not support empty tensors. "
              "Please ensure all input tensors have non-zero elements.")


def native_multi_head_attn_mid(query: torch.Tensor, key: torch.Tensor, value: torch.Tensor, *,
                               use_causal_mask: bool = False, dropout_p: float = 0.0,
                               training: bool = False, out: torch.Tensor | None = None) -> torch.Tensor:
    """Attention on middle-stage operands.

    ``query`` is ``[B, H_q, D, S_q]``, ``key`` ``[B, H_kv, D, S_k]``, ``value`` ``[B, H_kv, D_v, S_k]``.
    ``dropout_p`` is accepted for compatibility and not applied (the reference's kernel wrapper
    ignores it as well, native_multi_head_attn_mid.py:84-85); ``training`` changes nothing in the
    result.  With ``out`` the result is copied into it and ``out`` is returned.

    Raises ValueError for tensors that are not on the GPU and RuntimeError for empty tensors,
    operands that are not four-dimensional, mismatched batch / head / sequence / head-dim sizes
    and an ``out`` of the wrong shape.
    """
    for t, name in ((query, "query"), (key, "key"), (value, "value")):
        if t.device.type != "cuda":
            raise ValueError(f"Expected a ROCm GPU device for {name}, got {t.device}")
    if query.numel() == 0 or key.numel() == 0 or value.numel() == 0:
        raise RuntimeError(_EMPTY_MSG)
    if query.dim() != 4 or key.dim() != 4 or value.dim() != 4:
        raise RuntimeError("native_multi_head_attn_mid: query, key and value must be 4-dimensional [B, H, D, S]")
    q, k, v = query.transpose(-2, -1), key.transpose(-2, -1), value.transpose(-2, -1)
    ops.validate(ops.make_desc(q, k, v, None, 0.0, use_causal_mask, False, None))
    result, _ = ops.sdpa_forward(q, k, v, is_causal=use_causal_mask, need_lse=False)
    if out is not None:
        if tuple(out.shape) != tuple(result.shape):
            raise RuntimeError(f"Output tensor shape {tuple(out.shape)} doesn't match expected shape {tuple(result.shape)}")
        out.copy_(result)
        return out
    return result
