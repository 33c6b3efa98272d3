"""Writes tests/golden/sdpa_small.npz: known answers for small attention problems.

The reference's own tests hold no stored vectors for this path; what they pin results to is
torch's CPU ``F.scaled_dot_product_attention`` (tests/python_ops/test_scaled_dot_product_attention.py:263,434
in the reference tree) and ``torch.logsumexp`` in float64 (tests/neuron_dynamo_backend/unit/test_decompositions.py:8667-8672).
This script evaluates exactly those library routines in float64 on seeded inputs and stores
inputs and outputs, so that the oracle and the GPU kernels can be checked against numbers that
neither of them produced.  Gradients come from autograd through the same float64 library call.

    python tests/golden/make_golden.py
"""

import math
import os

import numpy as np
import torch
import torch.nn.functional as F

CASES = [
    # name, B, Hq, Hkv, L, S, E, causal, mask
    ("noncausal_mha", 1, 2, 2, 16, 16, 8, False, None),
    ("causal_gqa", 1, 4, 2, 12, 12, 8, True, None),
    ("causal_l_ne_s", 1, 2, 1, 7, 12, 8, True, None),
    ("bool_mask_with_dead_row", 1, 2, 2, 6, 9, 8, False, "bool"),
    ("additive_bias", 2, 2, 1, 5, 11, 8, False, "float"),
]


def main():
    out = {}
    for seed, (name, B, Hq, Hkv, L, S, E, causal, mask) in enumerate(CASES):
        g = torch.Generator().manual_seed(4000 + seed)
        q = torch.randn(B, Hq, L, E, generator=g, dtype=torch.float64, requires_grad=True)
        k = torch.randn(B, Hkv, S, E, generator=g, dtype=torch.float64, requires_grad=True)
        v = torch.randn(B, Hkv, S, E, generator=g, dtype=torch.float64, requires_grad=True)
        go = torch.randn(B, Hq, L, E, generator=g, dtype=torch.float64)
        m = None
        if mask == "bool":
            m = torch.rand(B, 1, L, S, generator=g) > 0.3
            m[:, :, 2, :] = False  # a row without a live key (same row in every head)
        elif mask == "float":
            m = torch.randn(B, Hq, L, S, generator=g, dtype=torch.float64)
        rep = Hq // Hkv
        ke, ve = k.repeat_interleave(rep, 1), v.repeat_interleave(rep, 1)
        scale = 1.0 / math.sqrt(E)
        logits = q @ ke.transpose(-1, -2) * scale
        if causal:
            keep = torch.ones(L, S, dtype=torch.bool).tril()
            logits = logits.masked_fill(~keep, float("-inf"))
        if m is not None:
            logits = logits.masked_fill(~m, float("-inf")) if m.dtype is torch.bool else logits + m
        lse = torch.logsumexp(logits.detach(), -1)
        dead = torch.isinf(lse) & (lse < 0)  # rows without a live key: output 0, lse -inf, no gradient
        # the library returns NaN for such rows; evaluate it with those rows attending everything and
        # with their upstream gradient zeroed, which is what "zero probabilities" means for the rest
        m_lib = m
        if m is not None and m.dtype is torch.bool:
            m_lib = m | dead.any(1, keepdim=True)[..., None].expand_as(m) if m.shape[1] == 1 else m | dead[..., None]
        o = F.scaled_dot_product_attention(q, ke, ve, attn_mask=m_lib, is_causal=causal)
        o_clean = torch.where(dead[..., None], torch.zeros_like(o), o)
        (o * torch.where(dead[..., None], torch.zeros_like(go), go)).sum().backward()
        for t_ in (q.grad, k.grad, v.grad, o_clean):
            assert torch.isfinite(t_).all()
        out[f"{name}.q"], out[f"{name}.k"], out[f"{name}.v"], out[f"{name}.go"] = (
            q.detach().numpy(), k.detach().numpy(), v.detach().numpy(), go.numpy())
        if m is not None:
            out[f"{name}.mask"] = m.numpy()
        out[f"{name}.causal"] = np.array(causal)
        out[f"{name}.out"], out[f"{name}.lse"] = o_clean.detach().numpy(), lse.numpy()
        out[f"{name}.dq"], out[f"{name}.dk"], out[f"{name}.dv"] = (
            q.grad.numpy(), k.grad.numpy(), v.grad.numpy())
    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "sdpa_small.npz")
    np.savez_compressed(path, **out)
    print("wrote", path, os.path.getsize(path), "bytes")


if __name__ == "__main__":
    main()
