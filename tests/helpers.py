"""Shared helpers for the parity tests: seeded inputs and oracle wrappers."""

import math

import torch

from oracle import sdpa_math as om


def seeded(shape_list, seed, dtype):
    """Draw the tensors in order from one CPU generator (fp32), then cast to ``dtype``."""
    g = torch.Generator(device="cpu").manual_seed(seed)
    return [torch.randn(s, generator=g).to(dtype) for s in shape_list]


def qkv(B, Hq, Hkv, L, S, E, Dv=None, dtype=torch.float32, seed=0, with_do=False):
    Dv = Dv or E
    shapes = [(B, Hq, L, E), (B, Hkv, S, E), (B, Hkv, S, Dv)]
    if with_do:
        shapes.append((B, Hq, L, Dv))
    return seeded(shapes, seed, dtype)


def oracle_fwd(q, k, v, attn_mask=None, is_causal=False, scale=None):
    """fp32 oracle on the (already cast) inputs: returns fp32 out and lse."""
    return om.sdpa_forward(q.float().cpu(), k.float().cpu(), v.float().cpu(),
                           attn_mask=None if attn_mask is None else attn_mask.cpu(),
                           is_causal=is_causal, scale=scale)


def oracle_bwd(go, q, k, v, out, lse, attn_mask=None, is_causal=False, scale=None):
    return om.sdpa_backward(go.float().cpu(), q.float().cpu(), k.float().cpu(), v.float().cpu(),
                            out.float().cpu(), lse.float().cpu(),
                            attn_mask=None if attn_mask is None else attn_mask.cpu(),
                            is_causal=is_causal, scale=scale, reduce_in_fp32=True)


def max_abs(a, b):
    a, b = a.float().cpu(), b.float().cpu()
    both_inf = torch.isinf(a) & torch.isinf(b) & (a.sign() == b.sign())
    d = (a - b).abs()
    d[both_inf] = 0.0
    return d.max().item() if d.numel() else 0.0


def tol_for(dtype, grads=False):
    if dtype is torch.float32:
        return 1e-5 if not grads else 5e-5
    return 5e-2 if grads else 2e-2


def rel_err(a, b):
    """Relative Frobenius error; guards against mistakes that hide under an absolute bound."""
    a, b = a.double().cpu(), b.double().cpu()
    finite = torch.isfinite(b)
    den = b[finite].norm().item()
    return (a[finite] - b[finite]).norm().item() / max(den, 1e-30)
