"""Oracle and HIP kernels against the committed known answers (tests/golden/sdpa_small.npz).

The vectors come from torch's float64 CPU library routines (see tests/golden/make_golden.py):
numbers that neither the oracle nor the kernels produced.
"""

import os

import numpy as np
import pytest
import torch

from oracle import sdpa_math as om

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "sdpa_small.npz")
CASES = ["noncausal_mha", "causal_gqa", "causal_l_ne_s", "bool_mask_with_dead_row", "additive_bias"]


def _load(name):
    z = np.load(GOLDEN)  # plain arrays only (allow_pickle stays off)
    g = {k.split(".", 1)[1]: torch.from_numpy(z[k]) for k in z.files if k.startswith(name + ".")}
    g["causal"] = bool(g["causal"])
    return g


def _close(a, b, tol):
    a, b = a.double().cpu(), b.double()
    fin = torch.isfinite(b)
    assert torch.equal(torch.isfinite(a), fin)
    assert (a[fin] - b[fin]).abs().max().item() <= tol * max(1.0, b[fin].abs().max().item())
    assert torch.equal(a[~fin], b[~fin])  # -inf log-sum-exp of dead rows


@pytest.mark.parametrize("name", CASES)
def test_oracle_matches_golden(name):
    g = _load(name)
    q, k, v, go = (g[x].float() for x in ("q", "k", "v", "go"))
    mask = g.get("mask")
    if mask is not None and mask.dtype is not torch.bool:
        mask = mask.float()
    out, lse = om.sdpa_forward(q, k, v, attn_mask=mask, is_causal=g["causal"])
    _close(out, g["out"], 2e-6)
    _close(lse, g["lse"], 2e-6)
    dq, dk, dv = om.sdpa_backward(go, q, k, v, out, lse, attn_mask=mask, is_causal=g["causal"])[:3]
    _close(dq, g["dq"], 5e-6)
    _close(dk, g["dk"], 5e-6)
    _close(dv, g["dv"], 5e-6)


@pytest.mark.gpu
@pytest.mark.parametrize("name", CASES)
def test_kernels_match_golden(name, gpu_device):
    import torch_neuronx_amd as amd

    g = _load(name)
    dev = gpu_device
    q, k, v, go = (g[x].float().to(dev) for x in ("q", "k", "v", "go"))
    mask = g.get("mask")
    if mask is not None:
        mask = (mask if mask.dtype is torch.bool else mask.float()).to(dev)
    out, lse = amd.sdpa_forward(q, k, v, attn_bias=mask, is_causal=g["causal"])
    _close(out, g["out"], 1e-5)  # float32 tolerance of the path: 1e-5
    _close(lse, g["lse"], 1e-5)
    dq, dk, dv = amd.sdpa_backward(go, q, k, v, out, lse, attn_bias=mask, is_causal=g["causal"])[:3]
    _close(dq, g["dq"], 1e-5)
    _close(dk, g["dk"], 1e-5)
    _close(dv, g["dv"], 1e-5)
