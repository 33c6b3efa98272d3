"""bf16 results at large logits: where the absolute tolerances stop being the right yardstick.

At scale 0.25 or 1.0 on N(0,1) data the softmax is close to one-hot, outputs reach |O| = 4 and more
(half a bf16 ulp there is already 1.6e-2) and gradients grow with the logits.  Randomised sweeps of
this library against the float32 oracle then show outputs 2.0-2.8e-2 and gradients up to 1.6e-1 away,
with relative errors that stay below one percent.  This file pins what those numbers are: rounding,
the same rounding the reference's own bf16 arithmetic has.

The reference rounds P to the input dtype before P V and the results to the input dtype
(torch_neuronx/_sdpa_math.py:94, :171-175).  The oracle run ON bf16 TENSORS does exactly that, so the
kernels are held to three things, on the configurations the sweeps flagged:

* no further from the float32 oracle than twice the distance of the bf16 oracle from it (plus one
  bf16 ulp of the largest value: the two sum in different orders);
* within the float32-oracle bound scaled by the size of the values, max(1, |ref|max);
* small relative (Frobenius) error.

The backward is given the output it would be given in use - the kernel's own bf16 output - on both
sides: delta = rowsum(dO * O) of a rounded O differs from that of the float32 O by about
sqrt(Dv) |dO| |O| 2^-9, which for a near-one-hot row is of the size of dP - delta itself.  That, not the
kernels, was the 3-5 % relative error of dQ / dK at L = 1 in the sweeps, where the oracle had been
fed its own float32 output.
"""

import pytest
import torch

from helpers import max_abs, rel_err, seeded
from oracle import sdpa_math as om

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def amd(gpu_device):
    import torch_neuronx_amd as amd

    return amd


def _ulp_bf16(x: float) -> float:
    import math

    return 2.0 ** (math.floor(math.log2(max(abs(x), 1e-30))) - 7)


# (B, Hq, Hkv, L, S, E, Dv, causal, mask, scale): taken from the sweeps
CASES = [
    (2, 1, 1, 128, 127, 256, 256, False, "none", 0.25),
    (3, 2, 2, 1, 96, 256, 128, False, "none", 1.0),      # L = 1, wide, asymmetric
    (3, 8, 2, 300, 300, 256, 128, False, "leftpad", 1.0),
    (1, 4, 1, 1030, 160, 192, 184, False, "bool_pad", 1.0),
    (1, 8, 2, 31, 384, 192, 192, False, "none", 1.0),
    (3, 3, 3, 700, 160, 256, 128, False, "none", 0.25),
    (1, 2, 1, 1500, 1500, 128, 128, False, "leftpad", 1.0),
    (1, 7, 1, 1500, 1100, 64, 64, True, "none", 1.0),
    (2, 2, 1, 1500, 5, 72, 72, False, "kv_lens", 1.0),
    (1, 7, 1, 1100, 5, 128, 128, False, "bool_pad", 1.0),
    (1, 2, 2, 2100, 900, 128, 128, False, "none", 1.0),
    (2, 2, 1, 1, 77, 192, 128, False, "none", 1.0),       # L = 1 again, another width
]


def _mask(kind, B, L, S, g):
    if kind == "none":
        return None, None
    lens = torch.randint(max(1, S // 2), S + 1, (B,), generator=g)
    lens[0] = S
    j = torch.arange(S)[None]
    if kind == "kv_lens":
        return None, lens.to(torch.int32)
    keep = (j >= (S - lens)[:, None]) if kind == "leftpad" else (j < lens[:, None])
    return keep[:, None, None, :], None


@pytest.mark.parametrize("case", CASES, ids=lambda c: f"B{c[0]}-{c[1]}x{c[2]}-L{c[3]}-S{c[4]}-E{c[5]}-{c[6]}-{c[8]}-{c[9]}")
def test_bf16_results_are_as_close_as_the_reference_arithmetic(amd, gpu_device, case):
    B, Hq, Hkv, L, S, E, Dv, causal, kind, scale = case
    dev = gpu_device
    g = torch.Generator().manual_seed(L * 7 + S)
    q, k, v, go = seeded([(B, Hq, L, E), (B, Hkv, S, E), (B, Hkv, S, Dv), (B, Hq, L, Dv)], L + S + E, torch.bfloat16)
    keep, lens = _mask(kind, B, L, S, g)
    if lens is not None:  # the oracle takes key counts as a padding mask
        keep = (torch.arange(S)[None] < lens[:, None])[:, None, None, :]
    kw = dict(is_causal=causal, scale=scale)
    out, lse = amd.sdpa_forward(q.to(dev), k.to(dev), v.to(dev), attn_bias=None if keep is None or lens is not None else keep.to(dev),
                                kv_lens=None if lens is None else lens.to(dev), **kw)
    grads = amd.sdpa_backward(go.to(dev), q.to(dev), k.to(dev), v.to(dev), out, lse,
                              attn_bias=None if keep is None or lens is not None else keep.to(dev),
                              kv_lens=None if lens is None else lens.to(dev), **kw)[:3]
    torch.cuda.synchronize()
    out_c, lse_c = out.cpu(), lse.cpu()

    # forward: float32 oracle, and the oracle in the reference's bf16 arithmetic
    ro32, rl32 = om.sdpa_forward(q.float(), k.float(), v.float(), attn_mask=keep, **kw)
    ro16, _ = om.sdpa_forward(q, k, v, attn_mask=keep, **kw)
    top = ro32.abs().max().item()
    e_ref, e_gpu = max_abs(ro16, ro32), max_abs(out_c, ro32)
    assert e_gpu <= 2.0 * e_ref + _ulp_bf16(top), ("out", e_gpu, e_ref, top)
    assert e_gpu <= 2e-2 * max(1.0, top) and rel_err(out_c, ro32) <= 1e-2
    assert max_abs(lse_c, rl32) <= 5e-3

    # backward, both oracles fed the kernel's bf16 output and lse
    rg32 = om.sdpa_backward(go.float(), q.float(), k.float(), v.float(), out_c.float(), lse_c, attn_mask=keep,
                            reduce_in_fp32=True, **kw)
    rg16 = om.sdpa_backward(go, q, k, v, out_c, lse_c, attn_mask=keep, **kw)
    for name, a, r32, r16 in zip(("dq", "dk", "dv"), grads, rg32, rg16):
        top = r32.abs().max().item()
        e_ref, e_gpu = max_abs(r16, r32), max_abs(a, r32)
        assert e_gpu <= 2.0 * e_ref + _ulp_bf16(top), (name, e_gpu, e_ref, top)
        assert e_gpu <= 5e-2 * max(1.0, top), (name, e_gpu, top)
        if top > 1e-3:
            assert rel_err(a, r32) <= 2e-2, (name, rel_err(a, r32))
