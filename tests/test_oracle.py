"""Pins the CPU oracle (oracle/sdpa_math.py) without importing the reference.

Each test is one of the checks the reference's own CPU tests make, or a closed
form / library routine / brute force that a plausible mistake in the oracle
(dropped term, wrong sign, transposed operand, wrong causal anchor, wrong GQA
head map) would fail.
"""

import math

import pytest
import torch
import torch.nn.functional as F

from oracle import sdpa_math as om


def _qkv(B, Hq, Hkv, L, S, E, Dv=None, dtype=torch.float32, seed=0):
    g = torch.Generator().manual_seed(seed)
    Dv = Dv or E
    q = torch.randn(B, Hq, L, E, generator=g).to(dtype)
    k = torch.randn(B, Hkv, S, E, generator=g).to(dtype)
    v = torch.randn(B, Hkv, S, Dv, generator=g).to(dtype)
    return q, k, v


def _f64_reference(q, k, v, bias, is_causal, scale):
    """float64 library SDPA; causal merged into the bias by hand (top-left anchored)."""
    L, S = q.shape[-2], k.shape[-2]
    m = torch.zeros(L, S, dtype=torch.float64)
    if is_causal:
        m = m.masked_fill(~torch.ones(L, S, dtype=torch.bool).tril(), float("-inf"))
    if bias is not None:
        m = m + bias.double()
    return F.scaled_dot_product_attention(q.double(), k.double(), v.double(), attn_mask=m, scale=scale)


@pytest.mark.parametrize("L,S", [(51, 51), (13, 51), (51, 13), (1, 7)])
@pytest.mark.parametrize("is_causal", [False, True])
@pytest.mark.parametrize("mask_kind", ["none", "float", "bool"])
def test_forward_matches_float64_library(L, S, is_causal, mask_kind):
    q, k, v = _qkv(2, 4, 4, L, S, 48)
    scale = 1.0 / math.sqrt(48)
    g = torch.Generator().manual_seed(1)
    if mask_kind == "none":
        mask = None
    elif mask_kind == "float":
        mask = torch.randn(2, 4, L, S, generator=g)
    else:
        mask = torch.rand(2, 4, L, S, generator=g) > 0.3
        mask[..., 0] = True  # keep every row alive for the library comparison
    kk, vv, bias, sc = om.normalize_sdpa_args(q, k, v, mask, scale)
    out, lse = om.compute_attention(q, kk, vv, bias, None, sc, is_causal, 0.0)
    ref = _f64_reference(q, k, v, bias, is_causal, scale)
    torch.testing.assert_close(out.double(), ref, rtol=1e-5, atol=1e-5)
    # closed form for the log-sum-exp
    logits = q.double() @ k.double().transpose(-2, -1) * scale
    if is_causal:
        logits = logits.masked_fill(~torch.ones(L, S, dtype=torch.bool).tril(), float("-inf"))
    if bias is not None:
        logits = logits + bias.double()
    torch.testing.assert_close(lse.double(), torch.logsumexp(logits, -1), rtol=1e-5, atol=1e-5)
    assert lse.dtype == torch.float32 and lse.shape == (2, 4, L)


def test_lse_of_bf16_inputs_uses_fp32_chain():
    # reference: test_decompositions.py:8659-8672 (relative error < 5e-4)
    q, k, v = _qkv(2, 4, 4, 51, 51, 48, dtype=torch.bfloat16)
    scale = 1.0 / math.sqrt(48)
    _, lse = om.compute_attention(q, k, v, None, None, scale, False, 0.0)
    golden = torch.logsumexp(q.double() @ k.double().transpose(-2, -1) * scale, -1)
    rel = (lse.double() - golden).norm() / golden.norm()
    assert rel < 5e-4


@pytest.mark.parametrize("is_causal", [False, True])
@pytest.mark.parametrize("with_bias", [False, True])
def test_forward_matches_brute_force(is_causal, with_bias):
    q, k, v = _qkv(1, 2, 2, 5, 7, 6, Dv=3, seed=3)
    bias = torch.randn(1, 2, 5, 7, generator=torch.Generator().manual_seed(9)) if with_bias else None
    if with_bias:
        bias[0, 1, 2, :] = float("-inf")  # one dead row
    out, lse = om.compute_attention(q, k, v, bias, None, 0.37, is_causal, 0.0)
    for h in range(2):
        bo, bl = om.brute_force_attention(q[0, h], k[0, h], v[0, h], None if bias is None else bias[0, h], 0.37, is_causal)
        torch.testing.assert_close(out[0, h].double(), torch.tensor(bo, dtype=torch.float64), rtol=1e-5, atol=1e-6)
        torch.testing.assert_close(lse[0, h].double(), torch.tensor(bl, dtype=torch.float64), rtol=1e-5, atol=1e-6)


@pytest.mark.parametrize("is_causal,dropout_p", [(False, 0.0), (True, 0.0), (False, 0.25)])
def test_backward_matches_autograd_of_forward(is_causal, dropout_p):
    # reference: test_decompositions.py:8699-8740
    q, k, v = [t.requires_grad_(True) for t in _qkv(2, 4, 4, 7, 7, 48)]
    g = torch.Generator().manual_seed(5)
    bias = torch.randn(2, 4, 7, 7, generator=g).requires_grad_(True)
    keep = torch.rand(2, 4, 7, 7, generator=g) >= dropout_p
    go = torch.randn(2, 4, 7, 48, generator=g)
    scale = 1.0 / math.sqrt(48)
    out, lse = om.compute_attention(q, k, v, bias, keep, scale, is_causal, dropout_p)
    out.backward(go)
    got = om.compute_attention_backward(
        go, q.detach(), k.detach(), v.detach(), bias.detach(), keep, out.detach(), lse.detach(), scale, is_causal, dropout_p
    )
    for a, e in zip(got, (q.grad, k.grad, v.grad, bias.grad)):
        torch.testing.assert_close(a, e, rtol=1e-4, atol=1e-5)


def test_backward_matches_float64_library_autograd():
    q, k, v = [t.double().requires_grad_(True) for t in _qkv(1, 3, 3, 9, 11, 8, Dv=5, seed=11)]
    go = torch.randn(1, 3, 9, 5, dtype=torch.float64, generator=torch.Generator().manual_seed(2))
    ref = F.scaled_dot_product_attention(q, k, v, is_causal=True, scale=0.3)
    ref.backward(go)
    out, lse = om.compute_attention(q.detach(), k.detach(), v.detach(), None, None, 0.3, True, 0.0)
    dq, dk, dv, db = om.compute_attention_backward(go, q.detach(), k.detach(), v.detach(), None, None, out, lse, 0.3, True, 0.0)
    assert db is None
    torch.testing.assert_close(dq, q.grad, rtol=1e-6, atol=1e-6)  # lse is stored in float32
    torch.testing.assert_close(dk, k.grad, rtol=1e-6, atol=1e-6)
    torch.testing.assert_close(dv, v.grad, rtol=1e-6, atol=1e-6)


def test_backward_row_identities():
    """sum_j dS_ij == 0 for live rows, and the row term equals rowsum(dO*O)."""
    q, k, v = _qkv(1, 2, 2, 6, 6, 8, seed=4)
    go = torch.randn(1, 2, 6, 8, generator=torch.Generator().manual_seed(6))
    bias = torch.zeros(1, 2, 6, 6)
    out, lse = om.compute_attention(q, k, v, bias, None, 0.5, True, 0.0)
    _, _, _, dlogits = om.compute_attention_backward(go, q, k, v, bias, None, out, lse, 0.5, True, 0.0)
    assert dlogits is not None
    torch.testing.assert_close(dlogits.sum(-1), torch.zeros(1, 2, 6), atol=1e-5, rtol=0)
    # strictly-upper entries are exactly zero under the causal mask
    assert torch.equal(dlogits.triu(1), torch.zeros_like(dlogits))


def test_backward_ring_correction_term():
    """With a foreign ``out`` the row term shifts by sum_d dO*(out - true_out)."""
    q, k, v = _qkv(1, 1, 1, 4, 4, 8, seed=8)
    go = torch.randn(1, 1, 4, 8, generator=torch.Generator().manual_seed(7))
    bias = torch.zeros(1, 1, 4, 4)
    out, lse = om.compute_attention(q, k, v, bias, None, 0.5, False, 0.0)
    shifted = out + 0.25
    _, _, dv0, dl0 = om.compute_attention_backward(go, q, k, v, bias, None, out, lse, 0.5, False, 0.0)
    _, _, dv1, dl1 = om.compute_attention_backward(go, q, k, v, bias, None, shifted, lse, 0.5, False, 0.0)
    p = torch.softmax(q @ k.transpose(-2, -1) * 0.5, -1)
    expect = dl0 - p * (go * 0.25).sum(-1, keepdim=True)
    torch.testing.assert_close(dl1, expect, rtol=1e-5, atol=1e-6)
    torch.testing.assert_close(dv0, dv1)


@pytest.mark.parametrize("Hq,Hkv", [(8, 2), (8, 1), (6, 6), (24, 6)])
def test_gqa_equals_upstream_enable_gqa(Hq, Hkv):
    q, k, v = [t.double().requires_grad_(True) for t in _qkv(2, Hq, Hkv, 10, 12, 16, seed=Hq)]
    go = torch.randn(2, Hq, 10, 16, dtype=torch.float64, generator=torch.Generator().manual_seed(1))
    ref = F.scaled_dot_product_attention(q, k, v, enable_gqa=True)
    ref.backward(go)
    out, lse = om.sdpa_forward(q.detach(), k.detach(), v.detach())
    torch.testing.assert_close(out, ref.detach(), rtol=1e-9, atol=1e-9)
    dq, dk, dv = om.sdpa_backward(go, q.detach(), k.detach(), v.detach(), out, lse)
    torch.testing.assert_close(dq, q.grad, rtol=1e-5, atol=1e-6)
    torch.testing.assert_close(dk, k.grad, rtol=1e-5, atol=1e-6)
    torch.testing.assert_close(dv, v.grad, rtol=1e-5, atol=1e-6)
    # head map: query head h reads kv head h // rep
    rep = Hq // Hkv
    h = Hq - 1
    one, _ = om.compute_attention(q.detach()[:, h : h + 1], k.detach()[:, h // rep : h // rep + 1],
                                  v.detach()[:, h // rep : h // rep + 1], None, None, 0.25, False, 0.0)
    torch.testing.assert_close(out[:, h : h + 1], one, rtol=1e-9, atol=1e-9)


def test_head_chunking_does_not_change_results():
    q, k, v = _qkv(2, 8, 2, 17, 19, 16, seed=2)
    mask = torch.rand(2, 1, 17, 19, generator=torch.Generator().manual_seed(3)) > 0.2
    a = om.sdpa_forward(q, k, v, attn_mask=mask, head_chunk=8)
    b = om.sdpa_forward(q, k, v, attn_mask=mask, head_chunk=3)
    assert torch.equal(a[0], b[0]) and torch.equal(a[1], b[1])


@pytest.mark.parametrize("S", [1, 3])
def test_chunking_keeps_a_per_batch_bias_in_the_backward(S):
    # A (B,1,1,1) bias has more than one element, so the backward applies it; the wrapper hands the
    # math one batch at a time, where each slice has a single element and would pass for the
    # placeholder that the backward ignores.  Checked against autograd of the library routine.
    B, H, L, E = 2, 2, 4, 8
    g = torch.Generator().manual_seed(9)
    q, k, v = [torch.randn(shape, generator=g, dtype=torch.float64).requires_grad_(True)
               for shape in ((B, H, L, E), (B, H, S, E), (B, H, S, E))]
    bias = 2 * torch.randn(B, 1, 1, 1, generator=g, dtype=torch.float64)
    go = torch.randn(B, H, L, E, generator=g, dtype=torch.float64)
    F.scaled_dot_product_attention(q, k, v, attn_mask=bias).backward(go)
    out, lse = om.sdpa_forward(q.detach(), k.detach(), v.detach(), attn_mask=bias)
    dq, dk, dv = om.sdpa_backward(go, q.detach(), k.detach(), v.detach(), out, lse, attn_mask=bias)
    for a, e in ((dq, q.grad), (dk, k.grad), (dv, v.grad)):
        torch.testing.assert_close(a, e, rtol=1e-5, atol=1e-6)  # lse is stored in float32


def test_reduce_gqa_gradients_with_different_head_dims():
    # reference: test_sdpa_nki_gates.py:142-168
    gk = torch.randn(2, 8, 5, 6)
    gv = torch.randn(2, 8, 5, 3)
    rk, rv = om.reduce_gqa_gradients(gk, gv, 2)
    assert rk.shape == (2, 2, 5, 6) and rv.shape == (2, 2, 5, 3)
    torch.testing.assert_close(rk[:, 1], gk[:, 4:8].sum(1))
    torch.testing.assert_close(rv[:, 0], gv[:, 0:4].sum(1))


def test_fully_masked_rows_forward_and_backward():
    # reference: test_decompositions.py:8742-8778, test_scaled_dot_product_attention.py:1003-1120
    q, k, v = _qkv(2, 4, 4, 7, 7, 48)
    bias = torch.zeros(2, 4, 7, 7)
    bias[:, :, :2, :] = float("-inf")
    go = torch.randn(2, 4, 7, 48, generator=torch.Generator().manual_seed(3))
    out, lse = om.compute_attention(q, k, v, bias, torch.empty(0), 0.1, False, 0.0)
    assert torch.equal(out[:, :, :2], torch.zeros(2, 4, 2, 48))
    assert torch.isinf(lse[:, :, :2]).all() and (lse[:, :, :2] < 0).all()
    grads = om.compute_attention_backward(go, q, k, v, bias, torch.empty(0), out, lse, 0.1, False, 0.0)
    for g in grads:
        assert g is not None and torch.isfinite(g).all()
    assert torch.equal(grads[0][:, :, :2], torch.zeros(2, 4, 2, 48))


def test_mask_and_causal_both_apply():
    # reference: test_decompositions.py:8674-8697
    q, k, v = _qkv(2, 4, 4, 51, 51, 48)
    mask = torch.randn(2, 4, 51, 51, generator=torch.Generator().manual_seed(4))
    kk, vv, bias, sc = om.normalize_sdpa_args(q, k, v, mask, None)
    out, _ = om.compute_attention(q, kk, vv, bias, None, sc, True, 0.0)
    torch.testing.assert_close(out.double(), _f64_reference(q, k, v, mask, True, sc), rtol=1e-5, atol=1e-5)


@pytest.mark.parametrize("saturation", [8, 32, 64])
def test_saturated_softmax_invariants(saturation):
    # reference: tests/python_ops/test_sdpa_math.py:30-63
    S, H, D = 512, 4, 128
    amp = {}
    for dtype in (torch.bfloat16, torch.float32):
        torch.manual_seed(0)
        q = (torch.randn(1, H, S, D) * saturation).to(dtype)
        k = (torch.randn(1, H, S, D) * saturation).to(dtype)
        v = torch.randn(1, H, S, D).to(dtype)
        scale = D**-0.5
        out, lse = om.compute_attention(q, k, v, None, None, scale, True, 0.0)
        if dtype is torch.bfloat16:
            logits = (q.float() @ k.float().transpose(-2, -1)) * scale
            idx = torch.arange(S)
            logits = logits.masked_fill(idx[:, None] < idx[None, :], float("-inf"))
            assert torch.exp(logits - lse.unsqueeze(-1)).max().item() <= 1.0 + 1e-3
        go = torch.full_like(out, 1e-7)
        dq, dk, _, _ = om.compute_attention_backward(go, q, k, v, None, None, out, lse, scale, True, 0.0)
        assert torch.isfinite(dq.float()).all() and torch.isfinite(dk.float()).all()
        amp[dtype] = (dq.float().abs().max().item(), dk.float().abs().max().item())
    for a, b in zip(amp[torch.bfloat16], amp[torch.float32]):
        assert a == pytest.approx(b, rel=0.25)


def test_placeholder_semantics():
    # reference: test_decompositions.py:8780-8880
    q, k, v = _qkv(2, 4, 4, 7, 7, 48)
    go = torch.randn(2, 4, 7, 48, generator=torch.Generator().manual_seed(3))
    out, lse = om.compute_attention(q, k, v, torch.zeros(1), torch.empty(0), 0.2, False, 0.0)
    a = om.compute_attention_backward(go, q, k, v, torch.zeros(1), torch.zeros(1), out, lse, 0.2, False, 0.5)
    b = om.compute_attention_backward(go, q, k, v, torch.zeros(1), torch.empty(0), out, lse, 0.2, False, 0.0)
    assert a[3] is None and b[3] is None
    for x, y in zip(a[:3], b[:3]):
        assert x.abs().sum() > 0 and torch.equal(x, y)
    with pytest.raises(ValueError):
        om.compute_attention(q, k, v, None, torch.ones(2, 4, 7, 7), 0.2, False, 1.5)


def test_dropout_one_zeroes_the_output():
    q, k, v = _qkv(1, 2, 2, 5, 5, 8)
    out, _ = om.compute_attention(q, k, v, None, torch.zeros(1, 2, 5, 5, dtype=torch.bool), 0.2, False, 1.0)
    assert torch.equal(out, torch.zeros_like(out))


def test_bf16_probabilities_are_rounded_before_pv():
    q, k, v = _qkv(1, 2, 2, 33, 33, 16, dtype=torch.bfloat16)
    out, _ = om.compute_attention(q, k, v, None, None, 0.25, False, 0.0)
    p = torch.softmax(q.float() @ k.float().transpose(-2, -1) * 0.25, -1)
    assert out.dtype == torch.bfloat16
    torch.testing.assert_close(out, p.to(torch.bfloat16) @ v, rtol=0, atol=1e-2)


def test_scale_zero_is_honoured():
    q, k, v = _qkv(1, 2, 2, 4, 6, 8)
    out, lse = om.sdpa_forward(q, k, v, scale=0.0)
    torch.testing.assert_close(out, v.mean(dim=2, keepdim=True).expand(1, 2, 4, 8))
    torch.testing.assert_close(lse, torch.full((1, 2, 4), math.log(6.0)))


def test_fp8_quantisation_definition_and_decode():
    g = torch.Generator().manual_seed(1005)
    B, Hq, Hkv, S, D = 3, 8, 2, 40, 16
    q = torch.randn(B, Hq, 1, D, generator=g).to(torch.bfloat16)
    k = torch.randn(B, Hkv, S, D, generator=g)
    v = torch.randn(B, Hkv, S, D, generator=g)
    kq, ks = om.quantize_kv_fp8(k)
    vq, vs = om.quantize_kv_fp8(v)
    assert kq.dtype == torch.float8_e4m3fn and ks.shape == (B, Hkv)
    torch.testing.assert_close(ks, k.abs().amax((-2, -1)) / 448.0)
    # e4m3 has 3 mantissa bits: relative error of a normal value is at most 2^-4
    kd = om.dequantize_kv_fp8(kq, ks)
    big = k.abs() > ks[:, :, None, None] * 2.0**-6 * 1.01
    assert ((kd - k).abs()[big] <= k.abs()[big] * 2.0**-4 + 1e-7).all()
    assert kd.abs().max() <= k.abs().max() * (1 + 1e-6)
    lens = torch.tensor([40, 1, 17])
    out, lse = om.decode_fp8kv(q, kq, vq, ks, vs, lens)
    vd = om.dequantize_kv_fp8(vq, vs)
    for b in range(B):
        n = int(lens[b])
        ref = F.scaled_dot_product_attention(
            q[b : b + 1].double(), kd[b : b + 1, :, :n].double(), vd[b : b + 1, :, :n].double(), enable_gqa=True
        )
        torch.testing.assert_close(out[b : b + 1].double(), ref, rtol=1e-5, atol=1e-5)
    # key-padding bias formulation gives the same answer as truncation
    pad = (torch.arange(S)[None, :] < lens[:, None])[:, None, None, :]
    o2, l2 = om.sdpa_forward(q.float(), kd, vd, attn_mask=pad)
    torch.testing.assert_close(o2, out, rtol=1e-5, atol=1e-6)
    torch.testing.assert_close(l2, lse, rtol=1e-5, atol=1e-6)


def test_decode_empty_sequence_matches_fully_masked_rows():
    g = torch.Generator().manual_seed(3)
    B, Hq, Hkv, S, D = 2, 4, 2, 8, 16
    q = torch.randn(B, Hq, 1, D, generator=g)
    kq, ks = om.quantize_kv_fp8(torch.randn(B, Hkv, S, D, generator=g))
    vq, vs = om.quantize_kv_fp8(torch.randn(B, Hkv, S, D, generator=g))
    lens = torch.tensor([0, 5])
    out, lse = om.decode_fp8kv(q, kq, vq, ks, vs, lens)
    pad = (torch.arange(S)[None, :] < lens[:, None])[:, None, None, :]
    o2, l2 = om.sdpa_forward(q, om.dequantize_kv_fp8(kq, ks), om.dequantize_kv_fp8(vq, vs), attn_mask=pad)
    assert torch.equal(out[0], torch.zeros_like(out[0])) and torch.isinf(lse[0]).all() and (lse[0] < 0).all()
    torch.testing.assert_close(o2, out, rtol=1e-5, atol=1e-6)
    torch.testing.assert_close(l2, lse, rtol=1e-5, atol=1e-6)


# ---- mask functors (sliding window, sink keys, sink logit) ------------------------------------------


def _functor_reference(q, k, v, window, sink_keys, sink_logit, scale):
    """float64 library routine on the explicit mask; the sink is one more key with a zero value
    whose logit arrives through the bias."""
    B, Hq, L, E = q.shape
    S = k.shape[2]
    rep = Hq // k.shape[1]
    q64 = q.double().requires_grad_(True)
    k64 = k.double().requires_grad_(True)
    v64 = v.double().requires_grad_(True)
    ke, ve = k64.repeat_interleave(rep, 1), v64.repeat_interleave(rep, 1)
    row, col = torch.arange(L)[:, None], torch.arange(S)[None]
    keep = col <= row
    if window:
        keep = keep & ((row - col < window) | (col < sink_keys))
    bias = torch.zeros(B, Hq, L, S, dtype=torch.float64).masked_fill(~keep, float("-inf"))
    z = None
    if sink_logit is not None:
        z = sink_logit.double().reshape(-1, Hq).expand(B, Hq).clone().requires_grad_(True)
        ke = torch.cat([ke, torch.zeros(B, Hq, 1, E, dtype=torch.float64)], 2)
        ve = torch.cat([ve, torch.zeros(B, Hq, 1, v.shape[3], dtype=torch.float64)], 2)
        bias = torch.cat([bias, z[:, :, None, None].expand(B, Hq, L, 1)], 3)
    out = F.scaled_dot_product_attention(q64, ke, ve, attn_mask=bias, scale=scale)
    logits = torch.matmul(q64, ke.transpose(-1, -2)) * scale + bias
    return out, torch.logsumexp(logits, -1), (q64, k64, v64, z)


@pytest.mark.parametrize("window,sink_keys,with_sink", [(5, 0, False), (7, 3, False), (0, 0, True), (4, 2, True), (64, 0, True)])
def test_functor_oracle_matches_float64_library(window, sink_keys, with_sink):
    g = torch.Generator().manual_seed(window * 7 + sink_keys)
    B, Hq, Hkv, L, S, E = 2, 4, 2, 19, 19, 16
    q, k, v, go = (torch.randn(s_, generator=g) for s_ in ((B, Hq, L, E), (B, Hkv, S, E), (B, Hkv, S, E), (B, Hq, L, E)))
    z = torch.randn(B, Hq, generator=g) * 2 if with_sink else None
    scale = 0.3
    out, lse = om.sdpa_forward_functor(q, k, v, is_causal=True, scale=scale, window=window, sink_keys=sink_keys, sink_logit=z)
    ro, rl, (q64, k64, v64, z64) = _functor_reference(q, k, v, window, sink_keys, z, scale)
    assert (out.double() - ro).abs().max() < 1e-5 and (lse.double() - rl).abs().max() < 1e-5
    dq, dk, dv, dz = om.sdpa_backward_functor(go, q, k, v, out, lse, is_causal=True, scale=scale, window=window,
                                              sink_keys=sink_keys, sink_logit=z)
    leaves = [q64, k64, v64] + ([z64] if with_sink else [])
    grads = torch.autograd.grad(ro, leaves, go.double())
    for a, r in zip((dq, dk, dv), grads[:3]):
        assert a.shape == r.shape and (a.double() - r).abs().max() < 1e-4
    if with_sink:
        assert (dz.double() - grads[3]).abs().max() < 1e-4
    else:
        assert dz is None


def test_window_mask_closed_forms():
    # a window at least as long as the sequence is the causal mask; window 1 keeps the diagonal;
    # row i keeps min(i + 1, window) keys plus the sink keys that the window does not already hold
    L = S = 11
    causal = torch.tril(torch.ones(L, S, dtype=torch.bool))
    assert torch.equal(om.window_keep_mask(L, S, 11), causal) and torch.equal(om.window_keep_mask(L, S, 0), causal)
    assert torch.equal(om.window_keep_mask(L, S, 1), torch.eye(L, dtype=torch.bool))
    m = om.window_keep_mask(L, S, 3, 2)
    for i in range(L):
        want = {j for j in range(S) if j <= i and (i - j < 3 or j < 2)}
        assert {j for j in range(S) if m[i, j]} == want
    assert om.window_keep_mask(5, 9, 2).sum() == 1 + 2 * 4  # L != S: anchored top-left


# ---- score functors, document ids, several sink logits ---------------------------------------------
# Pinned by the functor written out element by element on a float64 score matrix (a Python loop over
# heads, rows and keys), float64 softmax with the sink logits as extra columns, and autograd through
# all of it: a dropped term, a wrong sign of (j - i), a transposed (h, j) index or a missing
# derivative fails one of the cases below.


def _score_mod_reference(q, k, v, scale, causal, window, z, slopes, cap, kb, kw, doc):
    B, Hq, L, _ = q.shape
    S, rep = k.shape[2], q.shape[1] // k.shape[1]
    q64, k64, v64 = (t.double().requires_grad_(True) for t in (q, k, v))
    z64 = None if z is None else z.double().requires_grad_(True)
    kk, vv = k64.repeat_interleave(rep, 1), v64.repeat_interleave(rep, 1)
    heads = []
    for b in range(B):
        for h in range(Hq):
            rows = []
            for i in range(L):
                r = []
                for j in range(S):
                    s = (q64[b, h, i] * kk[b, h, j]).sum() * scale
                    if kw is not None:
                        s = s * kw[h, j].double()
                    if kb is not None:
                        s = s + kb[h, j].double()
                    if slopes is not None:
                        s = s + slopes[h].double() * (j - i)
                    if cap:
                        s = cap * torch.tanh(s / cap)
                    dead = (causal and j > i) or (window and i - j >= window) or (doc is not None and doc[b, i] != doc[b, j])
                    r.append(s * 0 + float("-inf") if dead else s)
                if z64 is not None:
                    r += [z64[b, h, n] for n in range(z64.shape[2])]
                rows.append(torch.stack(r))
            heads.append(torch.stack(rows))
    full = torch.stack(heads).reshape(B, Hq, L, -1)
    out = torch.softmax(full, -1)[..., :S] @ vv
    return out, torch.logsumexp(full, -1), (q64, k64, v64, z64)


@pytest.mark.parametrize("case", ["alibi_causal", "head_bias_document", "soft_cap", "weighted", "all_with_sinks", "window_alibi"])
def test_score_mod_oracle_matches_float64_element_by_element(case):
    B, Hq, Hkv, L, E = 2, 4, 2, 20, 8
    g = torch.Generator().manual_seed(31)
    q, k, v, go = (torch.randn(B, h, L, E, generator=g) for h in (Hq, Hkv, Hkv, Hq))
    scale = 0.4
    slopes = torch.exp2(-(torch.arange(Hq) + 1) * 8.0 / Hq)
    kb, kw = torch.randn(Hq, L, generator=g), torch.rand(Hq, L, generator=g) + 0.5
    doc = torch.stack([torch.arange(L) // 7, torch.arange(L) // 5])
    cfg = {
        "alibi_causal": dict(causal=True, slopes=slopes),
        "head_bias_document": dict(kb=kb, doc=doc),
        "soft_cap": dict(cap=2.0),
        "weighted": dict(kw=kw),
        "all_with_sinks": dict(causal=True, slopes=slopes, cap=1.5, kb=kb, kw=kw, doc=doc, z=torch.randn(B, Hq, 3, generator=g)),
        "window_alibi": dict(causal=True, window=6, slopes=slopes, z=torch.randn(B, Hq, 1, generator=g)),
    }[case]
    c = dict(causal=False, window=0, z=None, slopes=None, cap=0.0, kb=None, kw=None, doc=None)
    c.update(cfg)
    kwargs = dict(is_causal=c["causal"], scale=scale, window=c["window"], sink_logit=c["z"], alibi_slopes=c["slopes"],
                  softcap=c["cap"], key_bias=c["kb"], key_weight=c["kw"], doc_ids_q=c["doc"], doc_ids_k=c["doc"])
    out, lse = om.sdpa_forward_score_mod(q, k, v, **kwargs)
    ro, rl, (q64, k64, v64, z64) = _score_mod_reference(q, k, v, scale, c["causal"], c["window"], c["z"], c["slopes"], c["cap"],
                                                        c["kb"], c["kw"], c["doc"])
    assert (out.double() - ro).abs().max() <= 2e-6 and (lse.double() - rl).abs().max() <= 2e-6
    dq, dk, dv, dz = om.sdpa_backward_score_mod(go, q, k, v, out, lse, **kwargs)
    wrt = (q64, k64, v64) + ((z64,) if z64 is not None else ())
    grads = torch.autograd.grad(ro, wrt, go.double())
    for a, r in zip((dq, dk, dv), grads[:3]):
        assert (a.double() - r).abs().max() <= 5e-6
    if z64 is not None:
        assert dz.shape == c["z"].shape and (dz.double() - grads[3]).abs().max() <= 5e-6


def test_score_mod_oracle_reduces_to_the_plain_functor_path():
    # no score functor, one sink logit: the explicit restatement equals the older one built on compute_attention
    g = torch.Generator().manual_seed(5)
    q, k, v, go = (torch.randn(1, h, 33, 16, generator=g) for h in (4, 2, 2, 4))
    z = torch.randn(1, 4, generator=g)
    a, la = om.sdpa_forward_score_mod(q, k, v, is_causal=True, window=9, sink_keys=2, sink_logit=z)
    b, lb = om.sdpa_forward_functor(q, k, v, is_causal=True, window=9, sink_keys=2, sink_logit=z)
    assert (a - b).abs().max() <= 1e-6 and (la - lb).abs().max() <= 1e-6
    ga = om.sdpa_backward_score_mod(go, q, k, v, a, la, is_causal=True, window=9, sink_keys=2, sink_logit=z)
    gb = om.sdpa_backward_functor(go, q, k, v, b, lb, is_causal=True, window=9, sink_keys=2, sink_logit=z)
    for x, y in zip(ga, gb):
        assert (x - y).abs().max() <= 2e-6
