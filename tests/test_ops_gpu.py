"""GPU tests of the operator layer: ATen registrations, autograd end to end, the kernel-level
custom ops, error behaviour and layout contracts - the cases of the reference's
tests/python_ops/test_scaled_dot_product_attention.py, with the CPU oracle as the checker."""

import math

import pytest
import torch
import torch.nn.functional as F

from helpers import max_abs, oracle_bwd, oracle_fwd, qkv, rel_err, seeded

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def amd(gpu_device):
    import torch_neuronx_amd as amd

    return amd


@pytest.fixture
def calls(amd, monkeypatch):
    """Counts launches that go through the C ABI."""
    seen = {"fwd": 0, "bwd": 0}
    f0, b0 = amd.ops.sdpa_forward, amd.ops.sdpa_backward

    def f(*a, **k):
        seen["fwd"] += 1
        return f0(*a, **k)

    def b(*a, **k):
        seen["bwd"] += 1
        return b0(*a, **k)

    monkeypatch.setattr(amd.ops, "sdpa_forward", f)
    monkeypatch.setattr(amd.ops, "sdpa_backward", b)
    return seen


@pytest.mark.parametrize("Hq,Hkv", [(8, 8), (24, 6), (8, 1)])
@pytest.mark.parametrize("dtype", [torch.float32, torch.float16, torch.bfloat16])
def test_functional_sdpa_fwd_bwd_lands_in_the_library(amd, gpu_device, calls, Hq, Hkv, dtype):
    # reference accuracy matrix: test_scaled_dot_product_attention.py:220-302
    q, k, v, go = qkv(1, Hq, Hkv, 512, 512, 64, dtype=dtype, seed=Hq, with_do=True)
    go = go.clamp(-1, 1) * 0.1
    qd, kd, vd = (t.to(gpu_device).requires_grad_(True) for t in (q, k, v))
    out = F.scaled_dot_product_attention(qd, kd, vd, enable_gqa=Hq != Hkv)
    out.backward(go.to(gpu_device))
    if dtype is torch.float32 and Hq != Hkv:
        # upstream's compiled-in backend table for GPU tensors sends float32 + enable_gqa to its
        # composite math path, which never reaches a fused-attention op; nothing to check here
        assert calls["fwd"] == 0
        return
    assert calls["fwd"] == 1 and calls["bwd"] == 1, calls
    ro, rl = oracle_fwd(q, k, v)
    rdq, rdk, rdv = oracle_bwd(go, q, k, v, ro, rl)
    tol = (1e-4, 1e-4) if dtype is torch.float32 else (2e-2, 5e-2)
    assert max_abs(out, ro) <= tol[0]
    for a, r in ((qd.grad, rdq), (kd.grad, rdk), (vd.grad, rdv)):
        assert a.shape == r.shape
        assert max_abs(a, r) <= tol[1]
        assert rel_err(a, r) <= (1e-4 if dtype is torch.float32 else 3e-2)


def test_functional_sdpa_with_masks(amd, gpu_device, calls):
    q, k, v = qkv(2, 4, 4, 64, 96, 64, dtype=torch.bfloat16, seed=3)
    g = torch.Generator().manual_seed(1)
    for mask in (torch.rand(2, 1, 64, 96, generator=g) > 0.3, torch.randn(64, 96, generator=g).to(torch.bfloat16)):
        mask = mask.clone()
        if mask.dtype == torch.bool:
            mask[..., 0] = True
        out = F.scaled_dot_product_attention(q.to(gpu_device), k.to(gpu_device), v.to(gpu_device),
                                             attn_mask=mask.to(gpu_device))
        ro, _ = oracle_fwd(q, k, v, attn_mask=mask if mask.dtype == torch.bool else mask.float())
        assert max_abs(out, ro) <= 2e-2
    assert calls["fwd"] == 2


def test_overrideable_op_contract(amd, gpu_device):
    # 9-tuple, float32 (B,H,L) lse also under no_grad: test_scaled_dot_product_attention.py:847-930
    q, k, v = (t.to(gpu_device) for t in qkv(1, 8, 2, 128, 128, 64, dtype=torch.bfloat16, seed=2))
    with torch.no_grad():
        r = torch.ops.aten._scaled_dot_product_fused_attention_overrideable(q, k, v, None, 0.0, True, False)
    assert len(r) == 9
    out, lse, csq, csk, mq, mk, seed, off, dbg = r
    assert out.shape == (1, 8, 128, 64) and lse.shape == (1, 8, 128) and lse.dtype == torch.float32
    assert csq is None and csk is None and dbg is None and mq == 128 and mk == 128
    assert seed.numel() == 0 and off.numel() == 0
    ro, rl = oracle_fwd(q.cpu(), k.cpu(), v.cpu(), is_causal=True)
    assert max_abs(out, ro) <= 2e-2 and max_abs(lse, rl) <= 2e-3
    go = torch.randn_like(out)
    dq, dk, dv, db = torch.ops.aten._scaled_dot_product_fused_attention_overrideable_backward(
        go, q, k, v, None, [True, True, True, False], out, lse, None, None, 128, 128, 0.0, True, seed, off)
    assert db is None and dk.shape == k.shape
    rdq, rdk, rdv = oracle_bwd(go.cpu(), q.cpu(), k.cpu(), v.cpu(), ro, rl, is_causal=True)
    for a, r in ((dq, rdq), (dk, rdk), (dv, rdv)):
        assert max_abs(a, r) <= 5e-2 and rel_err(a, r) <= 3e-2


def test_error_behaviour(amd, gpu_device):
    # test_scaled_dot_product_attention.py:305-359 and NeuronDispatcher.cpp:2377-2459
    q, k, v = (t.to(gpu_device) for t in qkv(1, 8, 2, 16, 16, 64, dtype=torch.bfloat16))
    op = torch.ops.aten._scaled_dot_product_fused_attention_overrideable
    with pytest.raises(NotImplementedError, match="Debug mask"):
        op(q, k, v, None, 0.0, False, True)
    with pytest.raises(RuntimeError, match="Explicit attn_mask should not be set"):
        op(q, k, v, torch.zeros(1, 8, 16, 16, device=gpu_device, dtype=torch.bfloat16), 0.0, True, False)
    with pytest.raises(RuntimeError, match="must divide the number of heads in query"):
        op(q, k[:, :1].expand(1, 3, 16, 64), v[:, :1].expand(1, 3, 16, 64))
    with pytest.raises(RuntimeError, match="same dtype"):
        op(q, k.float(), v)


def test_float64_round_trip(amd, gpu_device):
    # test_scaled_dot_product_attention.py:1288-1335: float64 is computed as float32
    q, k, v = qkv(1, 2, 2, 33, 33, 16, dtype=torch.float64, seed=6)
    r = torch.ops.aten._scaled_dot_product_fused_attention_overrideable(
        q.to(gpu_device), k.to(gpu_device), v.to(gpu_device))
    assert r[0].dtype == torch.float64 and r[1].dtype == torch.float32
    ro, rl = oracle_fwd(q, k, v)
    assert max_abs(r[0], ro) <= 1e-5


def test_zero_size_dims_take_the_math_backend(amd, gpu_device, calls):
    # test_scaled_dot_product_attention.py:1224-1285 / SdpBackendSelection.cpp:54-56
    q = torch.randn(1, 2, 4, 8, device=gpu_device)
    k = torch.randn(1, 2, 0, 8, device=gpu_device)
    out = F.scaled_dot_product_attention(q, k, k)
    assert out.shape == (1, 2, 4, 8) and calls["fwd"] == 0
    assert torch._fused_sdp_choice(q, k, k) == 0
    kk = torch.randn(1, 2, 4, 8, device=gpu_device)
    assert torch._fused_sdp_choice(q, kk, kk) == 4


def test_zero_size_head_dims_take_the_math_backend(amd, gpu_device, calls):
    # test_scaled_dot_product_attention.py:1224-1285: D_qk = 0 and D_v = 0 go to the math backend
    # (SdpBackendSelection.cpp:54-56) and equal the CPU result; gradients keep their inputs' shapes
    g = torch.Generator().manual_seed(0)
    for value_dim in (1, 8):
        for scale in (1.0, None):
            q = torch.empty((1, 16, 16, 0), device=gpu_device)
            k = torch.empty((1, 16, 16, 0), device=gpu_device)
            v = torch.randn((1, 16, 16, value_dim), generator=g).to(gpu_device)
            assert torch._fused_sdp_choice(q, k, v, scale=scale) == 0
            out = F.scaled_dot_product_attention(q, k, v, dropout_p=0.0, scale=scale)
            ref = F.scaled_dot_product_attention(q.cpu(), k.cpu(), v.cpu(), dropout_p=0.0, scale=scale)
            assert out.shape == (1, 16, 16, value_dim) and out.device.type == "cuda"
            torch.testing.assert_close(out.cpu(), ref)
    for qs, ks, vs in (((1, 4, 10, 8), (1, 4, 10, 8), (1, 4, 10, 0)), ((1, 4, 10, 8), (1, 4, 0, 8), (1, 4, 0, 8))):
        q, k, v = (torch.randn(*s_, generator=g).to(gpu_device).requires_grad_(True) for s_ in (qs, ks, vs))
        out = F.scaled_dot_product_attention(q, k, v, dropout_p=0.0)
        assert out.shape == (*qs[:-1], vs[-1])
        ref = F.scaled_dot_product_attention(q.detach().cpu(), k.detach().cpu(), v.detach().cpu(), dropout_p=0.0)
        torch.testing.assert_close(out.detach().cpu(), ref)
        out.sum().backward()
        assert q.grad.shape == q.shape and k.grad.shape == k.shape and v.grad.shape == v.shape
    assert calls["fwd"] == 0 and calls["bwd"] == 0


@pytest.mark.parametrize("Hq,S,D", [(8, 1280, 256), (8, 512, 64)])
def test_backward_with_stride0_expanded_kv(amd, gpu_device, calls, Hq, S, D):
    # test_scaled_dot_product_attention.py:1123-1221: K/V from repeat_kv's expand + reshape (stride 0 on
    # batch and heads).  The gradients of such views are dense tensors that alias nothing (autograd then
    # sums them back to the one real head), their leaf strides equal what the CPU gives, and here the
    # values are also checked against the oracle.
    def repeat_kv(t, n):
        b, kv, s, d = t.shape
        return t[:, :, None, :, :].expand(b, kv, n, s, d).reshape(b, kv * n, s, d)

    q, k, v, go = qkv(1, Hq, 1, S, S, D, dtype=torch.bfloat16, seed=21, with_do=True)
    qd, kd, vd = (t.to(gpu_device).requires_grad_(True) for t in (q, k, v))
    k_in, v_in = repeat_kv(kd, Hq), repeat_kv(vd, Hq)
    assert k_in.stride()[:2] == (0, 0) and v_in.stride()[:2] == (0, 0)
    seen = {}
    k_in.register_hook(lambda g_: seen.__setitem__("dk", g_))
    v_in.register_hook(lambda g_: seen.__setitem__("dv", g_))
    out = F.scaled_dot_product_attention(qd, k_in, v_in, is_causal=True)
    out.backward(go.to(gpu_device))
    assert calls["fwd"] == 1 and calls["bwd"] == 1
    for g_ in (seen["dk"], seen["dv"]):  # dense, one slab per (expanded) head
        assert g_.shape == (1, Hq, S, D) and g_.stride() == (Hq * S * D, S * D, D, 1)
    qc, kc, vc = (t.clone().requires_grad_(True) for t in (q, k, v))
    F.scaled_dot_product_attention(qc, repeat_kv(kc, Hq), repeat_kv(vc, Hq), is_causal=True).backward(go)
    assert qd.grad.stride() == qc.grad.stride() and kd.grad.stride() == kc.grad.stride()
    assert vd.grad.stride() == vc.grad.stride() and kd.grad.shape == k.shape
    ro, rl = oracle_fwd(q, k, v, is_causal=True)
    rdq, rdk, rdv = oracle_bwd(go, q, k, v, ro, rl, is_causal=True)
    assert max_abs(out, ro) <= 2e-2
    assert max_abs(qd.grad, rdq) <= 5e-2 and rel_err(qd.grad, rdq) <= 3e-2
    # (the leaf gradient is the sum of eight bf16 head gradients: one more rounding per head)
    for a, r in ((kd.grad, rdk), (vd.grad, rdv)):
        assert rel_err(a, r) <= 3e-2 and max_abs(a, r) <= 5e-2 + 2e-2 * r.abs().max().item()


def test_unregister_brings_the_stock_kernels_back(amd, gpu_device, calls):
    q, k, v = (t.to(gpu_device) for t in qkv(1, 4, 4, 128, 128, 64, dtype=torch.bfloat16, seed=3))
    F.scaled_dot_product_attention(q, k, v, is_causal=True)
    assert calls["fwd"] == 1
    names = amd.registered_ops()
    assert "_scaled_dot_product_flash_attention" in names
    amd.unregister()
    try:
        assert amd.registered_ops() == []
        out = F.scaled_dot_product_attention(q, k, v, is_causal=True)  # the stock kernel (or its math path)
        assert calls["fwd"] == 1
        ro, _ = oracle_fwd(q.cpu(), k.cpu(), v.cpu(), is_causal=True)
        assert max_abs(out, ro) <= 2e-2
    finally:
        amd.register()
    assert set(amd.registered_ops()) == set(names)
    F.scaled_dot_product_attention(q, k, v, is_causal=True)
    assert calls["fwd"] == 2


@pytest.mark.parametrize("shape,dtype,causal,with_bias", [
    ((1, 4, 4, 256, 64), torch.bfloat16, False, False),
    ((1, 4, 2, 512, 64), torch.float32, True, False),
    ((1, 4, 4, 256, 256), torch.bfloat16, False, True),
    ((1, 4, 2, 512, 256), torch.float32, True, False),
    ((1, 2, 1, 577, 64), torch.bfloat16, False, False),
])
def test_reference_accuracy_cases_run_in_the_matrix_op_kernels(amd, gpu_device, monkeypatch, shape, dtype, causal, with_bias):
    """The five cases of the reference's accuracy test (tests/python_ops/test_scaled_dot_product_attention.py:
    362-387) through F.scaled_dot_product_attention and autograd, at its tolerances (forward 5e-2 / 1e-2,
    backward 5e-2 / 5e-2) against the CPU; forced into the MFMA kernels, so that none of them can pass
    through the generic ones."""
    from torch_neuronx_amd.python_ops import scaled_dot_product_fused_attention as impl
    monkeypatch.setattr(impl, "_force_kernel", lambda: amd._lib.KERNEL_MFMA)
    B, Hq, Hkv, S, D = shape
    q, k, v = qkv(B, Hq, Hkv, S, S, D, dtype=dtype, seed=S + D)
    bias = torch.randn(B, Hq, S, S, generator=torch.Generator().manual_seed(1)).to(dtype) if with_bias else None
    go = (torch.randn(B, Hq, S, D, generator=torch.Generator().manual_seed(2)).clamp(-1, 1) * 0.1).to(dtype)
    rep = Hq // Hkv

    def run(dev):
        qd, kd, vd = (t.to(dev).requires_grad_(True) for t in (q, k, v))
        kk, vv = (kd.repeat_interleave(rep, 1), vd.repeat_interleave(rep, 1)) if dev == "cpu" else (kd, vd)
        out = F.scaled_dot_product_attention(qd, kk, vv, attn_mask=None if bias is None else bias.to(dev), is_causal=causal,
                                             enable_gqa=(dev != "cpu" and rep > 1))
        out.backward(go.to(dev))
        return out.detach().cpu(), qd.grad.cpu(), kd.grad.cpu(), vd.grad.cpu()

    got, ref = run(gpu_device), run("cpu")
    torch.testing.assert_close(got[0].float(), ref[0].float(), atol=5e-2, rtol=1e-2)
    for a, b_ in zip(got[1:], ref[1:]):
        torch.testing.assert_close(a.float(), b_.float(), atol=5e-2, rtol=5e-2)


def test_a_keep_mask_of_one_element_is_a_placeholder(amd, gpu_device):
    """The reference treats a dropout mask of one element as absent (torch_neuronx/_sdpa_math.py:42-45):
    so do the forward and the backward here, whatever the byte says and whatever dropout_p is."""
    from oracle import sdpa_math as om
    dev = gpu_device
    q, k, v, go = (t.to(dev) for t in qkv(1, 1, 1, 1, 1, 64, dtype=torch.float32, seed=3, with_do=True))
    keep = torch.zeros(1, 1, 1, 1, dtype=torch.bool, device=dev)
    out, lse = amd.sdpa_forward(q, k, v, dropout_p=0.9, dropout_keep=keep)
    dq, dk, dv, _ = amd.sdpa_backward(go, q, k, v, out, lse, dropout_p=0.9, dropout_keep=keep)
    ro, rl = om.compute_attention(q.cpu(), k.cpu(), v.cpu(), None, keep.cpu(), 64**-0.5, False, 0.9)
    rdq, rdk, rdv, _ = om.compute_attention_backward(go.cpu(), q.cpu(), k.cpu(), v.cpu(), None, keep.cpu(), ro, rl, 64**-0.5, False, 0.9)
    assert max_abs(out, ro) <= 1e-6 and max_abs(out, v) <= 1e-6  # (one key: the output is its value row, undropped and unscaled)
    for a, r in ((dq, rdq), (dk, rdk), (dv, rdv)):
        assert max_abs(a, r) <= 1e-6


def test_dropout_extremes_and_mask_round_trip(amd, gpu_device):
    q, k, v = (t.to(gpu_device) for t in qkv(1, 2, 2, 32, 32, 32, dtype=torch.float32, seed=8))
    op = torch.ops.aten._scaled_dot_product_fused_attention_overrideable
    out1 = op(q, k, v, None, 1.0)[0]
    assert torch.equal(out1, torch.zeros_like(out1))
    r = op(q, k, v, None, 0.5)
    keep = r[6]
    assert keep.shape == (1, 2, 32, 32)
    from oracle import sdpa_math as om

    ro, rl = om.compute_attention(q.cpu(), k.cpu(), v.cpu(), None, keep.cpu().bool(), 32**-0.5, False, 0.5)
    assert max_abs(r[0], ro) <= 1e-5
    go = torch.randn_like(r[0])
    dq, dk, dv, _ = torch.ops.aten._scaled_dot_product_fused_attention_overrideable_backward(
        go, q, k, v, None, [True, True, True, False], r[0], r[1], None, None, 32, 32, 0.5, False, keep, r[7])
    rdq, rdk, rdv, _ = om.compute_attention_backward(go.cpu(), q.cpu(), k.cpu(), v.cpu(), None, keep.cpu().bool(),
                                                     ro, rl, 32**-0.5, False, 0.5)
    for a, b_ in ((dq, rdq), (dk, rdk), (dv, rdv)):
        assert max_abs(a, b_) <= 5e-5


def test_kernel_level_custom_ops(amd, gpu_device):
    q, k, v, go = (t.to(gpu_device) for t in qkv(2, 8, 2, 256, 256, 128, dtype=torch.bfloat16, seed=5, with_do=True))
    lse = torch.empty(2, 8, 256, dtype=torch.float32, device=gpu_device)
    out = amd.scaled_dot_product_attention_kernel(q, k, v, is_causal=True, training=True, lse=lse)
    out2 = amd.scaled_dot_product_attention_kernel(q, k, v, is_causal=True, dropout_p=0.3, seed=7)
    assert torch.equal(out, out2)  # dropout_p / seed are accepted and not consumed
    ro, rl = oracle_fwd(q.cpu(), k.cpu(), v.cpu(), is_causal=True)
    assert max_abs(out, ro) <= 2e-2 and max_abs(lse, rl) <= 2e-3
    dq, dk, dv = amd.scaled_dot_product_attention_backward_kernel(go, q, k, v, out, lse, True)
    tiled = lse.reshape(2, 8, 2, 128).transpose(-1, -2).contiguous()  # (B,H,128,L/128) form
    dq2, dk2, dv2 = amd.scaled_dot_product_attention_backward_kernel(go, q, k, v, out, tiled, True)
    assert torch.equal(dq, dq2) and torch.equal(dk, dk2)
    # a tiled buffer filled by the forward op holds row t * 128 + p at [p, t], which is what the
    # backward op reads from it: forward -> backward round trip through the 4-D form
    tiled_fwd = torch.empty(2, 8, 128, 2, dtype=torch.float32, device=gpu_device)
    out3 = amd.scaled_dot_product_attention_kernel(q, k, v, is_causal=True, training=True, lse=tiled_fwd)
    assert torch.equal(out3, out) and torch.equal(tiled_fwd, tiled)
    dq3, dk3, dv3 = amd.scaled_dot_product_attention_backward_kernel(go, q, k, v, out3, tiled_fwd, True)
    assert torch.equal(dq, dq3) and torch.equal(dk, dk3) and torch.equal(dv, dv3)
    with pytest.raises(ValueError):  # same element count, wrong shape: refused, not reshaped
        amd.scaled_dot_product_attention_kernel(q, k, v, is_causal=True, training=True,
                                                lse=torch.empty(2, 8, 2, 128, dtype=torch.float32, device=gpu_device))
    rdq, rdk, rdv = oracle_bwd(go.cpu(), q.cpu(), k.cpu(), v.cpu(), ro, rl, is_causal=True)
    for a, r in ((dq, rdq), (dk, rdk), (dv, rdv)):
        assert max_abs(a, r) <= 5e-2 and rel_err(a, r) <= 3e-2


def test_llama_style_transposed_views_fwd_bwd(amd, gpu_device):
    # model code hands in (B,S,H,D).transpose(1,2) views and transposes the output back
    B, S, Hq, Hkv, D = 2, 256, 8, 2, 128
    g = torch.Generator().manual_seed(4)
    xq = torch.randn(B, S, Hq, D, generator=g).to(torch.bfloat16).to(gpu_device).requires_grad_(True)
    xk = torch.randn(B, S, Hkv, D, generator=g).to(torch.bfloat16).to(gpu_device).requires_grad_(True)
    xv = torch.randn(B, S, Hkv, D, generator=g).to(torch.bfloat16).to(gpu_device).requires_grad_(True)
    out = F.scaled_dot_product_attention(xq.transpose(1, 2), xk.transpose(1, 2), xv.transpose(1, 2),
                                         is_causal=True, enable_gqa=True)
    assert out.transpose(1, 2).is_contiguous()
    y = out.transpose(1, 2).reshape(B, S, Hq * D)
    go = torch.randn(B, S, Hq * D, generator=g).to(torch.bfloat16).to(gpu_device)
    y.backward(go)
    q, k, v = (t.detach().cpu().transpose(1, 2) for t in (xq, xk, xv))
    ro, rl = oracle_fwd(q, k, v, is_causal=True)
    rdq, rdk, rdv = oracle_bwd(go.cpu().reshape(B, S, Hq, D).transpose(1, 2), q, k, v, ro, rl, is_causal=True)
    assert max_abs(out, ro) <= 2e-2
    for a, r in ((xq.grad, rdq), (xk.grad, rdk), (xv.grad, rdv)):
        assert max_abs(a.transpose(1, 2), r) <= 5e-2 and rel_err(a.transpose(1, 2), r) <= 3e-2


# ---- middle stage of native multi-head attention ([B, H, D, S] operands) ---------------------------
# cases of the reference's tests/python_ops/test_native_multi_head_attn_mid.py, checked against
# the oracle instead of only for shape and NaNs

@pytest.mark.parametrize("dtype,B,H,D,S,causal", [
    (torch.float32, 1, 8, 128, 512, False),
    (torch.float32, 2, 4, 64, 384, True),       # a length the reference sends to its fallback
    (torch.bfloat16, 1, 8, 128, 2048, False),
    (torch.bfloat16, 1, 8, 128, 2048, True),
    (torch.float16, 4, 16, 64, 1024, True),
])
def test_native_mha_mid(amd, gpu_device, dtype, B, H, D, S, causal):
    q, k, v = qkv(B, H, H, S, S, D, dtype=dtype, seed=77)
    # the op's layout: sequence last
    qm, km, vm = (t.transpose(-2, -1).contiguous().to(gpu_device) for t in (q, k, v))
    got = amd.native_multi_head_attn_mid(qm, km, vm, use_causal_mask=causal, dropout_p=0.0, training=False)
    assert got.shape == (B, H, S, D) and got.device.type == "cuda" and got.dtype == dtype
    ref, _ = oracle_fwd(q, k, v, is_causal=causal)
    tol = 1e-5 if dtype is torch.float32 else 2e-2  # fp32 1e-5, half precisions 2e-2 against the fp32 oracle
    assert max_abs(got, ref) <= tol
    assert rel_err(got, ref) <= (1e-5 if dtype is torch.float32 else 1e-2)


def test_native_mha_mid_gqa_and_value_width(amd, gpu_device):
    # general form: H_kv key/value heads, value rows of their own width
    B, Hq, Hkv, D, Dv, Sq, Sk = 2, 8, 2, 64, 32, 96, 160
    q, k, v = qkv(B, Hq, Hkv, Sq, Sk, D, Dv=Dv, dtype=torch.float32, seed=78)
    qm, km, vm = (t.transpose(-2, -1).contiguous().to(gpu_device) for t in (q, k, v))
    got = amd.native_multi_head_attn_mid(qm, km, vm)
    ref, _ = oracle_fwd(q, k.repeat_interleave(Hq // Hkv, 1), v.repeat_interleave(Hq // Hkv, 1))
    assert got.shape == (B, Hq, Sq, Dv)
    assert max_abs(got, ref) <= 1e-5


def test_native_mha_mid_out_variant(amd, gpu_device):
    B, H, D, S = 1, 8, 128, 512
    q, k, v = qkv(B, H, H, S, S, D, dtype=torch.bfloat16, seed=79)
    qm, km, vm = (t.transpose(-2, -1).contiguous().to(gpu_device) for t in (q, k, v))
    out = torch.empty(B, H, S, D, dtype=torch.bfloat16, device=gpu_device)
    got = amd.native_multi_head_attn_mid(qm, km, vm, out=out)
    assert got is out
    ref, _ = oracle_fwd(q, k, v)
    assert max_abs(out, ref) <= 2e-2
    with pytest.raises(RuntimeError, match="doesn't match expected shape"):
        amd.native_multi_head_attn_mid(qm, km, vm, out=torch.empty(B, H, D, S, dtype=torch.bfloat16, device=gpu_device))


def test_native_mha_mid_errors(amd, gpu_device):
    B, H, D, S = 1, 8, 128, 2048
    mk = lambda *shape: torch.randn(*shape, device=gpu_device)
    q, k, v = mk(B, H, D, S), mk(B, H, D, S), mk(B, H, D, S)
    with pytest.raises(RuntimeError):  # key shorter than value
        amd.native_multi_head_attn_mid(q, mk(B, H, D, S // 2), v)
    with pytest.raises(RuntimeError):  # value shorter than key
        amd.native_multi_head_attn_mid(q, k, mk(B, H, D, S // 2))
    with pytest.raises(RuntimeError):  # value in [B, H, S, D] order
        amd.native_multi_head_attn_mid(q, k, mk(B, H, S, D))
    with pytest.raises(RuntimeError, match="do not support empty tensors"):
        amd.native_multi_head_attn_mid(mk(0, H, D, S), mk(0, H, D, S), mk(0, H, D, S))
    with pytest.raises(RuntimeError, match="4-dimensional"):
        amd.native_multi_head_attn_mid(mk(H, D, S), mk(H, D, S), mk(H, D, S))
    with pytest.raises(ValueError):
        amd.native_multi_head_attn_mid(q.cpu(), k.cpu(), v.cpu())


# ---- HIP graph capture -----------------------------------------------------------------------------

def test_traced_module_reaches_the_library(amd, gpu_device, calls):
    # a compiled (traced with fake tensors, run with the eager backend) attention block: the registered
    # operators are what the traced graph calls, forward and backward, and the numbers are the eager ones
    q, k, v = (t.to(gpu_device).requires_grad_(True) for t in qkv(2, 8, 2, 256, 256, 64, dtype=torch.bfloat16, seed=21))

    def block(q, k, v):
        return F.scaled_dot_product_attention(q, k, v, is_causal=True, enable_gqa=True).float().square().sum()

    ref = block(q, k, v)
    ref.backward()
    eager = [t.grad.clone() for t in (q, k, v)]
    for t in (q, k, v):
        t.grad = None
    before = dict(calls)
    torch._dynamo.reset()
    got = torch.compile(block, backend="aot_eager")(q, k, v)
    got.backward()
    assert calls["fwd"] > before["fwd"] and calls["bwd"] > before["bwd"], calls
    assert torch.equal(got, ref)
    for t, e in zip((q, k, v), eager):
        assert torch.equal(t.grad, e)


@pytest.mark.parametrize("case", ["causal_gqa", "padding_mask", "bias_with_gradient", "float32"])
def test_compiled_module_with_the_default_backend(amd, gpu_device, calls, case):
    """torch.compile's default backend calls the attention operators as they are and asserts, in the code it
    generates, that their outputs have the sizes and strides upstream's operators promise (output laid out
    like the query for the flash operator and (B,L,H,Dv) for the memory-efficient one, 0-dim int64 seed and
    offset, gradients (B,L,H,D), the bias gradient a view of rows padded to 16 keys).  The replacements
    registered here keep those promises: the compiled block runs and gives the eager numbers."""
    dev = gpu_device
    g = torch.Generator().manual_seed(31)
    mk = lambda *shape, dtype=torch.bfloat16: torch.randn(*shape, generator=g).to(dtype).to(dev).requires_grad_(True)
    if case == "causal_gqa":
        args = (mk(2, 8, 256, 64), mk(2, 2, 256, 64), mk(2, 2, 256, 64))
        block = lambda q, k, v: (F.scaled_dot_product_attention(q * 1.0, k, v, is_causal=True, enable_gqa=True).float() * 2).square().sum()
    elif case == "padding_mask":
        args = (mk(2, 4, 128, 64), mk(2, 4, 128, 64), mk(2, 4, 128, 64))
        pad = torch.ones(2, 1, 1, 128, dtype=torch.bool, device=dev)
        pad[1, ..., 100:] = False
        block = lambda q, k, v: F.scaled_dot_product_attention(q, k, v, attn_mask=pad).float().square().sum()
    elif case == "bias_with_gradient":
        args = (mk(2, 4, 128, 64), mk(2, 4, 128, 64), mk(2, 4, 128, 64), mk(1, 4, 128, 120))
        block = lambda q, k, v, b: F.scaled_dot_product_attention(q, k[:, :, :120], v[:, :, :120], attn_mask=b).float().square().sum()
    else:
        args = (mk(2, 4, 128, 64, dtype=torch.float32),)
        block = lambda q: F.scaled_dot_product_attention(q, q, q, is_causal=True).square().sum()
    ref = block(*args)
    ref.backward()
    eager = [t.grad.clone() for t in args]
    for t in args:
        t.grad = None
    before = dict(calls)
    torch._dynamo.reset()
    got = torch.compile(block)(*args)
    got.backward()
    assert calls["fwd"] > before["fwd"] and calls["bwd"] > before["bwd"], calls
    assert torch.allclose(got, ref, rtol=1e-5)
    for t, e in zip(args, eager):
        assert max_abs(t.grad, e) <= 1e-6 * max(1.0, float(e.abs().max()))
    torch._dynamo.reset()


def test_functional_call_routed_by_the_reference_rules(amd, gpu_device, calls):
    """float32 with grouped heads: upstream's compiled-in backend choice for GPUs has no fused kernel for
    it and takes the unfused path (no call reaches the library); with ``route_functional`` the choice is
    the reference's (SdpBackendSelection.cpp:14-68: the fused operator for every plain 4-D call), forward
    and backward run in the library and agree with the oracle; switching it off restores the stock function."""
    stock = F.scaled_dot_product_attention
    q, k, v, go = qkv(2, 8, 2, 200, 200, 64, dtype=torch.float32, seed=3, with_do=True)
    qd, kd, vd = (t.to(gpu_device).requires_grad_(True) for t in (q, k, v))
    before = dict(calls)
    F.scaled_dot_product_attention(qd, kd, vd, is_causal=True, enable_gqa=True)
    assert calls == before
    amd.route_functional(True)
    try:
        assert F.scaled_dot_product_attention is not stock
        out = F.scaled_dot_product_attention(qd, kd, vd, is_causal=True, enable_gqa=True)
        out.backward(go.to(gpu_device))
        assert calls["fwd"] == before["fwd"] + 1 and calls["bwd"] == before["bwd"] + 1
        ro, rl = oracle_fwd(q, k, v, is_causal=True)
        rdq, rdk, rdv = oracle_bwd(go, q, k, v, ro, rl, is_causal=True)[:3]
        assert max_abs(out, ro) <= 2e-5
        for a, b_ in ((qd.grad, rdq), (kd.grad, rdk), (vd.grad, rdv)):
            assert max_abs(a, b_) <= 5e-5
        # what is no plain 4-D GPU call keeps upstream's route
        cpu = F.scaled_dot_product_attention(q, k, v, is_causal=True, enable_gqa=True)
        assert max_abs(cpu, ro) <= 2e-5
        with pytest.raises(RuntimeError):
            F.scaled_dot_product_attention(qd, kd, vd, is_causal=True)  # (heads differ and no enable_gqa: upstream's error)
    finally:
        amd.route_functional(False)
    assert F.scaled_dot_product_attention is stock


def test_replaced_upstream_operators_keep_upstream_layouts_and_redraw_the_dropout_mask(amd, gpu_device):
    """The flash and memory-efficient operators called directly with dropout: outputs in upstream's shapes
    and layouts; seed and offset are the generator's state before the draw, the backward draws the same
    keep-mask from them (the mask does not travel), and forward and backward agree with the oracle given
    that mask."""
    from oracle import sdpa_math as om
    from torch_neuronx_amd.python_ops import scaled_dot_product_fused_attention as impl

    dev = gpu_device
    B, H, L, S, D, p = 2, 4, 128, 120, 64, 0.2
    g = torch.Generator().manual_seed(77)
    mk = lambda *shape: torch.randn(*shape, generator=g).to(torch.bfloat16).to(dev)
    q, k, v, go, bias = mk(B, H, L, D), mk(B, H, S, D), mk(B, H, S, D), mk(B, H, L, D), mk(B, H, L, S)
    qc, kc, vc, gc, bc = (t.float().cpu() for t in (q, k, v, go, bias))
    torch.cuda.manual_seed(5)
    r = torch.ops.aten._scaled_dot_product_efficient_attention(q, k, v, bias, True, p, False)
    out, lse, seed, offset = r
    assert out.shape == (B, H, L, D) and out.stride() == (L * H * D, D, H * D, 1)
    assert lse.shape == (B, H, L) and lse.dtype == torch.float32
    for t in (seed, offset):
        assert t.dim() == 0 and t.dtype == torch.int64 and t.device.type == "cpu"
    assert int(seed) == 5
    keep = impl._keep_again(q, S, p, seed, offset).cpu().bool()
    assert 0.75 < keep.float().mean().item() < 0.85
    ro, rl = om.compute_attention(qc, kc, vc, bc, keep, D**-0.5, False, p)
    assert max_abs(out, ro) <= 2e-2 and max_abs(lse, rl) <= 2e-3
    dq, dk, dv, db = torch.ops.aten._scaled_dot_product_efficient_attention_backward(
        go, q, k, v, bias, out, lse, seed, offset, p, [True, True, True, True])
    for t, n in ((dq, L), (dk, S), (dv, S)):
        assert t.stride() == (n * H * D, D, H * D, 1)
    assert db.shape == (B, H, L, S) and db.stride() == (H * L * 128, L * 128, 128, 1)
    rdq, rdk, rdv, rdb = om.compute_attention_backward(gc, qc, kc, vc, bc, keep, ro, rl, D**-0.5, False, p)
    for a, b_ in ((dq, rdq), (dk, rdk), (dv, rdv), (db, rdb)):
        assert max_abs(a, b_) <= 5e-2 * max(1.0, float(b_.abs().max()))
    # the next call draws at a later offset, hence another mask
    r2 = torch.ops.aten._scaled_dot_product_flash_attention(q, k, v, p, False)
    assert int(r2[6]) == 5 and int(r2[7]) > int(offset)
    assert r2[6].dim() == 0 and r2[7].dim() == 0 and r2[8].numel() == 0
    keep2 = impl._keep_again(q, S, p, r2[6], r2[7]).cpu().bool()
    assert not torch.equal(keep2, keep)
    ro2, rl2 = om.compute_attention(qc, kc, vc, None, keep2, D**-0.5, False, p)
    assert max_abs(r2[0], ro2) <= 2e-2
    g3 = torch.ops.aten._scaled_dot_product_flash_attention_backward(go, q, k, v, r2[0], r2[1], None, None, L, S, p, False, r2[6], r2[7])
    r3 = om.compute_attention_backward(gc, qc, kc, vc, None, keep2, ro2, rl2, D**-0.5, False, p)
    for a, b_ in zip(g3, r3[:3]):
        assert max_abs(a, b_) <= 5e-2 * max(1.0, float(b_.abs().max()))
    # through autograd the forward keeps its mask for the backward, which takes it; a backward that does
    # not find it (evicted from the bounded store) draws it again: the same gradients, bit for bit
    qr, kr, vr = (t.clone().requires_grad_(True) for t in (q, k, v))
    impl._kept.clear()
    grads = []
    for lose_it in (False, True):
        torch.cuda.manual_seed(9)
        out = F.scaled_dot_product_attention(qr, kr, vr, dropout_p=p)
        assert len(impl._kept) == 1
        if lose_it:
            impl._kept.clear()
        out.backward(go)
        assert len(impl._kept) == 0
        grads.append([t.grad.clone() for t in (qr, kr, vr)])
        qr.grad = kr.grad = vr.grad = None
    for a, b_ in zip(*grads):
        assert torch.equal(a, b_)
    with torch.no_grad():  # (no backward can follow: nothing is kept)
        F.scaled_dot_product_attention(qr, kr, vr, dropout_p=p)
    assert len(impl._kept) == 0
    out = F.scaled_dot_product_attention(qr, kr, vr, dropout_p=p)  # a forward whose backward never comes ...
    assert len(impl._kept) == 1
    del out  # ... gives its mask back when its graph goes
    import gc
    gc.collect()
    assert len(impl._kept) == 0


def test_calls_can_be_captured_in_a_graph_and_replayed(amd, gpu_device):
    # The library only launches kernels on the stream it is given (no allocation, no memset, no
    # synchronisation), so forward, backward and decode can be recorded into one graph.  The graph
    # is replayed several times on fresh inputs, with eager work and synchronisations in between,
    # and every replay is checked against the eager result.
    from oracle import sdpa_math as om

    dev = gpu_device
    B, Hq, Hkv, L, E = 2, 8, 2, 256, 128
    g = torch.Generator().manual_seed(404)
    mk = lambda *s: torch.randn(*s, generator=g).to(torch.bfloat16).to(dev)
    q, k, v, go = mk(B, Hq, L, E), mk(B, Hkv, L, E), mk(B, Hkv, L, E), mk(B, Hq, L, E)
    bias = mk(1, Hq, L, L)
    qd = mk(4, Hq, 1, E)
    kq, ks = om.quantize_kv_fp8(torch.randn(4, Hkv, 512, E, generator=g))
    vq, vs = om.quantize_kv_fp8(torch.randn(4, Hkv, 512, E, generator=g))
    kq, vq, ks, vs = kq.to(dev), vq.to(dev), ks.to(dev), vs.to(dev)
    lens = torch.tensor([512, 1, 300, 77], dtype=torch.int32, device=dev)
    # calls that split their work over more workgroups and add the parts up in a second kernel: a
    # decode-like forward over long keys, a backward with one kv head
    q1, kl, vl = mk(1, Hq, 1, E), mk(1, Hkv, 4096, E), mk(1, Hkv, 4096, E)
    qm, km, vm, gom = mk(1, 8, 512, E), mk(1, 1, 512, E), mk(1, 1, 512, E), mk(1, 8, 512, E)

    def work():
        out, lse = amd.sdpa_forward(q, k, v, is_causal=True)
        dq, dk, dv, _ = amd.sdpa_backward(go, q, k, v, out, lse, is_causal=True)
        outb, lseb = amd.sdpa_forward(q, k, v, attn_bias=bias)
        dqb, dkb, dvb, dbb = amd.sdpa_backward(go, q, k, v, outb, lseb, attn_bias=bias, want_grad_bias=True)
        od, ld = amd.decode_fp8kv(qd, kq, vq, ks, vs, lens)
        o1, l1 = amd.sdpa_forward(q1, kl, vl)
        om_, lm = amd.sdpa_forward(qm, km, vm, is_causal=True)
        dqm, dkm, dvm, _ = amd.sdpa_backward(gom, qm, km, vm, om_, lm, is_causal=True)
        return [out, lse, dq, dk, dv, outb, dqb, dkb, dvb, dbb, od, ld, o1, l1, dqm, dkm, dvm]

    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        work()  # warm-up outside the capture (first-launch attribute calls, allocator pools)
    torch.cuda.current_stream().wait_stream(side)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        captured = work()
    for rep in range(3):
        for t in (q, k, v, go, qd, q1, kl, qm, km, gom):
            t.copy_(torch.randn(t.shape, generator=g).to(t.dtype))
        bias.mul_(0.5)
        eager = [t.clone() for t in work()]
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        for i, (a, b) in enumerate(zip(captured, eager)):
            assert torch.equal(a, b), (rep, i)


def _padding_case(dev, seed=11):
    B, H, L, E = 3, 4, 512, 64
    q, k, v = (t.to(dev) for t in qkv(B, H, H, L, L, E, dtype=torch.bfloat16, seed=seed))
    lens = torch.tensor([L, 300, 77])
    pad = (torch.arange(L)[None] < lens[:, None])[:, None, None, :]
    return q, k, v, pad


def test_masks_made_under_inference_mode(amd, gpu_device):
    """Tensors created under torch.inference_mode() have no version counter: their masks are taken as
    they are (no recognition, no cache, no tables) instead of raising.  Bool and additive masks, a
    recognisable one (causal) and a padding one, forward only, against the oracle."""
    from oracle import sdpa_math as om

    dev = gpu_device
    q, k, v, pad = _padding_case(dev)
    L = q.shape[2]
    amd.mask_patterns.clear_cache()
    with torch.inference_mode():
        tril = torch.ones(L, L, dtype=torch.bool, device=dev).tril()
        add = torch.zeros(L, L, dtype=torch.bfloat16, device=dev).masked_fill(~tril, float("-inf"))
        padd = pad.to(dev)
        big = torch.ones(1, 1, L, L, dtype=torch.bool, device=dev).tril()  # large enough for skip tables
        for mask, keep in ((tril, tril.cpu()), (add, tril.cpu()), (padd, pad), (big, tril.cpu())):
            assert mask.is_inference()
            out = F.scaled_dot_product_attention(q, k, v, attn_mask=mask)
            ro, _ = om.sdpa_forward(q.float().cpu(), k.float().cpu(), v.float().cpu(), attn_mask=keep)
            assert max_abs(out, ro) <= 2e-2
            r = torch.ops.aten._scaled_dot_product_fused_attention_overrideable(q, k, v, mask)
            assert max_abs(r[0], ro) <= 2e-2
    assert len(amd.mask_patterns._cache) == 0 and len(amd.mask_patterns._tile_cache) == 0


def test_mask_changed_in_place_between_calls(amd, gpu_device):
    """A verdict is valid for one version of the tensor: after an in-place write the next call follows
    the new contents (a padding mask whose lengths change, a causal mask that stops being one)."""
    from oracle import sdpa_math as om

    dev = gpu_device
    q, k, v, pad = _padding_case(dev, seed=12)
    L = q.shape[2]
    fused = torch.ops.aten._scaled_dot_product_fused_attention_overrideable
    ref = lambda keep: om.sdpa_forward(q.float().cpu(), k.float().cpu(), v.float().cpu(), attn_mask=keep)[0]
    amd.mask_patterns.clear_cache()
    padd = pad.to(dev)
    for _ in range(2):  # (the second call is served from the cache)
        assert max_abs(fused(q, k, v, padd)[0], ref(pad)) <= 2e-2
    pad2 = (torch.arange(L)[None] < torch.tensor([100, L, 9])[:, None])[:, None, None, :]
    padd.copy_(pad2)
    assert max_abs(fused(q, k, v, padd)[0], ref(pad2)) <= 2e-2
    pad3 = pad2.clone()
    pad3[1, 0, 0, 5] = False  # no longer "keys 0 .. n-1"
    padd.copy_(pad3)
    assert max_abs(fused(q, k, v, padd)[0], ref(pad3)) <= 2e-2
    tril = torch.ones(1, 1, L, L, dtype=torch.bool, device=dev).tril()
    for _ in range(2):
        assert max_abs(fused(q, k, v, tril)[0], ref(tril.cpu())) <= 2e-2
    tril[0, 0, 3, 400] = True
    assert max_abs(fused(q, k, v, tril)[0], ref(tril.cpu())) <= 2e-2
    with amd.mask_patterns.left_alone():  # the per-call opt-out: the mask is taken as it is
        looked = amd.mask_patterns.stats["looked"]
        assert max_abs(fused(q, k, v, padd)[0], ref(pad3)) <= 2e-2
        assert amd.mask_patterns.stats["looked"] == looked


def test_a_captured_call_reads_its_mask_on_every_replay(amd, gpu_device):
    """The usual graph contract: warm up with the static mask tensor, capture, then update the mask
    in place between replays.  A captured call never uses a cached verdict about the mask (that
    would freeze the old key counts into the graph): every replay follows the tensor's contents."""
    from oracle import sdpa_math as om

    dev = gpu_device
    q, k, v, pad = _padding_case(dev, seed=13)
    L = q.shape[2]
    padd = pad.to(dev)
    tril = torch.ones(1, 1, L, L, dtype=torch.bool, device=dev).tril()
    fused = torch.ops.aten._scaled_dot_product_fused_attention_overrideable
    amd.mask_patterns.clear_cache()

    def work():
        return [fused(q, k, v, padd)[0], fused(q, k, v, tril)[0], F.scaled_dot_product_attention(q, k, v, attn_mask=padd)]

    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        for _ in range(2):
            work()  # warm-up: the verdicts of both masks are in the cache now
    torch.cuda.current_stream().wait_stream(side)
    assert len(amd.mask_patterns._cache) >= 2
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        captured = work()
    for lens in ([L, 300, 77], [5, L, 200], [L, L, L]):
        keep = (torch.arange(L)[None] < torch.tensor(lens)[:, None])[:, None, None, :]
        padd.copy_(keep)
        tril[0, 0, 7, L - 1] = lens[0] == 5  # the second replay's mask is not causal
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        ro = om.sdpa_forward(q.float().cpu(), k.float().cpu(), v.float().cpu(), attn_mask=keep)[0]
        rt = om.sdpa_forward(q.float().cpu(), k.float().cpu(), v.float().cpu(), attn_mask=tril.cpu())[0]
        assert max_abs(captured[0], ro) <= 2e-2 and max_abs(captured[2], ro) <= 2e-2, lens
        assert max_abs(captured[1], rt) <= 2e-2, lens


def test_fallback_to_the_generic_kernel_can_be_logged(gpu_device):
    """MI355_SDPA_LOG_FALLBACK=1: a call that the matrix-op kernels cannot take (head dim 100) says so
    on stderr, with the reason; a call they take says nothing.  (A child process: the switch is read once.)"""
    import os
    import subprocess
    import sys

    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    code = (
        "import sys, torch\n"
        f"sys.path.insert(0, {root!r}); sys.path.insert(0, {os.path.join(root, 'torch-neuronx_amd')!r})\n"
        "import torch_neuronx_amd as amd\n"
        "d = torch.device('cuda:0')\n"
        "q = torch.randn(1, 2, 64, 128, device=d, dtype=torch.bfloat16)\n"
        "amd.sdpa_forward(q, q, q, is_causal=True)\n"
        "print('--', file=sys.stderr, flush=True)\n"
        "q = torch.randn(1, 2, 64, 100, device=d, dtype=torch.bfloat16)\n"
        "o, l = amd.sdpa_forward(q, q, q)\n"
        "amd.sdpa_backward(q, q, q, q, o, l)\n"
        "torch.cuda.synchronize()\n"
    )
    env = dict(os.environ, MI355_SDPA_LOG_FALLBACK="1")
    r = subprocess.run([sys.executable, "-c", code], env=env, capture_output=True, text=True, timeout=300)
    assert r.returncode == 0, r.stderr
    before, _, after = r.stderr.partition("--")
    assert "mi355_sdpa" not in before
    assert "forward runs in the generic kernel: head dims are not multiples of 8" in after
    assert "backward runs in the generic kernel" in after


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("kind", ["odd_keys_16bit", "odd_keys_bool", "offset_slice", "odd_row_stride", "odd_keys_grad"])
def test_biases_that_are_not_dword_aligned_still_run_in_the_matrix_op_kernels(amd, gpu_device, dtype, kind):
    # the host repacks such a bias once (over its own extents) rather than letting the call leave the
    # matrix-op kernels; forced, so the call fails if they refuse it.  Forward, backward and - for the
    # last kind - the gradient of the bias over a number of keys that is no multiple of four.
    from oracle import sdpa_math as om

    dev = gpu_device
    B, Hq, Hkv, L, E = 2, 4, 2, 130, 64
    S = 150 if kind == "odd_keys_grad" else 77 if kind.startswith("odd_keys") else 96
    q, k, v, go = seeded([(B, Hq, L, E), (B, Hkv, S, E), (B, Hkv, S, E), (B, Hq, L, E)], len(kind), dtype)
    g = torch.Generator().manual_seed(S)
    if kind == "odd_keys_bool":
        bias = torch.rand(B, 1, L, S, generator=g) < 0.7
        bias[..., 0] = True
    elif kind == "offset_slice":
        bias = torch.randn(1, Hq, L, S + 1, generator=g).to(dtype)[..., 1:]   # rows start at an odd element
    elif kind == "odd_row_stride":
        bias = torch.randn(1, Hq, L, S + 3, generator=g).to(dtype)[..., :S]   # rows are an odd number of elements apart
    else:
        bias = torch.randn(B, Hq, L, S, generator=g).to(dtype)
    bd = bias.to(dev)
    if kind == "offset_slice":
        bd = torch.randn(1, Hq, L, S + 1, device=dev).to(dtype)
        bd[..., 1:] = bias.to(dev)
        bd = bd[..., 1:]
    elif kind == "odd_row_stride":
        bd = torch.zeros(1, Hq, L, S + 3, device=dev, dtype=dtype)
        bd[..., :S] = bias.to(dev)
        bd = bd[..., :S]
    MFMA = amd._lib.KERNEL_MFMA
    qd, kd, vd, god = (t.to(dev) for t in (q, k, v, go))
    want_gb = kind == "odd_keys_grad"
    out, lse = amd.sdpa_forward(qd, kd, vd, attn_bias=bd, force_kernel=MFMA)
    res = amd.sdpa_backward(god, qd, kd, vd, out, lse, attn_bias=bd, want_grad_bias=want_gb, force_kernel=MFMA)
    mask = bias if bias.dtype == torch.bool else bias.float()
    ro, rl = om.sdpa_forward(q.float(), k.float(), v.float(), attn_mask=mask)
    assert max_abs(out, ro) <= 2e-2 and max_abs(lse, rl) <= 5e-3
    rg = om.sdpa_backward(go.float(), q.float(), k.float(), v.float(), ro, rl, attn_mask=mask, reduce_in_fp32=True)
    for a, r in zip(res[:3], rg[:3]):
        assert max_abs(a, r) <= 5e-2 and rel_err(a, r) <= 3e-2
    if want_gb:
        rep = Hq // Hkv
        ke, ve = k.float().repeat_interleave(rep, 1), v.float().repeat_interleave(rep, 1)
        co, cl = om.compute_attention(q.float(), ke, ve, mask, None, E**-0.5, False, 0.0)
        rdb = om.compute_attention_backward(go.float(), q.float(), ke, ve, mask, None, co, cl, E**-0.5, False, 0.0)[3]
        db = res[3]
        assert db.shape == (B, Hq, L, S) and db.is_contiguous()
        assert max_abs(db, rdb) <= 5e-2 and rel_err(db, rdb) <= 2e-2
