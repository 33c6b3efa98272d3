"""GPU parity of the score functors (ALiBi, a captured per-head per-key bias or weight, a tanh soft
cap), document ids and several sink logits against the CPU oracle, forward and backward, through the
C ABI.  They stand in for the score_mod / mask_mod / joint_mod functions the reference renders into
its templated kernels (flex_attention.py.jinja:74-92, flex_attention_bwd.py.jinja:958-988); the cases
are the ones of the reference's own tests
(tests/neuron_dynamo_backend/unit/fx/passes/test_flex_attention_legalization.py:1028-1075, :1200-1235)
plus sizes that reach the tile skipping and the key-block item ranges of the kernels."""

import pytest
import torch

from helpers import max_abs, rel_err, seeded
from oracle import sdpa_math as om

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def amd(gpu_device):
    import torch_neuronx_amd as amd

    return amd


def _functors(pattern, B, Hq, L, S, seed):
    g = torch.Generator().manual_seed(seed)
    slopes = torch.exp2(-(torch.arange(Hq) + 1) * 8.0 / Hq)
    bias = torch.randn(Hq, S, generator=g)
    weight = torch.rand(Hq, S, generator=g) + 0.5
    doc = (torch.arange(max(L, S)) // 96).to(torch.int32)[None].expand(B, -1)
    docs = dict(doc_ids_q=doc[:, :L].contiguous(), doc_ids_k=doc[:, :S].contiguous(), doc_ids_sorted=True)
    return {
        "alibi": dict(is_causal=True, alibi_slopes=slopes),
        "document": dict(**docs),
        "document_unsorted_promise": dict(doc_ids_q=docs["doc_ids_q"], doc_ids_k=docs["doc_ids_k"]),
        "causal_document": dict(is_causal=True, **docs),
        "head_bias": dict(key_bias=bias),
        "head_bias_document": dict(key_bias=bias, **docs),
        "soft_cap": dict(softcap=2.0),
        "weighted": dict(key_weight=weight),
        "window_alibi_cap": dict(is_causal=True, window=64, alibi_slopes=slopes, softcap=3.0),
        # (causal ALiBi walks its key tiles from the diagonal down in the forward: with vectors per key beside it)
        "alibi_key_vectors": dict(is_causal=True, alibi_slopes=slopes, key_bias=bias, key_weight=weight),
        # (... a head with a slope that is not positive walks upwards)
        "alibi_signs": dict(is_causal=True, alibi_slopes=slopes * torch.tensor([1.0, -1.0, 0.0, 1.0]).repeat((Hq + 3) // 4)[:Hq]),
        "everything": dict(is_causal=True, alibi_slopes=slopes, softcap=2.5, key_bias=bias, key_weight=weight,
                           sink_logit=torch.randn(B, Hq, 3, generator=g), **docs),
    }[pattern]


def _check(amd, dev, B, Hq, Hkv, L, S, E, dtype, pattern, seed, force=0, scale=None, Dv=None):
    Dv = Dv or E
    q, k, v, go = seeded([(B, Hq, L, E), (B, Hkv, S, E), (B, Hkv, S, Dv), (B, Hq, L, Dv)], seed, dtype)
    kw = _functors(pattern, B, Hq, L, S, seed + 1)
    dkw = {n: (t.to(dev) if torch.is_tensor(t) else t) for n, t in kw.items()}
    qd, kd, vd, god = (t.to(dev) for t in (q, k, v, go))
    out, lse = amd.sdpa_forward(qd, kd, vd, scale=scale, force_kernel=force, **dkw)
    res = amd.sdpa_backward(god, qd, kd, vd, out, lse, scale=scale, force_kernel=force, **dkw)
    torch.cuda.synchronize()
    okw = {n: t for n, t in kw.items() if n != "doc_ids_sorted"}
    ro, rl = om.sdpa_forward_score_mod(q.float(), k.float(), v.float(), scale=scale, **okw)
    rg = om.sdpa_backward_score_mod(go.float(), q.float(), k.float(), v.float(), ro, rl, scale=scale, **okw)
    half = dtype is not torch.float32
    assert max_abs(out, ro) <= (2e-2 if half else 2e-5), pattern
    assert max_abs(lse, rl) <= (5e-3 if half else 2e-5), pattern
    for name, a, r in zip(("dq", "dk", "dv"), res[:3], rg[:3]):
        assert a.shape == r.shape
        assert max_abs(a, r) <= (5e-2 if half else 1e-4) * max(1.0, r.abs().max().item()), (pattern, name)
        assert rel_err(a, r) <= (3e-2 if half else 2e-5), (pattern, name)
    if "sink_logit" in kw:
        assert res[4].shape == kw["sink_logit"].shape
        assert max_abs(res[4], rg[3]) <= (5e-2 if half else 1e-4) and rel_err(res[4], rg[3]) <= (3e-2 if half else 2e-5)
    return out, lse, res


PATTERNS = ["alibi", "document", "document_unsorted_promise", "causal_document", "head_bias", "head_bias_document",
            "soft_cap", "weighted", "window_alibi_cap", "alibi_key_vectors", "alibi_signs", "everything"]


@pytest.mark.parametrize("pattern", PATTERNS)
@pytest.mark.parametrize("L", [128, 256])
def test_reference_cases_float32(amd, gpu_device, pattern, L):
    # B=1, Hq=4, Hkv=2, E=16, documents of 96 ids: the shapes of the reference's tests, in their dtype
    _check(amd, gpu_device, 1, 4, 2, L, L, 16, torch.float32, pattern, seed=L + len(pattern))


@pytest.mark.parametrize("pattern", PATTERNS)
@pytest.mark.parametrize("B,Hq,Hkv,L,S,E", [(1, 4, 2, 256, 256, 16), (2, 4, 1, 300, 500, 96), (1, 2, 2, 200, 200, 128),
                                            (1, 2, 1, 160, 200, 256)])  # (... and the width-256 instances)
def test_float32_in_the_matrix_op_kernels(amd, gpu_device, pattern, B, Hq, Hkv, L, S, E):
    # float32 inputs on the float32 matrix op, forced (the call fails if those kernels refuse it)
    _check(amd, gpu_device, B, Hq, Hkv, L, S, E, torch.float32, pattern, seed=L + E, force=amd._lib.KERNEL_MFMA)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("pattern", PATTERNS)
def test_reference_cases_in_the_matrix_op_kernels(amd, gpu_device, dtype, pattern):
    # the same cases in 16-bit inputs, forced into the matrix-op kernels (the call fails if they refuse it)
    _check(amd, gpu_device, 1, 4, 2, 256, 256, 16, dtype, pattern, seed=7, force=amd._lib.KERNEL_MFMA)


@pytest.mark.parametrize("pattern", PATTERNS)
@pytest.mark.parametrize("B,Hq,Hkv,L,S,E", [
    (2, 8, 2, 1024, 1024, 128),   # several 256-row workgroups and key blocks per head: tile ranges, item ranges
    (1, 4, 4, 777, 777, 64),      # ragged last tiles
    (2, 4, 1, 300, 500, 96),      # L != S, padded head dim, one kv head
])
def test_functor_kernels_at_size(amd, gpu_device, pattern, B, Hq, Hkv, L, S, E):
    _check(amd, gpu_device, B, Hq, Hkv, L, S, E, torch.bfloat16, pattern, seed=L + S, force=amd._lib.KERNEL_MFMA)


@pytest.mark.parametrize("pattern", PATTERNS)
@pytest.mark.parametrize("B,Hq,Hkv,L,S,E,Dv", [
    (1, 4, 2, 512, 512, 256, 256),   # head dim 256 (one wavefront per SIMD in every kernel)
    (2, 4, 1, 300, 500, 192, 128),   # D_qk != D_v, L != S, ragged tiles
    (1, 2, 2, 777, 777, 160, 160),   # a head dim between 128 and 256
])
def test_functor_kernels_at_wide_head_dims(amd, gpu_device, pattern, B, Hq, Hkv, L, S, E, Dv):
    # head dims above 128 and D_qk != D_v: the forward's functor variant at width 256 and the wide backward
    # kernels' functor mode, forced (the call fails if the matrix-op kernels refuse it)
    _check(amd, gpu_device, B, Hq, Hkv, L, S, E, torch.bfloat16, pattern, seed=L + E, force=amd._lib.KERNEL_MFMA, Dv=Dv)


def test_document_ids_equal_the_same_mask_as_a_tensor(amd, gpu_device):
    # document ids (sorted, with tile skipping) against the explicit boolean mask of the same pattern
    dev = gpu_device
    B, Hq, Hkv, L, E = 2, 8, 2, 2048, 128
    q, k, v = (t.to(dev) for t in seeded([(B, Hq, L, E), (B, Hkv, L, E), (B, Hkv, L, E)], 3, torch.bfloat16))
    cuts = torch.tensor([[0, 300, 301, 1500, 2048], [0, 64, 1024, 1030, 2048]])
    doc = torch.stack([torch.bucketize(torch.arange(L), c[1:-1], right=True) for c in cuts]).to(torch.int32)
    a, la = amd.sdpa_forward(q, k, v, is_causal=True, doc_ids_q=doc.to(dev), doc_ids_k=doc.to(dev), doc_ids_sorted=True)
    keep = (doc[:, :, None] == doc[:, None, :]) & torch.ones(L, L, dtype=torch.bool).tril()
    b, lb = amd.sdpa_forward(q, k, v, attn_bias=keep[:, None].to(dev))
    assert max_abs(a, b) <= 4e-3 and max_abs(la, lb) <= 1e-4
    # rows whose document holds no key at all (ids that never meet): zeros and lse = -inf
    dq_ = doc.clone()
    dq_[0, :100] = -5
    c, lc = amd.sdpa_forward(q, k, v, doc_ids_q=dq_.to(dev), doc_ids_k=doc.to(dev))
    assert torch.all(c[0, :, :100] == 0) and torch.all(lc[0, :, :100] == float("-inf"))


def test_long_sequence_document_packing(amd, gpu_device):
    # one S = 4096, D = 128 case: 8 documents of 512, causal, head subset against the oracle
    dev = gpu_device
    B, Hq, Hkv, L, E = 1, 8, 2, 4096, 128
    q, k, v, go = seeded([(B, Hq, L, E), (B, Hkv, L, E), (B, Hkv, L, E), (B, Hq, L, E)], 11, torch.bfloat16)
    doc = (torch.arange(L) // 512).to(torch.int32)[None]
    slopes = torch.exp2(-(torch.arange(Hq) + 1) * 8.0 / Hq)
    kw = dict(is_causal=True, doc_ids_q=doc.to(dev), doc_ids_k=doc.to(dev), doc_ids_sorted=True, alibi_slopes=slopes.to(dev))
    qd, kd, vd, god = (t.to(dev) for t in (q, k, v, go))
    out, lse = amd.sdpa_forward(qd, kd, vd, **kw)
    dq, dk, dv, _ = amd.sdpa_backward(god, qd, kd, vd, out, lse, **kw)
    hs, hk = slice(0, 4), slice(0, 1)  # the first kv head and its four query heads
    ro, rl = om.sdpa_forward_score_mod(q[:, hs].float(), k[:, hk].float(), v[:, hk].float(), is_causal=True, doc_ids_q=doc,
                                       doc_ids_k=doc, alibi_slopes=slopes[hs])
    rdq, rdk, rdv, _ = om.sdpa_backward_score_mod(go[:, hs].float(), q[:, hs].float(), k[:, hk].float(), v[:, hk].float(), ro, rl,
                                                  is_causal=True, doc_ids_q=doc, doc_ids_k=doc, alibi_slopes=slopes[hs])
    assert max_abs(out[:, hs], ro) <= 2e-2 and max_abs(lse[:, hs], rl) <= 5e-3
    assert rel_err(dq[:, hs], rdq) <= 3e-2 and rel_err(dk[:, hk], rdk) <= 3e-2 and rel_err(dv[:, hk], rdv) <= 3e-2


def test_score_functor_argument_errors(amd, gpu_device):
    dev = gpu_device
    q, k, v = (t.to(dev) for t in seeded([(1, 2, 64, 64)] * 3, 1, torch.bfloat16))
    with pytest.raises(ValueError, match="come together"):
        amd.sdpa_forward(q, k, v, doc_ids_q=torch.zeros(1, 64, dtype=torch.int32))
    with pytest.raises(ValueError, match="alibi_slopes must have shape"):
        amd.sdpa_forward(q, k, v, alibi_slopes=torch.zeros(3))
    with pytest.raises(RuntimeError, match="softcap"):
        amd.sdpa_forward(q, k, v, softcap=-1.0, alibi_slopes=torch.zeros(2))
    # a functor together with a bias has no matrix-op kernel: forced there, the call says so
    with pytest.raises(RuntimeError, match="functor"):
        amd.sdpa_forward(q, k, v, softcap=2.0, attn_bias=torch.zeros(1, 1, 64, 64, device=dev, dtype=torch.bfloat16),
                         force_kernel=amd._lib.KERNEL_MFMA)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_prefix_length_mask_mod_is_a_key_count(amd, gpu_device, dtype):
    # the reference's mask_mod with an external buffer (test_flex_attention_legalization.py:783-800):
    # kv_idx <= prefix_length[b], a per-batch prefix of the keys - here the call's kv_lens = prefix_length + 1,
    # which the matrix-op kernels take without a mask tensor (tiles past the prefix are never read)
    dev = gpu_device
    B, H, L, S, E = 2, 2, 8, 8, 16
    q, k, v, go = seeded([(B, H, L, E), (B, H, S, E), (B, H, S, E), (B, H, L, E)], 5, dtype)
    prefix_length = torch.tensor([4, 6], dtype=torch.int32)
    keep = (torch.arange(S)[None] <= prefix_length[:, None])[:, None, None, :]
    lens = (prefix_length + 1).to(dev)
    MFMA = amd._lib.KERNEL_MFMA
    out, lse = amd.sdpa_forward(q.to(dev), k.to(dev), v.to(dev), kv_lens=lens, force_kernel=MFMA)
    dq, dk, dv, _ = amd.sdpa_backward(go.to(dev), q.to(dev), k.to(dev), v.to(dev), out, lse, kv_lens=lens, force_kernel=MFMA)
    ro, rl = om.sdpa_forward(q.float(), k.float(), v.float(), attn_mask=keep)
    rg = om.sdpa_backward(go.float(), q.float(), k.float(), v.float(), ro, rl, attn_mask=keep, reduce_in_fp32=True)
    half = dtype is not torch.float32
    assert max_abs(out, ro) <= (2e-2 if half else 1e-5) and max_abs(lse, rl) <= (5e-3 if half else 1e-5)
    for a, r in zip((dq, dk, dv), rg):
        assert max_abs(a, r) <= (5e-2 if half else 1e-5)
    # ... and the same mask as a tensor is recognised as that key count by the operator
    fused = torch.ops.aten._scaled_dot_product_fused_attention_overrideable
    mask = keep.expand(B, 1, L, S).contiguous().to(dev)
    amd.mask_patterns.clear_cache()
    fused(q.to(dev), k.to(dev), v.to(dev), mask)
    torch.cuda.synchronize()
    pat = amd.mask_patterns.classify(mask)
    assert pat[0] == "all" and pat[1].tolist() == [5, 7]
    r = fused(q.to(dev), k.to(dev), v.to(dev), mask)
    assert max_abs(r[0], ro) <= (2e-2 if half else 1e-5)
