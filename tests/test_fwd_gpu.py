"""GPU parity of the forward kernels against the CPU oracle, through the C ABI."""

import math

import pytest
import torch

from helpers import max_abs, oracle_fwd, qkv, rel_err, tol_for

pytestmark = pytest.mark.gpu

GENERIC, MFMA = 1, 2


@pytest.fixture(scope="module")
def amd(gpu_device):
    import torch_neuronx_amd as amd

    return amd


def _run(amd, q, k, v, dev, **kw):
    out, lse = amd.sdpa_forward(q.to(dev), k.to(dev), v.to(dev), **kw)
    torch.cuda.synchronize()
    return out, lse


def test_config1_fp32_noncausal_mha(amd, gpu_device):
    # benchmark configuration 1: B=2,H=4,S=128,D=64 fp32, scale 1/8, max-abs <= 1e-5
    q, k, v = qkv(2, 4, 4, 128, 128, 64, dtype=torch.float32, seed=1001)
    out, lse = _run(amd, q, k, v, gpu_device, scale=0.125)
    ro, rl = oracle_fwd(q, k, v, scale=0.125)
    assert max_abs(out, ro) <= 1e-5
    assert max_abs(lse, rl) <= 1e-5
    assert out.dtype == torch.float32 and lse.dtype == torch.float32 and lse.shape == (2, 4, 128)


def test_config2_bf16_causal_mha(amd, gpu_device):
    # benchmark configuration 2: B=4,H=12,S=1024,D=64 bf16 causal; output within 2e-2 of the fp32 oracle
    q, k, v = qkv(4, 12, 12, 1024, 1024, 64, dtype=torch.bfloat16, seed=1002)
    out, lse = _run(amd, q, k, v, gpu_device, is_causal=True, scale=0.125, force_kernel=MFMA)
    ro, rl = oracle_fwd(q, k, v, is_causal=True, scale=0.125)
    assert out.dtype == torch.bfloat16
    assert max_abs(out, ro) <= 2e-2
    assert max_abs(lse, rl) <= 1e-3


def test_config3_llama8b_shape_head_subset(amd, gpu_device):
    # benchmark configuration 3 at full size on the GPU; the oracle checks a subset of heads
    # (first/last of a group, first/last kv head) to stay within seconds on the CPU.
    q, k, v = qkv(1, 32, 8, 8192, 8192, 128, dtype=torch.bfloat16, seed=1003)
    out, lse = _run(amd, q, k, v, gpu_device, is_causal=True, force_kernel=MFMA)
    assert lse.shape == (1, 32, 8192) and lse.dtype == torch.float32
    for h in (0, 3, 13, 31):
        hk = h // 4
        ro, rl = oracle_fwd(q[:, h : h + 1], k[:, hk : hk + 1], v[:, hk : hk + 1], is_causal=True)
        assert max_abs(out[:, h : h + 1], ro) <= 2e-2, f"head {h}"
        assert max_abs(lse[:, h : h + 1], rl) <= 2e-3, f"head {h}"
    # size-independent property: under a causal mask row 0 attends to key 0 only
    torch.testing.assert_close(out[0, :, 0].float().cpu(), v[0].repeat_interleave(4, 0)[:, 0].float(), rtol=0, atol=0)
    s00 = (q[0, :, 0].float() * k[0].repeat_interleave(4, 0)[:, 0].float()).sum(-1) / math.sqrt(128)
    assert max_abs(lse[0, :, 0], s00) <= 1e-4


SHAPES = [
    # B, Hq, Hkv, L, S, E, causal   (reference parity matrix + edge cases)
    (1, 8, 8, 512, 512, 64, False),
    (1, 24, 6, 512, 512, 64, False),
    (1, 8, 1, 512, 512, 64, False),
    (1, 4, 2, 512, 512, 64, True),
    (1, 2, 1, 577, 577, 64, False),
    (1, 2, 1, 577, 577, 64, True),
    (2, 4, 4, 51, 51, 64, True),
    (2, 4, 2, 13, 51, 128, True),
    (2, 4, 2, 51, 13, 128, True),
    (1, 4, 4, 128, 1024, 128, False),
    (1, 4, 1, 200, 333, 128, True),
    (2, 8, 2, 1, 257, 128, False),
    (1, 8, 8, 2048, 2048, 128, True),
]


@pytest.mark.parametrize("shape", SHAPES)
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("tile", [3, 4])  # 128 / 256 query rows per workgroup
def test_mfma_forward_matrix(amd, gpu_device, shape, dtype, tile):
    B, Hq, Hkv, L, S, E, causal = shape
    q, k, v = qkv(B, Hq, Hkv, L, S, E, dtype=dtype, seed=L * 7 + S)
    out, lse = _run(amd, q, k, v, gpu_device, is_causal=causal, force_kernel=tile)
    ro, rl = oracle_fwd(q, k, v, is_causal=causal)
    assert max_abs(out, ro) <= 2e-2
    assert rel_err(out, ro) <= 1e-2
    assert max_abs(lse, rl) <= 2e-3


def test_mfma_forward_rows_far_apart(amd, gpu_device):
    # key / value rows 512 KiB apart: one (batch, head) spans 2 GiB, beyond the 32-bit row
    # addressing of the head-dim-128 kernels, so the call is served by the 64-bit-address kernel
    B, Hq, Hkv, L, S, E = 1, 2, 1, 160, 4096, 128
    q, k, v = qkv(B, Hq, Hkv, L, S, E, dtype=torch.bfloat16, seed=77)
    pitch = 262144
    assert S * pitch * 2 >= 2**31
    kd = torch.empty(B, Hkv, S, pitch, dtype=torch.bfloat16, device=gpu_device)[..., :E]
    vd = torch.empty(B, Hkv, S, pitch, dtype=torch.bfloat16, device=gpu_device)[..., :E]
    kd.copy_(k)
    vd.copy_(v)
    out, lse = amd.sdpa_forward(q.to(gpu_device), kd, vd, is_causal=False, force_kernel=MFMA)
    torch.cuda.synchronize()
    ro, rl = oracle_fwd(q, k, v)
    assert max_abs(out, ro) <= 2e-2
    assert max_abs(lse, rl) <= 2e-3


GENERIC_SHAPES = SHAPES[:9] + [
    (1, 4, 4, 256, 256, 256, False),
    (1, 4, 2, 512, 512, 256, True),
    (2, 8, 1, 12, 12, 16, False),
    (2, 8, 2, 10, 10, 16, True),
    (1, 4, 4, 6, 6, 12, False),
    (1, 2, 2, 6, 10, 40, False),
]


@pytest.mark.parametrize("shape", GENERIC_SHAPES)
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16])
def test_generic_forward_matrix(amd, gpu_device, shape, dtype):
    B, Hq, Hkv, L, S, E, causal = shape
    q, k, v = qkv(B, Hq, Hkv, L, S, E, dtype=dtype, seed=L * 5 + S)
    out, lse = _run(amd, q, k, v, gpu_device, is_causal=causal, force_kernel=GENERIC)
    ro, rl = oracle_fwd(q, k, v, is_causal=causal)
    assert max_abs(out, ro) <= tol_for(dtype)
    assert max_abs(lse, rl) <= (2e-5 if dtype is torch.float32 else 2e-3)


def test_asymmetric_head_dims_generic(amd, gpu_device):
    # reference: D_qk=192, D_v=128 (MLA-style)
    q, k, v = qkv(1, 4, 2, 96, 96, 192, Dv=128, dtype=torch.float32, seed=5)
    out, lse = _run(amd, q, k, v, gpu_device, is_causal=True)
    ro, rl = oracle_fwd(q, k, v, is_causal=True)
    assert out.shape == (1, 4, 96, 128)
    assert max_abs(out, ro) <= 1e-5 and max_abs(lse, rl) <= 1e-5


@pytest.mark.parametrize("mask_kind", ["float", "bool", "bool_bcast", "float_bcast"])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_masks_and_bias(amd, gpu_device, mask_kind, dtype):
    B, H, L, S, E = 2, 4, 51, 77, 48
    q, k, v = qkv(B, H, H, L, S, E, dtype=dtype, seed=77)
    g = torch.Generator().manual_seed(3)
    if mask_kind == "float":
        mask = torch.randn(B, H, L, S, generator=g).to(dtype)
    elif mask_kind == "float_bcast":
        mask = torch.randn(1, 1, L, S, generator=g).to(dtype)
    elif mask_kind == "bool":
        mask = torch.rand(B, H, L, S, generator=g) > 0.3
    else:
        mask = (torch.rand(B, 1, 1, S, generator=g) > 0.3)
    out, lse = _run(amd, q, k, v, gpu_device, attn_bias=mask.to(gpu_device))
    ro, rl = oracle_fwd(q, k, v, attn_mask=mask if mask.dtype == torch.bool else mask.float())
    assert max_abs(out, ro) <= tol_for(dtype)
    assert max_abs(lse, rl) <= (2e-5 if dtype is torch.float32 else 2e-3)


MASKED_MFMA_CASES = [
    # B, Hq, Hkv, L, S, mask kind, causal
    (2, 4, 2, 96, 160, "float_same", False),
    (2, 4, 2, 96, 160, "float32", False),
    (2, 4, 4, 130, 76, "float_bcast_q", False),     # (B,1,1,S): one bias row for every query
    (1, 8, 2, 300, 512, "float_bcast_bh", True),    # (1,1,L,S) together with the causal mask
    (2, 4, 2, 96, 160, "bool", False),
    (3, 4, 1, 70, 132, "bool_padding", False),      # (B,1,1,S) key-padding mask
    (1, 4, 4, 257, 1024, "bool_rows_dead", False),  # some query rows see no key at all
    (2, 8, 2, 512, 2048, "float_same", True),
]


@pytest.mark.parametrize("case", MASKED_MFMA_CASES)
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("tile", [3, 4])
def test_mfma_forward_with_bias_and_masks(amd, gpu_device, case, dtype, tile):
    # additive bias / bool keep-mask inside the head-dim-128 MFMA kernels (forced: a call they
    # cannot take is an error, not a fallback)
    B, Hq, Hkv, L, S, kind, causal = case
    q, k, v = qkv(B, Hq, Hkv, L, S, 128, dtype=dtype, seed=L + 3 * S)
    g = torch.Generator().manual_seed(L * 31 + S)
    if kind == "float_same":
        mask = (2.0 * torch.randn(B, Hq, L, S, generator=g)).to(dtype)
    elif kind == "float32":
        mask = 2.0 * torch.randn(B, Hq, L, S, generator=g)
    elif kind == "float_bcast_q":
        mask = (2.0 * torch.randn(B, 1, 1, S, generator=g)).to(dtype)
    elif kind == "float_bcast_bh":
        mask = (2.0 * torch.randn(1, 1, L, S, generator=g)).to(dtype)
    elif kind == "bool":
        mask = torch.rand(B, Hq, L, S, generator=g) > 0.3
    elif kind == "bool_padding":
        lens = torch.tensor([S, 5, 67])[:B]
        mask = (torch.arange(S)[None, :] < lens[:, None])[:, None, None, :]
    else:
        mask = torch.rand(B, 1, L, S, generator=g) > 0.5
        mask[:, :, 3:40] = False
        mask[:, :, L - 1] = False
    out, lse = _run(amd, q, k, v, gpu_device, attn_bias=mask.to(gpu_device), is_causal=causal, force_kernel=tile)
    ro, rl = oracle_fwd(q, k, v, attn_mask=mask if mask.dtype == torch.bool else mask.float(), is_causal=causal)
    assert max_abs(out, ro) <= 2e-2
    assert rel_err(out, ro) <= 1e-2
    assert max_abs(lse, rl) <= 3e-3
    if kind == "bool_rows_dead":
        assert torch.equal(out[:, :, 3:40].float().cpu(), torch.zeros(B, Hq, 37, 128))
        assert torch.isinf(lse[:, :, 3:40]).all() and (lse[:, :, 3:40] < 0).all()


@pytest.mark.parametrize("kind", ["window", "left_padding", "late_and_low", "late_and_high"])
@pytest.mark.parametrize("D", [64, 128])
@pytest.mark.parametrize("tile", [3, 4])
def test_mfma_forward_rows_whose_first_keys_are_masked(amd, gpu_device, kind, D, tile):
    # The MFMA forward takes a row's softmax reference from its first key tile.  Rows whose first
    # tiles are fully masked have none until a live key arrives; what arrives may lie far below or
    # far above zero in the exponent.
    B, Hq, Hkv, L, S = 2, 4, 2, 200, 328
    q, k, v = qkv(B, Hq, Hkv, L, S, D, dtype=torch.bfloat16, seed=D + 5)
    i, j = torch.arange(L)[:, None], torch.arange(S)[None, :]
    if kind == "window":
        mask = (j <= i + 40) & (j >= i - 23)  # sliding window: row i starts at key i - 23
    elif kind == "left_padding":
        start = torch.tensor([0, 150])[:B]
        mask = (j[None] >= start[:, None, None])[:, None].expand(B, 1, L, S)
    else:
        # keys 0..99 masked, the live ones carry a bias of -200 / +60 (log2 domain: -288 / +87):
        # probabilities against a reference of 0 would underflow / overflow
        mask = torch.full((1, 1, L, S), float("-inf"))
        mask[..., 100:] = -200.0 if kind == "late_and_low" else 60.0
        mask[..., 100:] += torch.randn(L, S - 100, generator=torch.Generator().manual_seed(3))
    out, lse = _run(amd, q, k, v, gpu_device, attn_bias=mask.to(gpu_device), force_kernel=tile)
    ro, rl = oracle_fwd(q, k, v, attn_mask=mask if mask.dtype == torch.bool else mask.float())
    assert torch.isfinite(lse).all()
    assert max_abs(out, ro) <= 2e-2
    assert rel_err(out, ro) <= 1e-2
    assert max_abs(lse, rl) <= 3e-3


@pytest.mark.parametrize("kind", ["float", "bool", "kv_lens"])
@pytest.mark.parametrize("tile", [3, 4])
def test_mfma_forward_masked_head_dim_64(amd, gpu_device, kind, tile):
    B, Hq, Hkv, L, S = 2, 6, 3, 150, 264
    q, k, v = qkv(B, Hq, Hkv, L, S, 64, dtype=torch.bfloat16, seed=64)
    g = torch.Generator().manual_seed(640)
    kw, mask = {}, None
    if kind == "float":
        mask = (2.0 * torch.randn(B, 1, L, S, generator=g)).to(torch.bfloat16)
        kw["attn_bias"] = mask.to(gpu_device)
    elif kind == "bool":
        mask = torch.rand(1, Hq, L, S, generator=g) > 0.4
        kw["attn_bias"] = mask.to(gpu_device)
    else:
        lens = torch.tensor([77, 264], dtype=torch.int32)
        mask = (torch.arange(S)[None, :] < lens[:, None])[:, None, None, :]
        kw["kv_lens"] = lens.to(gpu_device)
    out, lse = _run(amd, q, k, v, gpu_device, force_kernel=tile, **kw)
    ro, rl = oracle_fwd(q, k, v, attn_mask=mask if mask.dtype == torch.bool else mask.float())
    assert max_abs(out, ro) <= 2e-2 and rel_err(out, ro) <= 1e-2 and max_abs(lse, rl) <= 3e-3


@pytest.mark.parametrize("tile", [3, 4])
def test_mfma_forward_with_kv_lens(amd, gpu_device, tile):
    # per-batch key counts inside the MFMA kernels, including an empty and a one-key batch; the
    # rows of the cache past a batch's count hold NaN and must never reach the output
    B, Hq, Hkv, L, S = 4, 8, 2, 200, 640
    q, k, v = qkv(B, Hq, Hkv, L, S, 128, dtype=torch.bfloat16, seed=41)
    lens = torch.tensor([640, 0, 1, 333], dtype=torch.int32)
    kd, vd = k.clone(), v.clone()
    for bi in range(B):
        kd[bi, :, int(lens[bi]):] = float("nan")
        vd[bi, :, int(lens[bi]):] = float("nan")
    out, lse = _run(amd, q, kd, vd, gpu_device, kv_lens=lens.to(gpu_device), force_kernel=tile)
    pad = (torch.arange(S)[None, :] < lens[:, None])[:, None, None, :]
    ro, rl = oracle_fwd(q, k, v, attn_mask=pad)
    assert torch.isfinite(out.float()).all()
    assert max_abs(out, ro) <= 2e-2 and max_abs(lse, rl) <= 3e-3
    assert torch.equal(out[1].float().cpu(), torch.zeros(Hq, L, 128))
    assert torch.isinf(lse[1]).all() and (lse[1] < 0).all()


def test_fully_masked_rows_give_zero_and_minus_inf(amd, gpu_device):
    # reference: tests/python_ops/test_scaled_dot_product_attention.py:1003-1064
    q, k, v = qkv(1, 4, 4, 32, 32, 32, dtype=torch.float32, seed=9)
    mask = torch.ones(1, 1, 32, 32, dtype=torch.bool)
    mask[:, :, :10, :] = False
    out, lse = _run(amd, q, k, v, gpu_device, attn_bias=mask.to(gpu_device))
    assert torch.equal(out[:, :, :10].cpu(), torch.zeros(1, 4, 10, 32))
    assert torch.isinf(lse[:, :, :10]).all() and (lse[:, :, :10] < 0).all()
    ro, rl = oracle_fwd(q, k, v, attn_mask=mask)
    assert max_abs(out, ro) <= 1e-5 and max_abs(lse, rl) <= 1e-5


def test_kv_lens_equals_key_padding_mask(amd, gpu_device):
    q, k, v = qkv(3, 4, 2, 5, 64, 32, dtype=torch.float32, seed=4)
    lens = torch.tensor([64, 1, 17], dtype=torch.int32)
    out, lse = _run(amd, q, k, v, gpu_device, kv_lens=lens.to(gpu_device))
    pad = (torch.arange(64)[None, :] < lens[:, None])[:, None, None, :]
    ro, rl = oracle_fwd(q, k, v, attn_mask=pad)
    assert max_abs(out, ro) <= 1e-5 and max_abs(lse, rl) <= 1e-5


@pytest.mark.parametrize("tile", [3, 4])
@pytest.mark.parametrize("per_head", [False, True])
def test_mfma_forward_padding_masks_with_holes_and_dead_batches(amd, gpu_device, tile, per_head):
    # per-key keep-masks (no row stride): the kernel stops at the last kept key of a (batch, head),
    # skips nothing in front of it, and a row of the mask that keeps no key gives zeros and lse = -inf
    B, Hq, Hkv, L, S = 4, 4, 2, 200, 328
    q, k, v = qkv(B, Hq, Hkv, L, S, 128, dtype=torch.bfloat16, seed=77)
    g = torch.Generator().manual_seed(5)
    mask = torch.zeros(B, Hq if per_head else 1, 1, S, dtype=torch.bool)
    mask[0, :, :, :S] = True                      # keeps every key
    mask[1, :, :, 40:133] = True                  # left and right padding
    mask[1, :, :, 64:96] = False                  # ... with a whole tile dropped in the middle
    mask[2] = torch.rand(mask[2].shape, generator=g) > 0.5
    mask[2, :, :, 300:] = False                   # ragged end inside a tile
    # batch 3 keeps nothing
    if per_head: mask[0, 1, :, 7:] = False        # heads of a batch differ
    out, lse = _run(amd, q, k, v, gpu_device, attn_bias=mask.to(gpu_device), force_kernel=tile)
    ro, rl = oracle_fwd(q, k, v, attn_mask=mask)
    assert torch.equal(out[3].cpu().float(), torch.zeros(Hq, L, 128))
    assert torch.isinf(lse[3]).all() and (lse[3] < 0).all()
    assert max_abs(out, ro) <= 2e-2
    assert max_abs(lse[:3], rl[:3]) <= 2e-3


def test_scale_zero_and_explicit_scale(amd, gpu_device):
    q, k, v = qkv(1, 2, 2, 40, 40, 64, dtype=torch.bfloat16, seed=8)
    for sc in (0.0, 0.25, 0.5):
        out, lse = _run(amd, q, k, v, gpu_device, scale=sc)
        ro, rl = oracle_fwd(q, k, v, scale=sc)
        assert max_abs(out, ro) <= 2e-2 and max_abs(lse, rl) <= 2e-3


@pytest.mark.parametrize("kernel", [GENERIC, 3, 4])
def test_noncontiguous_inputs_keep_query_layout(amd, gpu_device, kernel):
    # reference: test_scaled_dot_product_attention.py:943-1000 - (B,L,H,D).transpose(1,2) views,
    # last-dim chunks of a fused QKV buffer, as_strided with gaps
    B, H, L, E = 2, 4, 130, 64
    g = torch.Generator().manual_seed(21)
    base = torch.randn(B, L, H, 3 * E, generator=g).to(torch.bfloat16).to(gpu_device)
    q, k, v = (t.transpose(1, 2) for t in base.chunk(3, dim=-1))
    assert not q.is_contiguous()
    out, lse = amd.sdpa_forward(q, k, v, is_causal=True, force_kernel=kernel)
    ro, rl = oracle_fwd(q.cpu(), k.cpu(), v.cpu(), is_causal=True)
    assert max_abs(out, ro) <= 2e-2
    expect = torch.empty(B, L, H, E).transpose(1, 2).stride()
    assert out.stride() == expect
    assert lse.is_contiguous()


def test_expanded_kv_stride0(amd, gpu_device):
    # reference: test_scaled_dot_product_attention.py:1123-1221 (repeat_kv style expand)
    q, k, v = qkv(1, 8, 1, 512, 512, 64, dtype=torch.bfloat16, seed=12)
    ke = k.to(gpu_device).expand(1, 8, 512, 64)
    ve = v.to(gpu_device).expand(1, 8, 512, 64)
    out, lse = amd.sdpa_forward(q.to(gpu_device), ke, ve, is_causal=True)
    ro, rl = oracle_fwd(q, k, v, is_causal=True)
    assert max_abs(out, ro) <= 2e-2


@pytest.mark.parametrize("tile", [3, 4])
@pytest.mark.parametrize("causal", [False, True])
@pytest.mark.parametrize("kind", ["rising", "falling", "spiky", "huge"])
def test_softmax_reference_tracking_under_stress(amd, gpu_device, kind, causal, tile):
    """Logit profiles that make the running softmax reference move often, rarely, or violently.

    The long-sequence forward kernel keeps no row maximum in its fast path: it raises its
    reference only when a tile's probability sums run away.  Rising logits trigger that again and
    again, falling logits never after the first tile, spikes arrive in the middle of a row, and
    'huge' logits overflow exp2 against a stale reference.  All must match the oracle.
    """
    B, Hq, Hkv, L, S, E = 1, 2, 1, 256, 1024, 128
    g = torch.Generator().manual_seed({"rising": 1, "falling": 2, "spiky": 3, "huge": 4}[kind])
    q = torch.randn(B, Hq, L, E, generator=g)
    k = torch.randn(B, Hkv, S, E, generator=g)
    v = torch.randn(B, Hkv, S, E, generator=g)
    u = torch.nn.functional.normalize(torch.randn(E, generator=g), dim=0)
    q = q + 6.0 * u  # every query has a strong component along u ...
    ramp = torch.linspace(-1.0, 1.0, S)
    if kind == "rising":
        k = k + (9.0 * ramp)[None, None, :, None] * u  # ... so the logit grows with the key index
    elif kind == "falling":
        k = k - (9.0 * ramp)[None, None, :, None] * u
    elif kind == "spiky":
        spikes = torch.zeros(S)
        spikes[torch.tensor([37, 300, 301, 640, 1001])] = torch.tensor([4.0, 9.0, 9.5, 14.0, 20.0])
        k = k + spikes[None, None, :, None] * u
    else:
        k = k + (60.0 * ramp)[None, None, :, None] * u  # logits of several hundred: exp2 overflows without care
    q, k, v = q.to(torch.bfloat16), k.to(torch.bfloat16), v.to(torch.bfloat16)
    out, lse = _run(amd, q, k, v, gpu_device, is_causal=causal, force_kernel=tile)
    ro, rl = oracle_fwd(q, k, v, is_causal=causal)
    assert torch.isfinite(out.float()).all() and torch.isfinite(lse).all()
    assert max_abs(out, ro) <= 2e-2  # bf16 output tolerance of the path
    assert max_abs(lse, rl) <= 2e-3 * max(1.0, rl.abs().max().item())


@pytest.mark.parametrize("E", [8, 32, 40, 56, 72, 80, 96, 112, 120, 136, 160, 192, 248, 256])
@pytest.mark.parametrize("variant", ["plain", "causal_gqa", "bias"])
def test_mfma_forward_narrow_head_dims(amd, gpu_device, E, variant):
    # head dims below 64 / 128 / 256 (multiples of 8) run in the next wider MFMA kernel, the tail of every
    # row counting as zeros; the tensors are slices of wider ones whose tails hold NaN, so a read
    # past a row's end would show
    B, Hq, Hkv, L, S = (2, 4, 4, 150, 264) if variant != "causal_gqa" else (2, 8, 2, 200, 200)
    q, k, v = qkv(B, Hq, Hkv, L, S, E, dtype=torch.bfloat16, seed=E)
    dev = gpu_device

    def wide(t):
        w = torch.full(t.shape[:-1] + (E + 8,), float("nan"), dtype=t.dtype, device=dev)
        w[..., :E] = t.to(dev)
        return w[..., :E]

    kw = {}
    mask = None
    if variant == "bias":
        mask = (2.0 * torch.randn(1, Hq, L, S, generator=torch.Generator().manual_seed(E))).to(torch.bfloat16)
        kw["attn_bias"] = mask.to(dev)
    causal = variant == "causal_gqa"
    for tile in (3, 4):
        out, lse = amd.sdpa_forward(wide(q), wide(k), wide(v), is_causal=causal, force_kernel=tile, **kw)
        assert out.shape == (B, Hq, L, E)
        ro, rl = oracle_fwd(q, k, v, attn_mask=None if mask is None else mask.float(), is_causal=causal)
        assert torch.isfinite(out.float()).all()
        assert max_abs(out, ro) <= 2e-2
        assert rel_err(out, ro) <= 1e-2
        assert max_abs(lse, rl) <= 3e-3


@pytest.mark.parametrize("E,Dv", [(192, 128), (128, 64), (96, 64), (256, 128), (64, 32)])
@pytest.mark.parametrize("causal", [False, True])
def test_mfma_forward_value_rows_narrower_than_keys(amd, gpu_device, E, Dv, causal):
    # D_qk > D_v (multi-head latent attention: 192 / 128, reference gate cases
    # tests/neuron_dynamo_backend/unit/test_sdpa_nki_gates.py:52-56) inside the MFMA forward kernel
    B, Hq, Hkv, L, S = 2, 8, 2, 200, 264
    q, k, v = qkv(B, Hq, Hkv, L, S, E, Dv=Dv, dtype=torch.bfloat16, seed=E + Dv)
    out, lse = _run(amd, q, k, v, gpu_device, is_causal=causal, force_kernel=MFMA)
    assert out.shape == (B, Hq, L, Dv)
    ro, rl = oracle_fwd(q, k, v, is_causal=causal)
    assert max_abs(out, ro) <= 2e-2
    assert rel_err(out, ro) <= 1e-2
    assert max_abs(lse, rl) <= 3e-3


# ---- short query sequences under grouped-query attention: the heads of a kv group share a workgroup ----
GROUPED = [
    # B, Hq, Hkv, L, S, D, causal, kv_lens
    (3, 8, 2, 1, 704, 128, False, None),     # a decode step, 4 heads per group
    (2, 32, 8, 1, 4096, 128, False, [4096, 1000]),
    (2, 8, 1, 5, 300, 64, False, None),      # 8 heads per group
    (2, 4, 2, 40, 40, 128, True, None),      # two 32-row blocks per head, causal
    (1, 16, 4, 32, 513, 64, True, [400]),
    (2, 8, 4, 64, 200, 256, False, None),    # head dim 256: four wavefronts, two heads x two blocks
    (1, 6, 2, 17, 90, 96, False, None),      # three heads per group: one head per workgroup, same answers
    # more heads per kv head than wavefronts, or a number that does not divide them: a share of the
    # group's heads per workgroup (8 of 32, 8 of 16, 2 of 6, 4 of 12; 4 of 8 at head dim 256)
    (2, 32, 1, 1, 4096, 128, False, [4096, 1234]),
    (1, 64, 4, 2, 700, 64, False, None),
    (3, 12, 2, 1, 1000, 128, False, None),
    (1, 24, 2, 30, 260, 64, True, None),
    (2, 8, 1, 1, 520, 256, False, [520, 77]),
    (1, 8, 1, 1, 4096, 256, False, [3000]),  # ... and split keys at head dim 256 (no bias there)
    (2, 4, 4, 2, 2048, 192, False, None),
    # few (batch, kv head) pairs and many keys: the keys are split over workgroups and merged
    (1, 32, 8, 1, 8192, 128, False, [5000]),
    (2, 8, 2, 3, 4096, 64, False, [4096, 100]),
    (1, 16, 4, 8, 3000, 96, False, None),   # (also with a left-padding mask and a bias: split with a bias)
    (2, 8, 2, 1, 2048, 128, False, [0, 2048]),  # a batch without keys: zeros and lse = -inf
    (1, 8, 4, 33, 2500, 128, False, None),
    (2, 12, 12, 1, 4096, 64, False, [4096, 777]),  # one query head per kv head: split all the same
]


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("case", GROUPED, ids=lambda c: "B%d_Hq%d_Hkv%d_L%d_S%d_D%d_c%d" % c[:7])
def test_short_queries_with_grouped_heads(amd, gpu_device, case, dtype):
    B, Hq, Hkv, L, S, D, causal, lens = case
    q, k, v = qkv(B, Hq, Hkv, L, S, D, dtype=dtype, seed=L + S + D)
    kw, mask = {}, None
    if lens is not None:
        kw["kv_lens"] = torch.tensor(lens, dtype=torch.int32, device=gpu_device)
        mask = (torch.arange(S)[None] < torch.tensor(lens)[:, None])[:, None, None, :].expand(B, 1, L, S)
    if causal:
        cm = torch.ones(L, S, dtype=torch.bool).tril()
        mask = cm[None, None].expand(B, 1, L, S) if mask is None else mask & cm
    out, lse = amd.sdpa_forward(q.to(gpu_device), k.to(gpu_device), v.to(gpu_device), is_causal=causal, force_kernel=MFMA, **kw)
    ro, rl = oracle_fwd(q, k, v, attn_mask=mask)
    assert max_abs(out, ro) <= (2e-2 if dtype == torch.bfloat16 else 4e-3)
    assert max_abs(lse, rl) <= 2e-3 and torch.equal(torch.isfinite(lse.cpu()), torch.isfinite(rl))
    if not causal and lens is None and S % 4 == 0:
        # a mask that does not depend on the head keeps the heads together: left padding per key
        # (bool, what a batch of left-padded prompts sends with every decode step), and a per-score bias
        start = torch.randint(0, S // 2, (B,), generator=torch.Generator().manual_seed(S))
        lp = (torch.arange(S)[None] >= start[:, None])[:, None, None, :]
        out, lse = amd.sdpa_forward(q.to(gpu_device), k.to(gpu_device), v.to(gpu_device), attn_bias=lp.to(gpu_device), force_kernel=MFMA)
        ro, rl = oracle_fwd(q, k, v, attn_mask=lp.expand(B, 1, L, S))
        assert max_abs(out, ro) <= (2e-2 if dtype == torch.bfloat16 else 4e-3) and max_abs(lse, rl) <= 2e-3
        if B * Hkv < 256 and S >= 512:  # (these split their keys as well)
            need = B * Hq * L * 4
            assert need > 0
        bias = torch.randn(B, 1, L, S, generator=torch.Generator().manual_seed(S + 1)).to(dtype)
        out, lse = amd.sdpa_forward(q.to(gpu_device), k.to(gpu_device), v.to(gpu_device), attn_bias=bias.to(gpu_device), force_kernel=MFMA)
        ro, rl = oracle_fwd(q, k, v, attn_mask=bias.float())
        assert max_abs(out, ro) <= (2e-2 if dtype == torch.bfloat16 else 4e-3) and max_abs(lse, rl) <= 3e-3


# ---- float32 inputs on the float32 matrix op --------------------------------------------------------
# (the reference's fused gate takes float32, decompositions.py:2131-2158; shapes of its accuracy
# matrix, tests/python_ops/test_scaled_dot_product_attention.py:220-302 and :362-387)
F32_SHAPES = [
    # B, Hq, Hkv, L, S, E, causal
    (2, 4, 4, 128, 128, 64, False),      # config 1
    (1, 8, 8, 512, 512, 64, False),
    (1, 24, 6, 512, 512, 64, False),
    (1, 8, 1, 512, 512, 64, True),
    (1, 4, 2, 512, 512, 128, True),
    (2, 4, 2, 51, 51, 48, True),
    (2, 4, 2, 13, 51, 48, False),
    (1, 2, 1, 577, 577, 64, True),
    (1, 4, 4, 6, 6, 8, False),
    (2, 8, 2, 300, 1100, 128, True),
    (1, 2, 2, 200, 70, 104, True),
    (1, 4, 2, 512, 512, 256, True),      # (:362-387) head dim 256: width-256 instances, two dK/dV workgroups per key block
    (2, 2, 1, 100, 160, 160, False),
    (1, 3, 3, 40, 300, 136, True),
]


@pytest.mark.parametrize("shape", F32_SHAPES)
def test_float32_matrix_op_forward_and_backward(amd, gpu_device, shape):
    from helpers import oracle_bwd, rel_err

    B, Hq, Hkv, L, S, E, causal = shape
    q, k, v, go = qkv(B, Hq, Hkv, L, S, E, dtype=torch.float32, seed=L + S + E, with_do=True)
    qd, kd, vd, god = (t.to(gpu_device) for t in (q, k, v, go))
    out, lse = amd.sdpa_forward(qd, kd, vd, is_causal=causal, force_kernel=MFMA)
    dq, dk, dv, _ = amd.sdpa_backward(god, qd, kd, vd, out, lse, is_causal=causal, force_kernel=MFMA)
    torch.cuda.synchronize()
    ro, rl = oracle_fwd(q, k, v, is_causal=causal)
    rdq, rdk, rdv = oracle_bwd(go, q, k, v, ro, rl, is_causal=causal)
    assert max_abs(out, ro) <= 1e-5 and max_abs(lse, rl) <= 1e-5
    for a, r in ((dq, rdq), (dk, rdk), (dv, rdv)):
        assert a.shape == r.shape and a.dtype == torch.float32
        assert rel_err(a, r) <= 2e-6 and max_abs(a, r) <= 2e-5 * max(1.0, r.abs().max().item())
    # the library picks these kernels by itself for such calls, and the generic kernels agree with them
    out2, lse2 = amd.sdpa_forward(qd, kd, vd, is_causal=causal)
    assert torch.equal(out2, out) and torch.equal(lse2, lse)
    out3, _ = amd.sdpa_forward(qd, kd, vd, is_causal=causal, force_kernel=GENERIC)
    assert max_abs(out3, out) <= 1e-5


def test_float32_matrix_op_at_unequal_head_dims(amd, gpu_device):
    """D_qk = 192, D_v = 128 and D_qk = 128, D_v = 64 in float32 (forced into the float32 matrix-op kernels),
    causal with key counts, forward and backward against the oracle."""
    from oracle import sdpa_math as om

    dev = gpu_device
    for B, Hq, Hkv, L, S, E, Dv in ((2, 4, 2, 160, 192, 192, 128), (1, 4, 4, 100, 100, 128, 64), (1, 2, 1, 70, 130, 256, 8)):
        g = torch.Generator().manual_seed(E + Dv)
        q, k, v, go = (torch.randn(s_, generator=g) for s_ in ((B, Hq, L, E), (B, Hkv, S, E), (B, Hkv, S, Dv), (B, Hq, L, Dv)))
        lens = torch.randint(1, S + 1, (B,), generator=g).to(torch.int32)
        mask = (torch.arange(S)[None] < lens[:, None])[:, None, None, :].expand(B, Hq, L, S) & torch.ones(L, S, dtype=torch.bool).tril()
        bias = torch.where(mask, 0.0, float("-inf"))
        rep = Hq // Hkv
        kf, vf = k.repeat_interleave(rep, 1), v.repeat_interleave(rep, 1)
        ro, rl = om.compute_attention(q, kf, vf, bias, None, E**-0.5, False, 0.0)
        rdq, rdk, rdv, _ = om.compute_attention_backward(go, q, kf, vf, bias, None, ro, rl, E**-0.5, False, 0.0)
        rdk, rdv = rdk.view(B, Hkv, rep, S, E).sum(2), rdv.view(B, Hkv, rep, S, Dv).sum(2)
        kw = dict(is_causal=True, kv_lens=lens.to(dev), force_kernel=MFMA)
        out, lse = amd.sdpa_forward(q.to(dev), k.to(dev), v.to(dev), **kw)
        dq, dk, dv, _ = amd.sdpa_backward(go.to(dev), q.to(dev), k.to(dev), v.to(dev), out, lse, **kw)
        assert out.shape == (B, Hq, L, Dv) and dv.shape == (B, Hkv, S, Dv) and dk.shape == (B, Hkv, S, E)
        assert max_abs(out, ro) <= 1e-5 and max_abs(lse, rl) <= 1e-5
        for a, r in ((dq, rdq), (dk, rdk), (dv, rdv)):
            assert max_abs(a, r) <= 3e-5 * max(1.0, r.abs().max().item())


@pytest.mark.parametrize("shape", [(3, 4, 2, 100, 160, 64, False, [160, 1, 77]), (2, 8, 8, 300, 300, 128, True, [300, 130]),
                                   (2, 2, 2, 64, 96, 40, False, [0, 96])])
def test_float32_matrix_op_with_key_counts(amd, gpu_device, shape):
    """Per-batch key counts in the float32 kernels (what a right-padding mask becomes), forward and
    backward, against the oracle on the equivalent keep-mask; a batch without keys gives zeros."""
    from helpers import oracle_bwd, rel_err

    B, Hq, Hkv, L, S, E, causal, lens = shape
    q, k, v, go = qkv(B, Hq, Hkv, L, S, E, dtype=torch.float32, seed=L + S + E, with_do=True)
    qd, kd, vd, god = (t.to(gpu_device) for t in (q, k, v, go))
    kl = torch.tensor(lens, dtype=torch.int32, device=gpu_device)
    out, lse = amd.sdpa_forward(qd, kd, vd, is_causal=causal, kv_lens=kl, force_kernel=MFMA)
    dq, dk, dv, _ = amd.sdpa_backward(god, qd, kd, vd, out, lse, is_causal=causal, kv_lens=kl, force_kernel=MFMA)
    torch.cuda.synchronize()
    keep = (torch.arange(S)[None] < torch.tensor(lens)[:, None])[:, None, None, :].expand(B, 1, L, S)
    if causal:
        keep = keep & torch.ones(L, S, dtype=torch.bool).tril()
    ro, rl = oracle_fwd(q, k, v, attn_mask=keep)
    rdq, rdk, rdv = oracle_bwd(go, q, k, v, ro, rl, attn_mask=keep)
    assert max_abs(out, ro) <= 1e-5 and max_abs(lse, rl) <= 1e-5
    for a, r in ((dq, rdq), (dk, rdk), (dv, rdv)):
        assert torch.isfinite(a).all() and max_abs(a, r) <= 2e-5 * max(1.0, r.abs().max().item())
    out2, lse2 = amd.sdpa_forward(qd, kd, vd, is_causal=causal, kv_lens=kl)  # chosen by the library itself
    assert torch.equal(out2, out) and torch.equal(lse2, lse)


F32_FEW_ROWS = [
    # B, Hq, Hkv, L, S, E, extras
    (8, 32, 8, 1, 1023, 128, ""),            # a decode step: the heads of a kv group as rows, keys split
    (1, 32, 8, 1, 8192, 128, ""),
    (2, 8, 8, 1, 700, 64, ""),               # no group: keys split only
    (1, 4, 4, 100, 2000, 64, ""),            # a hundred rows against many keys
    (3, 16, 4, 1, 1500, 128, "lens"),
    (2, 16, 4, 1, 1100, 64, "key_bias"),     # a (B,1,1,S) additive padding mask
    (2, 8, 2, 1, 900, 128, "head_bias"),     # a bias per head: the heads stay heads
    (2, 8, 2, 1, 900, 128, "dropout"),
    (1, 8, 2, 1, 3000, 256, ""),             # width 256
    (2, 6, 3, 1, 40, 64, ""),                # few keys: grouped, not split
    (8, 32, 8, 4, 1024, 128, ""),            # four rows per head: sixteen rows per kv head
    (2, 8, 2, 5, 600, 64, "key_bias"),
    (2, 8, 2, 5, 600, 64, "rows_first"),     # q laid out (B,L,H,E): the heads stay heads
    (8, 32, 32, 1, 1024, 64, ""),
]


@pytest.mark.parametrize("case", F32_FEW_ROWS, ids=lambda c: "B%d_Hq%d_Hkv%d_L%d_S%d_E%d_%s" % c)
def test_float32_few_query_rows(amd, gpu_device, case):
    """Float32 with one query row per head (a decode step) or few rows against many keys: the heads of a kv
    group run as the rows of one head and the key tiles are split over workgroups into the workspace.
    Against the oracle, with and without the workspace (the same call unsplit)."""
    from oracle import sdpa_math as om

    B, Hq, Hkv, L, S, E, extra = case
    dev = gpu_device
    MFMA = amd._lib.KERNEL_MFMA
    g = torch.Generator().manual_seed(S + E)
    q, k, v = qkv(B, Hq, Hkv, L, S, E, dtype=torch.float32, seed=S + E)
    kw, bias, keep, pdrop = {}, None, None, 0.0
    if extra == "lens":
        lens = torch.tensor([S, 1, 777][:B])
        kw["kv_lens"] = lens.to(torch.int32).to(dev)
        bias = torch.where((torch.arange(S)[None] < lens[:, None])[:, None, None, :], 0.0, float("-inf")).expand(B, Hq, L, S)
    elif extra == "key_bias":
        bias = torch.randn(B, 1, 1, S, generator=g)
        bias[1, ..., S // 2:] = float("-inf")
        kw["attn_bias"] = bias.to(dev)
    elif extra == "head_bias":
        bias = torch.randn(1, Hq, 1, S, generator=g)
        kw["attn_bias"] = bias.to(dev)
    elif extra == "dropout":
        pdrop = 0.25
        keep = torch.rand(B, Hq, L, S, generator=g) >= pdrop
        kw.update(dropout_p=pdrop, dropout_keep=keep.to(dev))
    rep = Hq // Hkv
    ro, rl = om.compute_attention(q, k.repeat_interleave(rep, 1), v.repeat_interleave(rep, 1),
                                  None if bias is None else bias.expand(B, Hq, L, S), keep, E**-0.5, False, pdrop)
    qd, kd, vd = (t.to(dev) for t in (q, k, v))
    if extra == "rows_first":
        qd = qd.transpose(1, 2).contiguous().transpose(1, 2)
    out, lse = amd.sdpa_forward(qd, kd, vd, force_kernel=MFMA, **kw)
    assert max_abs(out, ro) <= 2e-5 and max_abs(lse, rl) <= 2e-5
    # the same call through the C ABI without a workspace: unsplit, the same numbers up to the order of the sums
    lib = amd._lib.load()
    real = lib.mi355_sdpa_fwd_workspace_bytes
    need = []
    try:
        class _NoWorkspace:
            def __call__(self, p):
                need.append(real(p))
                return 0
        lib.mi355_sdpa_fwd_workspace_bytes = _NoWorkspace()
        out2, lse2 = amd.sdpa_forward(qd, kd, vd, force_kernel=MFMA, **kw)
    finally:
        lib.mi355_sdpa_fwd_workspace_bytes = real
    assert (need[0] > 0) == (S >= 512), need
    assert max_abs(out2, out) <= 1e-5 and max_abs(lse2, lse) <= 1e-5


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
def test_split_key_merge_ignores_what_earlier_kernels_left_in_lds(amd, gpu_device, dtype):
    """The merge of a call with split keys keeps the parts' weights in LDS and adds the parts eight at a
    time: the slots past the last part must count as zero whatever an earlier kernel left there (a NaN
    times the zero of an absent part is a NaN).  Reductions over NaN tensors run first, on every compute
    unit; few parts (four), so that most of the eight slots are unused."""
    dev = gpu_device
    B, Hq, Hkv, L, S, E = 2, 96, 8, 32, 1100, 256
    if dtype is torch.float32:
        B, Hq, Hkv, L, S, E = 8, 32, 8, 1, 520, 128
    q, k, v = qkv(B, Hq, Hkv, L, S, E, dtype=dtype, seed=11)
    lens = torch.tensor(([546, 1064] if dtype is torch.bfloat16 else [520] * B), dtype=torch.int32)
    keep = (torch.arange(S)[None] < lens[:, None])[:, None, None, :].expand(B, 1, L, S)
    ro, rl = oracle_fwd(q, k, v, attn_mask=keep)
    qd, kd, vd, ld = q.to(dev), k.to(dev), v.to(dev), lens.to(dev)
    poison = torch.full((1 << 24,), float("nan"), device=dev)
    for _ in range(5):
        poison.view(4096, -1).sum(1)
        torch.softmax(poison.view(8192, -1), dim=1)
        torch.cumsum(poison.view(16384, -1), dim=1)
        out, lse = amd.sdpa_forward(qd, kd, vd, kv_lens=ld, force_kernel=amd._lib.KERNEL_MFMA)
        assert torch.isfinite(out.float()).all()
        assert max_abs(out, ro) <= (2e-2 if dtype is torch.bfloat16 else 2e-5) and max_abs(lse, rl) <= 2e-3


F32_MASKED = [
    # B, Hq, Hkv, L, S, E, causal, kind of mask, kv_lens
    (2, 4, 2, 100, 160, 64, False, "f32_full", None),
    (2, 4, 4, 96, 96, 128, False, "bf16_b1", None),
    (1, 8, 2, 300, 300, 128, False, "bool_full", None),
    (3, 2, 2, 33, 70, 40, False, "f16_key", [70, 5, 33]),
    (2, 4, 2, 64, 64, 64, True, "dropout", None),
    (2, 6, 6, 200, 130, 128, False, "dropout", [130, 77]),
    (1, 2, 2, 128, 128, 32, False, "dropout_all", None),
    (2, 4, 2, 100, 160, 64, False, "f32_full+dropout", None),
    (1, 8, 2, 300, 300, 128, True, "bool_full+dropout", None),
    (3, 2, 2, 33, 70, 40, False, "f16_key+dropout", [70, 5, 33]),
    (1, 2, 2, 100, 160, 256, True, "f32_full+dropout", None),   # width 256
    (2, 2, 1, 70, 96, 192, False, "bool_full", [96, 40]),
]


@pytest.mark.parametrize("case", F32_MASKED, ids=lambda c: "%s_L%d_S%d_E%d" % (c[7], c[3], c[4], c[5]))
def test_float32_matrix_op_with_a_bias_or_dropout(amd, gpu_device, case):
    """Per-score bias / keep-mask of every dtype and dropout in the float32 kernels (forced: the call
    fails if they cannot take it), forward and backward, against the oracle."""
    from oracle import sdpa_math as om

    B, Hq, Hkv, L, S, E, causal, kind, lens = case
    dev = gpu_device
    g = torch.Generator().manual_seed(L * 3 + S)
    q, k, v, go = qkv(B, Hq, Hkv, L, S, E, dtype=torch.float32, seed=L + S + E, with_do=True)
    kw, bias, keep, pdrop = {}, None, None, 0.0
    kind, _, both = kind.partition("+")
    if both:
        pdrop = 0.3
        keep = torch.rand(B, Hq, L, S, generator=g) >= pdrop
    if kind == "f32_full":
        bias = torch.randn(B, Hq, L, S, generator=g)
    elif kind == "bf16_b1":
        bias = torch.randn(1, Hq, L, S, generator=g).to(torch.bfloat16)
    elif kind == "bool_full":
        bias = torch.rand(B, 1, L, S, generator=g) > 0.4
        bias[..., 0] = True
    elif kind == "f16_key":
        bias = torch.randn(B, 1, 1, S, generator=g).to(torch.float16)
    elif kind == "dropout":
        pdrop = 0.3
        keep = torch.rand(B, Hq, L, S, generator=g) >= pdrop
    elif kind == "dropout_all":
        pdrop = 1.0
        keep = torch.zeros(B, Hq, L, S, dtype=torch.bool)
    if bias is not None:
        kw["attn_bias"] = bias.to(dev)
    if keep is not None:
        kw["dropout_p"], kw["dropout_keep"] = pdrop, keep.to(dev)
    add = None
    if bias is not None:
        add = (torch.where(bias, 0.0, float("-inf")) if bias.dtype == torch.bool else bias.float()).expand(B, Hq, L, S)
    if lens is not None:
        kw["kv_lens"] = torch.tensor(lens, dtype=torch.int32, device=dev)
        pad = torch.where(torch.arange(S)[None] < torch.tensor(lens)[:, None], 0.0, float("-inf"))[:, None, None, :].expand(B, Hq, L, S)
        add = pad if add is None else add + pad
    if causal:
        cm = torch.where(torch.ones(L, S, dtype=torch.bool).tril(), 0.0, float("-inf"))[None, None].expand(B, Hq, L, S)
        add = cm if add is None else add + cm
    rep = Hq // Hkv
    kf, vf = k.repeat_interleave(rep, 1), v.repeat_interleave(rep, 1)
    ro, rl = om.compute_attention(q, kf, vf, add, keep, E**-0.5, False, pdrop)
    rdq, rdk, rdv, _ = om.compute_attention_backward(go, q, kf, vf, add, keep, ro, rl, E**-0.5, False, pdrop)
    rdk, rdv = rdk.view(B, Hkv, rep, S, E).sum(2), rdv.view(B, Hkv, rep, S, E).sum(2)
    qd, kd, vd, god = (t.to(dev) for t in (q, k, v, go))
    out, lse = amd.sdpa_forward(qd, kd, vd, is_causal=causal, force_kernel=MFMA, **kw)
    dq, dk, dv, _ = amd.sdpa_backward(god, qd, kd, vd, out, lse, is_causal=causal, force_kernel=MFMA, **kw)
    live = torch.isfinite(rl)
    assert max_abs(out, ro) <= 2e-5 and max_abs(lse.cpu()[live], rl[live]) <= 2e-5
    assert torch.equal(torch.isfinite(lse.cpu()), live)
    for a, r in ((dq, rdq), (dk, rdk), (dv, rdv)):
        assert torch.isfinite(a).all() and max_abs(a, r) <= 3e-5 * max(1.0, r.abs().max().item())


def test_float32_matrix_op_refuses_what_it_does_not_serve(amd, gpu_device):
    q, k, v = (t.to(gpu_device) for t in qkv(1, 2, 2, 64, 64, 64, dtype=torch.float32, seed=1))
    keep = torch.ones(1, 2, 64, 64, dtype=torch.uint8, device=gpu_device)
    with pytest.raises(NotImplementedError, match="float32 MFMA"):  # dropout together with a functor
        amd.sdpa_forward(q, k, v, window=16, is_causal=True, dropout_p=0.5, dropout_keep=keep, force_kernel=MFMA)
    out, _ = amd.sdpa_forward(q, k, v, window=64, is_causal=True, dropout_p=0.5, dropout_keep=keep)  # served by the generic kernel
    ro, _ = oracle_fwd(q.cpu(), k.cpu(), v.cpu(), is_causal=True)
    assert max_abs(out, 2.0 * ro) <= 2e-5


def test_split_keys_need_the_workspace_and_agree_with_the_unsplit_call(amd, gpu_device):
    """Through the C ABI: the size query says that a decode-like call would split its keys; with the
    workspace it does (and merges), without it the same call runs unsplit; both agree with the oracle,
    and with each other to float32 rounding."""
    import ctypes as C

    from torch_neuronx_amd import _lib

    B, Hq, Hkv, S, D = 1, 32, 8, 8192, 128
    q, k, v = (t.to(gpu_device) for t in qkv(B, Hq, Hkv, 1, S, D, dtype=torch.bfloat16, seed=77))

    def call(with_ws):
        out = torch.empty_like(q)
        lse = torch.empty(B, Hq, 1, dtype=torch.float32, device=gpu_device)
        p = _lib.FwdParams()
        p.q, p.k, p.v, p.out = (_lib.tensor4(t) for t in (q, k, v, out))
        p.lse, p.dtype, p.scale, p.force_kernel = lse.data_ptr(), _lib.dtype_id(q.dtype), D**-0.5, MFMA
        need = _lib.load().mi355_sdpa_fwd_workspace_bytes(C.byref(p))
        assert need == B * Hq * 32 * 1 * (D + 1) * 4  # 256 tiles in 32 parts of 8
        ws = torch.empty(need, dtype=torch.uint8, device=gpu_device)
        if with_ws:
            p.workspace, p.workspace_bytes = ws.data_ptr(), need
        with _lib.on_device(q.device):
            _lib.check(_lib.load().mi355_sdpa_fwd(C.byref(p), _lib.current_stream(q.device)))
        torch.cuda.synchronize()
        return out, lse

    o1, l1 = call(True)
    o0, l0 = call(False)
    ro, rl = oracle_fwd(q.cpu(), k.cpu(), v.cpu())
    for o, l in ((o1, l1), (o0, l0)):
        assert max_abs(o, ro) <= 2e-2 and max_abs(l, rl) <= 2e-3
    assert max_abs(o1, o0) <= 4e-3 and max_abs(l1, l0) <= 1e-5
