"""Tile skip tables of masks that only exist as tensors: the tables themselves against a plain torch
restatement, and the kernels that use them (forward walks the live key tiles only, dK/dV leaves out
the dead query tiles) against the same kernels without tables and against the CPU oracle, through
the C ABI.  The tables are the run-time counterpart of the reference's static tile elimination
(torch_neuronx/neuron_dynamo_backend/flex_attention/flex_attention.py.jinja:15-33)."""

import pytest
import torch

from helpers import max_abs, oracle_bwd, oracle_fwd, qkv

pytestmark = pytest.mark.gpu

MFMA = 2


@pytest.fixture(scope="module")
def amd(gpu_device):
    import torch_neuronx_amd as amd

    return amd


def document_mask(lengths, B=1, causal=False):
    """Block-diagonal keep-mask of packed sequences: a query sees the keys of its own document."""
    n = sum(lengths)
    doc = torch.repeat_interleave(torch.arange(len(lengths)), torch.tensor(lengths))
    m = doc[:, None] == doc[None, :]
    if causal:
        m = m & torch.tril(torch.ones(n, n, dtype=torch.bool))
    return m[None, None].expand(B, 1, n, n).contiguous()


def as_kind(mask, kind):
    if kind == "bool":
        return mask
    dt = {"float32": torch.float32, "float16": torch.float16, "bfloat16": torch.bfloat16}[kind]
    return torch.where(mask, 0.0, float("-inf")).to(dt)


def reference_tables(mask):
    """live[b,h,row block of 64][key tile of 32], live_t[b,h,key block of 128][query tile of 64] as bools."""
    keep = mask if mask.dtype == torch.bool else mask != float("-inf")
    Bm, Hm, L, S = keep.shape
    nrb, ntl, nkb = (L + 63) // 64, (S + 31) // 32, (S + 127) // 128
    pad = torch.zeros(Bm, Hm, nrb * 64, nkb * 128, dtype=torch.bool)
    pad[:, :, :L, :S] = keep
    live = pad.view(Bm, Hm, nrb, 64, nkb * 4, 32).any(dim=5).any(dim=3)[..., :ntl]
    live_t = pad.view(Bm, Hm, nrb, 64, nkb, 128).any(dim=5).any(dim=3).transpose(2, 3)
    return live, live_t


def unpack(words, shape_prefix, nbits):
    w = words.cpu().view(*shape_prefix, -1).to(torch.int64) & 0xFFFFFFFF
    bits = (w[..., None] >> torch.arange(32)) & 1
    return bits.flatten(-2)[..., :nbits].bool()


@pytest.mark.parametrize("kind", ["bool", "float32", "float16", "bfloat16"])
@pytest.mark.parametrize("shape", [(1, 1, 512, 512), (2, 3, 200, 1096), (1, 2, 1000, 72), (2, 1, 4100, 4100)])
def test_tables_match_a_torch_restatement(amd, gpu_device, kind, shape):
    Bm, Hm, L, S = shape
    g = torch.Generator().manual_seed(L * 7 + S)
    # blocks of 40 x 56 scores kept with probability 0.3, with single kept scores sprinkled in
    coarse = torch.rand(Bm, Hm, (L + 39) // 40, (S + 55) // 56, generator=g) < 0.3
    mask = coarse.repeat_interleave(40, 2).repeat_interleave(56, 3)[:, :, :L, :S].clone()
    mask |= torch.rand(Bm, Hm, L, S, generator=g) < 2e-5
    m = as_kind(mask, kind).to(gpu_device)
    maps = amd.ops.mask_tile_maps(m, Bm, Hm, L, S)
    assert maps is not None
    torch.cuda.synchronize()
    live, live_t = reference_tables(mask)
    nrb, ntl, nkb = (L + 63) // 64, (S + 31) // 32, (S + 127) // 128
    assert torch.equal(unpack(maps[0], (Bm, Hm, nrb), ntl), live)
    assert torch.equal(unpack(maps[1], (Bm, Hm, nkb), nrb), live_t)


def test_masks_without_tables(amd, gpu_device):
    # a mask per key (nothing to skip by row block) and one whose rows are not dword aligned
    per_key = (torch.rand(2, 1, 1, 512) > 0.5).to(gpu_device)
    assert amd.ops.mask_tile_maps(per_key, 2, 4, 512, 512) is None
    odd = (torch.rand(1, 1, 300, 510) > 0.5).to(gpu_device)
    assert amd.ops.mask_tile_maps(odd, 1, 1, 300, 510) is None


CASES = [
    # B, Hq, Hkv, E, document lengths, mask batch, kind
    (1, 4, 2, 128, [300, 212, 512], 1, "bool"),
    (2, 8, 2, 128, [1000, 24, 500, 524], 2, "bool"),
    (2, 4, 4, 64, [700, 324], 1, "bfloat16"),
    (1, 4, 1, 128, [256, 256, 256, 256], 1, "float32"),
    (1, 2, 2, 256, [384, 640], 1, "bool"),
    (1, 4, 4, 96, [100, 412, 512], 1, "float16"),
    (2, 4, 2, 192, [300, 600, 124], 2, "bool"),
]


@pytest.mark.parametrize("case", CASES)
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_forward_and_backward_with_tables(amd, gpu_device, case, dtype):
    B, Hq, Hkv, E, lengths, Bm, kind = case
    n = sum(lengths)
    q, k, v, go = qkv(B, Hq, Hkv, n, n, E, dtype=dtype, seed=n + E, with_do=True)
    mask = document_mask(lengths, Bm, causal=True)
    if Bm > 1:
        mask[1] = document_mask(list(reversed(lengths)), 1)[0]  # the second batch: another layout, not causal
    mask[0, 0, 70:75] = False  # a few rows that see nothing
    m = as_kind(mask, kind)
    if kind in ("float16", "bfloat16") and m.dtype != dtype:
        m = m.to(dtype)
    qd, kd, vd, god, md = (t.to(gpu_device) for t in (q, k, v, go, m))
    o0, l0 = amd.sdpa_forward(qd, kd, vd, attn_bias=md, force_kernel=MFMA)
    o1, l1 = amd.sdpa_forward(qd, kd, vd, attn_bias=md, force_kernel=MFMA, live_tiles=True)
    torch.cuda.synchronize()
    # skipped tiles contribute exact zeros: the same numbers with and without the tables
    assert max_abs(o1, o0.cpu()) <= 1e-6 and torch.equal(torch.isinf(l1), torch.isinf(l0))
    fin = ~torch.isinf(l0)
    assert (l1[fin] - l0[fin]).abs().max().item() <= 1e-5
    ro, rl = oracle_fwd(q, k, v, attn_mask=mask.expand(B, 1, n, n) if kind == "bool" else m.float().expand(B, 1, n, n))
    assert max_abs(o1, ro) <= 2e-2
    assert torch.equal(torch.isinf(l1.cpu()), torch.isinf(rl)) and (l1.cpu()[fin.cpu()] - rl[fin.cpu()]).abs().max().item() <= 5e-3
    g0 = amd.sdpa_backward(god, qd, kd, vd, o0, l0, attn_bias=md, force_kernel=MFMA)
    g1 = amd.sdpa_backward(god, qd, kd, vd, o0, l0, attn_bias=md, force_kernel=MFMA, live_tiles=True)
    torch.cuda.synchronize()
    # (dK and dV: a call with few key blocks deals a block's query tiles to several workgroups, and
    # the tables change which tiles a workgroup adds up before the float32 partial sums meet: one
    # rounding step of the output dtype at most)
    step = 2.0**-7 if dtype == torch.bfloat16 else 2.0**-10
    for a, b_ in zip(g1[:3], g0[:3]):
        a, b_ = a.float().cpu(), b_.float().cpu()
        assert ((a - b_).abs() <= step * b_.abs() + 1e-6).all()
    bias = mask.expand(B, 1, n, n) if kind == "bool" else m.float().expand(B, 1, n, n)
    rq, rk, rv = oracle_bwd(go, q, k, v, ro, rl, attn_mask=bias)[:3]
    for a, r in zip(g1[:3], (rq, rk, rv)):
        assert max_abs(a, r) <= 5e-2


@pytest.mark.parametrize("shape", [(2, 4, 2, 700, 1100, 128, "head"), (1, 6, 3, 1100, 700, 64, "batch"), (2, 2, 2, 520, 2080, 128, "one")])
def test_rectangular_block_sparse_masks_with_tables(amd, gpu_device, shape):
    # L != S, masks with their own head or batch extent, rows and whole row blocks without a kept score
    B, Hq, Hkv, L, S, E, extent = shape
    q, k, v, go = qkv(B, Hq, Hkv, L, S, E, dtype=torch.bfloat16, seed=L + S, with_do=True)
    g = torch.Generator().manual_seed(L * 3 + S)
    Bm, Hm = (B, Hq) if extent == "head" else (B, 1) if extent == "batch" else (1, 1)
    coarse = torch.rand(Bm, Hm, (L + 47) // 48, (S + 79) // 80, generator=g) < 0.25
    mask = coarse.repeat_interleave(48, 2).repeat_interleave(80, 3)[:, :, :L, :S].contiguous()
    qd, kd, vd, god, md = (t.to(gpu_device) for t in (q, k, v, go, mask))
    o0, l0 = amd.sdpa_forward(qd, kd, vd, attn_bias=md, force_kernel=MFMA)
    o1, l1 = amd.sdpa_forward(qd, kd, vd, attn_bias=md, force_kernel=MFMA, live_tiles=True)
    g0 = amd.sdpa_backward(god, qd, kd, vd, o0, l0, attn_bias=md, force_kernel=MFMA)
    g1 = amd.sdpa_backward(god, qd, kd, vd, o0, l0, attn_bias=md, force_kernel=MFMA, live_tiles=True)
    torch.cuda.synchronize()
    assert max_abs(o1, o0.cpu()) <= 1e-6 and max_abs(l1, l0.cpu()) <= 1e-5
    for a, b_ in zip(g1[:3], g0[:3]):  # (one rounding step where the call splits a key block's query tiles: see above)
        a, b_ = a.float().cpu(), b_.float().cpu()
        assert ((a - b_).abs() <= 2.0**-7 * b_.abs() + 1e-6).all()
    ro, rl = oracle_fwd(q, k, v, attn_mask=mask)
    assert max_abs(o1, ro) <= 2e-2 and max_abs(l1, rl) <= 5e-3
    for a, r in zip(g1[:3], oracle_bwd(go, q, k, v, ro, rl, attn_mask=mask)[:3]):
        assert max_abs(a, r) <= 5e-2


def test_workgroups_without_a_live_tile(amd, gpu_device):
    # whole 256-row blocks of queries see no key: zeros, lse = -inf, zero gradients
    B, H, n, E = 1, 2, 1024, 128
    q, k, v, go = qkv(B, H, H, n, n, E, dtype=torch.bfloat16, seed=5, with_do=True)
    mask = torch.ones(1, 1, n, n, dtype=torch.bool)
    mask[:, :, 256:768] = False
    mask[:, :, :, 512:] = False
    qd, kd, vd, god, md = (t.to(gpu_device) for t in (q, k, v, go, mask))
    out, lse = amd.sdpa_forward(qd, kd, vd, attn_bias=md, force_kernel=MFMA, live_tiles=True)
    dq, dk, dv, _ = amd.sdpa_backward(god, qd, kd, vd, out, lse, attn_bias=md, force_kernel=MFMA, live_tiles=True)
    torch.cuda.synchronize()
    assert torch.all(out[:, :, 256:768] == 0) and torch.all(torch.isinf(lse[:, :, 256:768]))
    assert torch.all(dq[:, :, 256:768] == 0) and torch.all(dk[:, :, 512:] == 0) and torch.all(dv[:, :, 512:] == 0)
    ro, rl = oracle_fwd(q, k, v, attn_mask=mask)
    assert max_abs(out, ro) <= 2e-2
    rq, rk, rv = oracle_bwd(go, q, k, v, ro, rl, attn_mask=mask)[:3]
    assert max_abs(dq, rq) <= 5e-2 and max_abs(dk, rk) <= 5e-2 and max_abs(dv, rv) <= 5e-2


def test_document_mask_through_the_operator_skips_tiles(amd, gpu_device):
    # eight packed documents of 512 over 4096 keys through the registered operator: the tables are
    # built once per mask tensor, results equal the call without them, and seven eighths of the
    # tiles are not computed
    from torch_neuronx_amd import mask_patterns

    B, Hq, Hkv, n, E = 2, 16, 4, 4096, 128
    q, k, v = (t.to(gpu_device) for t in qkv(B, Hq, Hkv, n, n, E, dtype=torch.bfloat16, seed=11))
    mask = document_mask([512] * 8).to(gpu_device)
    mask_patterns.clear_cache()
    before = dict(mask_patterns.stats)
    op = torch.ops.aten._scaled_dot_product_fused_attention_overrideable
    first = op(q, k, v, attn_bias=mask)[0]  # first sight: nothing is known about the mask yet, it is taken as it is
    torch.cuda.synchronize()
    assert mask_patterns.stats.get("tile_builds", 0) == before.get("tile_builds", 0)
    out = op(q, k, v, attn_bias=mask)[0]  # known to be no pattern by now: tables
    out2 = op(q, k, v, attn_bias=mask)[0]
    torch.cuda.synchronize()
    assert max_abs(first, out) <= 1e-6
    assert mask_patterns.stats.get("tile_builds", 0) - before.get("tile_builds", 0) == 1
    assert mask_patterns.stats.get("tile_hits", 0) - before.get("tile_hits", 0) == 1
    ref, _ = amd.sdpa_forward(q, k, v, attn_bias=mask, force_kernel=MFMA)
    assert max_abs(out, ref.cpu()) <= 1e-6 and torch.equal(out, out2)

    def timed(fn, n_it=10):
        for _ in range(3):
            fn()
        a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        a.record()
        for _ in range(n_it):
            fn()
        b.record()
        torch.cuda.synchronize()
        return a.elapsed_time(b) / n_it

    t_plain = timed(lambda: amd.sdpa_forward(q, k, v, attn_bias=mask, force_kernel=MFMA))
    t_table = timed(lambda: op(q, k, v, attn_bias=mask))
    assert t_table < 0.4 * t_plain, (t_table, t_plain)
    # ... and so does the backward (dQ walks the live key tiles, dK/dV the live query tiles)
    go = torch.randn_like(out)
    lse = op(q, k, v, attn_bias=mask)[1]
    maps = mask_patterns.tile_maps(mask, B, Hq, n, n)
    b_plain = timed(lambda: amd.sdpa_backward(go, q, k, v, out, lse, attn_bias=mask, force_kernel=MFMA), 5)
    b_table = timed(lambda: amd.sdpa_backward(go, q, k, v, out, lse, attn_bias=mask, force_kernel=MFMA, live_tiles=maps), 5)
    assert b_table < 0.4 * b_plain, (b_table, b_plain)
