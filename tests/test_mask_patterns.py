"""Recognition of masks that the kernels generate by themselves (causal, sliding window with sink
keys, keep-everything): the run-time counterpart of the reference's causal-mask recovery
(fx/passes/sdpa_causal_mask.py:162-289).  The host logic is checked on the CPU against brute force;
the device row summary, the routing and its effect on results and time are GPU tests."""

import numpy as np
import pytest
import torch
import torch.nn.functional as F

from helpers import max_abs, qkv, rel_err
from oracle import sdpa_math as om


def rows_of(mask: np.ndarray) -> np.ndarray:
    """Brute-force row summary of a boolean (L, S) mask."""
    L, S = mask.shape
    out = np.zeros((L, 4), dtype=np.int32)
    for i in range(L):
        kept = np.flatnonzero(mask[i])
        hi = int(kept[-1]) if kept.size else -1
        dropped = np.flatnonzero(~mask[i])
        lead = int(dropped[0]) if dropped.size else S
        gaps = dropped[dropped < hi]
        out[i] = (hi, kept.size, lead, int(gaps[-1]) + 1 if gaps.size else 0)
    return out


def pattern(mask_bool: torch.Tensor):
    from torch_neuronx_amd.mask_patterns import pattern_from_rows

    m = mask_bool.numpy()
    return pattern_from_rows(rows_of(m), *m.shape)


def rebuild(pat, L, S):
    if pat == ("all",):
        return torch.ones(L, S, dtype=torch.bool)
    if pat == ("causal",):
        return om.window_keep_mask(L, S, 0)
    return om.window_keep_mask(L, S, pat[1], pat[2])


@pytest.mark.parametrize("L,S", [(16, 16), (9, 30), (30, 9), (1, 5), (64, 64)])
def test_causal_and_full_masks_are_recognised(L, S):
    assert pattern(torch.ones(L, S, dtype=torch.bool)) == ("all",)
    tril = torch.tril(torch.ones(L, S, dtype=torch.bool))
    want = ("all",) if (tril.all()) else ("causal",)
    assert pattern(tril) == want


@pytest.mark.parametrize("L,W,N", [(40, 7, 0), (40, 7, 3), (40, 1, 0), (40, 16, 16), (40, 10, 30), (33, 32, 1), (70, 64, 0)])
def test_window_masks_are_recognised(L, W, N):
    m = om.window_keep_mask(L, L, W, N)
    pat = pattern(m)
    assert pat is not None and torch.equal(rebuild(pat, L, L), m)  # (N may come back smaller when the window covers it)
    if N < L - W:
        assert pat == ("window", W, N)


def test_anything_else_is_left_alone():
    g = torch.Generator().manual_seed(0)
    L = 48
    assert pattern(torch.rand(L, L, generator=g) < 0.5) is None
    tril = torch.tril(torch.ones(L, L, dtype=torch.bool))
    for (i, j) in [(10, 3), (30, 12), (5, 5), (0, 1), (20, 30)]:  # (a key dropped in the last row only would be a window)
        m = tril.clone()
        m[i, j] = not m[i, j]
        assert pattern(m) is None, (i, j)
    w = om.window_keep_mask(L, L, 9, 2)
    for (i, j) in [(30, 1), (30, 22), (30, 5), (47, 39), (12, 2)]:
        m = w.clone()
        m[i, j] = not m[i, j]
        assert pattern(m) is None, (i, j)
    assert pattern(torch.triu(torch.ones(L, L, dtype=torch.bool))) is None       # upper triangle
    assert pattern(torch.tril(torch.ones(L, L, dtype=torch.bool), -1)) is None   # strictly lower: row 0 is dead
    pad = torch.ones(L, L, dtype=torch.bool)
    pad[:, 40:] = False
    assert pattern(pad) is None                                                   # key padding


def test_recognition_is_sound_on_random_near_patterns():
    # whatever is recognised rebuilds exactly the mask it came from
    g = torch.Generator().manual_seed(1)
    seen = 0
    for trial in range(300):
        L = int(torch.randint(2, 40, (1,), generator=g))
        S = int(torch.randint(2, 40, (1,), generator=g))
        W = int(torch.randint(0, 12, (1,), generator=g))
        N = int(torch.randint(0, 6, (1,), generator=g)) if W else 0
        m = om.window_keep_mask(L, S, W, N)
        if trial % 3 == 0:
            i, j = int(torch.randint(0, L, (1,), generator=g)), int(torch.randint(0, S, (1,), generator=g))
            m[i, j] = not m[i, j]
        pat = pattern(m)
        if pat is not None:
            seen += 1
            assert torch.equal(rebuild(pat, L, S), m), (L, S, W, N, pat)
    assert seen > 100


def test_window_masks_with_right_padding_are_recognised():
    # what model code builds for a sliding-window model from a padded batch: window & causal & key < len[b]
    from torch_neuronx_amd.mask_patterns import window_lens_pattern_from_rows

    def rows3(m):
        return np.stack([rows_of(x.numpy()) for x in m])

    def rebuild3(pat, L, S):
        W, N, lens = pat[1], pat[2], pat[3]
        return torch.stack([om.window_keep_mask(L, S, W, N) & (torch.arange(S)[None] < int(n)) for n in lens])

    g = torch.Generator().manual_seed(5)
    seen = exact = 0
    for trial in range(300):
        L = int(torch.randint(2, 40, (1,), generator=g))
        S = L if trial % 2 else int(torch.randint(2, 40, (1,), generator=g))
        W = int(torch.randint(1, 12, (1,), generator=g))
        N = int(torch.randint(0, 5, (1,), generator=g))
        B = int(torch.randint(1, 5, (1,), generator=g))
        lens = torch.randint(0, S + 1, (B,), generator=g)
        m = om.window_keep_mask(L, S, W, N)[None] & (torch.arange(S)[None] < lens[:, None])[:, None, :]
        if trial % 3 == 0:
            b, i, j = (int(torch.randint(0, n, (1,), generator=g)) for n in (B, L, S))
            m[b, i, j] = not m[b, i, j]
        pat = window_lens_pattern_from_rows(rows3(m), L, S)
        if pat is not None:  # whatever is recognised rebuilds exactly the mask it came from
            seen += 1
            assert torch.equal(rebuild3(pat, L, S), m), (L, S, W, N, lens.tolist(), pat)
        elif trial % 3 and min(L, int(lens.max())) > W + N:  # an unperturbed mask in which the window shows is recognised
            raise AssertionError((L, S, W, N, lens.tolist()))
        exact += trial % 3 != 0
    assert seen > 100
    # left padding and a causal mask with padding are other patterns
    L = S = 24
    left = om.window_keep_mask(L, S, 5, 0)[None] & (torch.arange(S)[None] >= torch.tensor([0, 4])[:, None])[:, None, :]
    assert window_lens_pattern_from_rows(rows3(left), L, S) is None
    tril = torch.tril(torch.ones(L, S, dtype=torch.bool))[None]
    assert window_lens_pattern_from_rows(rows3(tril), L, S) is None


# ---- GPU ----------------------------------------------------------------------------------------------


def test_padding_masks_become_key_counts():
    # what model code builds from right padding, with or without causality folded in, per batch
    from torch_neuronx_amd.mask_patterns import lens_pattern_from_rows

    def rows3(m):
        return np.stack([rows_of(x.numpy()) for x in m])

    L, S = 12, 20
    lens = torch.tensor([20, 7, 1, 13])
    pad = (torch.arange(S)[None] < lens[:, None])[:, None, :].expand(4, L, S)
    pat = lens_pattern_from_rows(rows3(pad), L, S, rows_broadcast=False)
    assert pat[0] == "all" and pat[1].tolist() == lens.tolist()
    pat = lens_pattern_from_rows(rows3(pad[:, :1]), L, S, rows_broadcast=True)
    assert pat[0] == "all" and pat[1].tolist() == lens.tolist()
    tril = torch.tril(torch.ones(L, S, dtype=torch.bool))
    pat = lens_pattern_from_rows(rows3(pad & tril), L, S, rows_broadcast=False)
    # (a batch whose padding starts behind the last row's diagonal is indistinguishable from no padding)
    assert pat[0] == "causal" and pat[1].tolist() == [20, 7, 1, 20]
    for b in range(4):
        n = int(pat[1][b])
        assert torch.equal(pad[b] & tril, tril & (torch.arange(S)[None] < min(n, int(lens[b]))))
    # anything else is left alone: left padding, a hole, a row that keeps a later key
    left = (torch.arange(S)[None] >= lens[:, None])[:, None, :].expand(4, L, S)
    assert lens_pattern_from_rows(rows3(left), L, S, rows_broadcast=False) is None
    holed = (pad & tril).clone()
    holed[1, 9, 3] = False
    assert lens_pattern_from_rows(rows3(holed), L, S, rows_broadcast=False) is None
    late = (pad & tril).clone()
    late[1, 9, 15] = True
    assert lens_pattern_from_rows(rows3(late), L, S, rows_broadcast=False) is None
    one_row_causal = (pad & tril)[:, :1]
    assert lens_pattern_from_rows(rows3(one_row_causal), L, S, rows_broadcast=True)[0] == "all"  # row 0 keeps key 0 only, everywhere


@pytest.fixture(scope="module")
def amd(gpu_device):
    import torch_neuronx_amd as amd

    return amd


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [torch.bool, torch.float32, torch.bfloat16, torch.float16])
def test_device_row_summary_matches_brute_force(amd, gpu_device, dtype):
    import ctypes as C

    from torch_neuronx_amd import _lib

    g = torch.Generator().manual_seed(3)
    L, S = 37, 203
    keep = torch.rand(L, S, generator=g) < 0.6
    keep[5] = False
    keep[6] = True
    m = keep if dtype is torch.bool else torch.zeros(L, S, dtype=dtype).masked_fill(~keep, float("-inf"))
    wide = torch.zeros(L, S + 13, dtype=m.dtype)
    wide[:, :S] = m
    md = wide.to(gpu_device)[:, :S]  # row stride != S
    rows = torch.empty(L, 4, dtype=torch.int32, device=gpu_device)
    rc = _lib.load().mi355_sdpa_mask_rows(md.data_ptr(), _lib.dtype_id(md.dtype), L, S, md.stride(0), rows.data_ptr(),
                                          _lib.current_stream(gpu_device))
    assert rc == 0
    assert np.array_equal(rows.cpu().numpy(), rows_of(keep.numpy()))
    if dtype is not torch.bool:  # a real bias value makes the row "not a mask"
        md2 = md.clone()
        md2[3, 100] = 0.5
        _lib.load().mi355_sdpa_mask_rows(md2.data_ptr(), _lib.dtype_id(md2.dtype), L, S, md2.stride(0), rows.data_ptr(),
                                         _lib.current_stream(gpu_device))
        got = rows.cpu().numpy()
        assert got[3, 1] == -1 and (np.delete(got, 3, 0)[:, 1] >= 0).all()


def _within(fn, base, limit, attempts=3):
    """Whether ``fn`` runs within ``limit`` times the time of ``base`` (timings on a shared machine: the best
    of up to three rounds counts); the rounds seen, for the assertion message."""
    seen = []
    for _ in range(attempts):
        seen.append((_best_ms(fn), _best_ms(base)))
        if seen[-1][0] <= limit * seen[-1][1]:
            return True, seen
    return False, seen


def _best_ms(fn, reps=5, inner=10):
    best = 1e9
    for _ in range(reps):
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(inner):
            fn()
        e1.record()
        torch.cuda.synchronize()
        best = min(best, e0.elapsed_time(e1) / inner)
    return best


@pytest.mark.gpu
def test_tril_mask_takes_the_causal_kernel(amd, gpu_device, monkeypatch):
    dev = gpu_device
    L = 4096
    # (no GQA here: upstream sends a mask together with enable_gqa to its composite math path)
    q, k, v, go = (t.to(dev) for t in qkv(1, 8, 8, L, L, 128, dtype=torch.bfloat16, seed=2, with_do=True))
    tril = torch.ones(L, L, dtype=torch.bool, device=dev).tril()[None, None]
    amd.mask_patterns.clear_cache()
    seen = []
    f0 = amd.ops.sdpa_forward
    monkeypatch.setattr(amd.ops, "sdpa_forward", lambda *a, **kw: (seen.append(kw), f0(*a, **kw))[1])
    # the reference's own operator, with the mask as the caller made it
    fused = torch.ops.aten._scaled_dot_product_fused_attention_overrideable
    fused_bwd = torch.ops.aten._scaled_dot_product_fused_attention_overrideable_backward
    # first sight: the mask travels on with its verdict, and the kernels take the decision on the device
    r_v = fused(q, k, v, tril)
    assert seen[-1]["attn_bias"] is not None and seen[-1].get("mask_verdict") is not None
    r_c = fused(q, k, v, None, 0.0, True)
    assert max_abs(r_v[0], r_c[0]) <= 4e-3 and max_abs(r_v[1], r_c[1]) <= 1e-4
    g_v = fused_bwd(go, q, k, v, tril, [True, True, True, False], r_v[0], r_v[1], None, None, L, L, 0.0, False, r_v[6], r_v[7])
    g_c = fused_bwd(go, q, k, v, None, [True, True, True, False], r_c[0], r_c[1], None, None, L, L, 0.0, True, r_c[6], r_c[7])
    for a, b in zip(g_v[:3], g_c[:3]):
        assert max_abs(a, b) <= 2e-2 and rel_err(a, b) <= 5e-3
    # once the verdict's copy has reached the host (no call waits for it), the mask is dropped for the flag
    torch.cuda.synchronize()
    r_m = fused(q, k, v, tril)
    assert seen[-1]["attn_bias"] is None and seen[-1]["is_causal"] is True
    assert torch.equal(r_m[0], r_c[0]) and torch.equal(r_m[1], r_c[1])  # the same kernel, bit for bit
    g_m = fused_bwd(go, q, k, v, tril, [True, True, True, False], r_m[0], r_m[1], None, None, L, L, 0.0, False, r_m[6], r_m[7])
    for a, b in zip(g_m[:3], g_c[:3]):
        assert torch.equal(a, b)
    # ... and at its speed
    ok, seen_t = _within(lambda: fused(q, k, v, tril), lambda: fused(q, k, v, None, 0.0, True), 1.10)
    assert ok, seen_t
    # a mask that changes in place is looked at again
    tril[0, 0, 100, 3000] = True
    r_x = fused(q, k, v, tril)
    assert seen[-1]["attn_bias"] is not None and not torch.equal(r_x[0], r_c[0])
    tril[0, 0, 100, 3000] = False
    # the functional API: an additive mask that the caller keeps is recognised (and cached) ...
    fm = torch.zeros(L, L, device=dev, dtype=torch.bfloat16).masked_fill(~tril[0, 0], float("-inf"))
    F.scaled_dot_product_attention(q, k, v, attn_mask=fm)
    torch.cuda.synchronize()
    out_f = F.scaled_dot_product_attention(q, k, v, attn_mask=fm)
    assert seen[-1]["attn_bias"] is None and seen[-1]["is_causal"] is True and torch.equal(out_f, r_c[0])
    # ... while a boolean one reaches the fused op as a fresh additive tensor on every call: each of them
    # gets its verdict on the device (after a few, no copy to the host any more)
    amd.mask_patterns.clear_cache()
    looked0 = amd.mask_patterns.stats["looked"]
    for _ in range(8):
        out_b = F.scaled_dot_product_attention(q, k, v, attn_mask=tril)
        assert seen[-1]["attn_bias"] is not None and seen[-1].get("mask_verdict") is not None
    assert amd.mask_patterns.stats["looked"] - looked0 == 3
    assert max_abs(out_b, r_c[0]) <= 4e-3


def _holed(keep3, b):
    """One kept score dropped in batch ``b``: the middle one of the row that keeps the most."""
    keep3 = keep3.clone()
    i = int(keep3[b].sum(-1).argmax())
    kept = torch.nonzero(keep3[b, i]).flatten()
    keep3[b, i, kept[kept.numel() // 2]] = False
    return keep3


def _keep_masks(L, S, B):
    """Boolean (Bm, Lm, S) masks by name: the patterns, near misses, and masks that are none."""
    g = torch.Generator().manual_seed(L + S)
    tril = torch.tril(torch.ones(L, S, dtype=torch.bool))
    lens = torch.randint(1, S + 1, (B,), generator=g)
    lens[0] = S
    pad = (torch.arange(S)[None] < lens[:, None])[:, None, :]
    holed = (tril[None] & pad).clone()
    holed[B - 1, L // 2, 0] = False
    return {
        "all": torch.ones(1, L, S, dtype=torch.bool),
        "causal": tril[None],
        "padding": pad.expand(B, L, S),
        "padding_one_row": pad,
        "causal_padding": tril[None] & pad,
        "window": om.window_keep_mask(L, S, max(L // 4, 1), 0)[None],
        "window_sinks": om.window_keep_mask(L, S, max(L // 4, 2), 2)[None],
        "window_padding": om.window_keep_mask(L, S, max(L // 4, 1), 0)[None] & pad,
        "window_sinks_padding": om.window_keep_mask(L, S, max(L // 5, 2), 3)[None] & pad,
        "window_padding_holed": _holed(om.window_keep_mask(L, S, max(L // 4, 1), 0)[None] & pad, B - 1),
        "left_padding": (torch.arange(S)[None] >= (S - lens)[:, None])[:, None, :].expand(B, L, S),
        "random": (torch.rand(1, L, S, generator=g) < 0.5),
        "holed": holed,
        "upper": torch.triu(torch.ones(L, S, dtype=torch.bool))[None],
        "nothing": torch.zeros(1, L, S, dtype=torch.bool),
    }


def _expected_verdict(keep3: torch.Tensor, B: int, L: int):
    """(kind, window, sink keys, lens) by the host rules on brute-force row summaries."""
    from torch_neuronx_amd.mask_patterns import lens_pattern_from_rows, window_lens_pattern_from_rows

    Bm, Lm, S = keep3.shape
    rows = np.stack([rows_of(m.numpy()) for m in keep3])
    pat = lens_pattern_from_rows(rows, L, S, rows_broadcast=Lm == 1 and L > 1)
    if pat is not None:
        lens = np.broadcast_to(pat[1], (B,)) if Bm == 1 else pat[1]
        return (1 if pat[0] == "all" else 2), 0, 0, [int(x) for x in lens]
    if Lm == L and L > 1 and (rows[:, :, 1] >= 0).all():
        pat = window_lens_pattern_from_rows(rows, L, S)
        if pat is not None:
            lens = np.broadcast_to(pat[3], (B,)) if Bm == 1 else pat[3]
            return 3, pat[1], pat[2], [int(x) for x in lens]
    return 0, 0, 0, [S] * B


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [torch.bool, torch.bfloat16, torch.float32])
@pytest.mark.parametrize("L,S", [(64, 64), (37, 203), (200, 96), (1, 50), (300, 300)])
def test_device_verdict_follows_the_host_rules(amd, gpu_device, dtype, L, S):
    B, Hq = 3, 2
    for name, keep in _keep_masks(L, S, B).items():
        m = keep if dtype is torch.bool else torch.zeros(keep.shape, dtype=dtype).masked_fill(~keep, float("-inf"))
        md = m.to(gpu_device)[:, None]  # (Bm, 1, Lm, S)
        v = amd.ops.mask_verdict(md, B, Hq, L, S)
        assert v is not None, name
        got = v.cpu().tolist()
        kind, window, sinks, lens = _expected_verdict(keep, B, L)
        assert got[0] == kind and got[1] == window and got[2] == sinks, (name, got[:4], (kind, window, sinks))
        assert got[8:8 + B] == lens and got[3] == int(any(n != S for n in lens)), (name, got[:8 + B], lens)
    if dtype is not torch.bool:  # one real bias value: not a mask
        m = torch.zeros(1, 1, L, S, dtype=dtype)
        m[0, 0, L // 2, S // 3] = 0.5
        assert amd.ops.mask_verdict(m.to(gpu_device), B, Hq, L, S)[0].item() == 0
    # a mask that depends on the head, or whose keys are strided, has no verdict
    assert amd.ops.mask_verdict(torch.ones(1, Hq, L, S, dtype=torch.bool, device=gpu_device), B, Hq, L, S) is None
    if S > 1:
        assert amd.ops.mask_verdict(torch.ones(1, 1, L, 2 * S, dtype=torch.bool, device=gpu_device)[..., ::2], B, Hq, L, S) is None


@pytest.mark.gpu
@pytest.mark.parametrize("D", [64, 128])
@pytest.mark.parametrize("name", ["causal", "causal_padding", "padding", "all", "random", "window", "holed",
                                  "window_sinks", "window_padding", "window_sinks_padding", "window_padding_holed"])
def test_calls_with_a_verdict_equal_the_calls_they_stand_for(amd, gpu_device, name, D):
    # forward and backward through the C ABI with mask + verdict, against the same call with the flag and
    # key counts (for a pattern) or with the mask alone (for anything else): the same kernels, bit for bit
    dev = gpu_device
    B, Hq, Hkv, L = 3, 4, 2, 640
    q, k, v, go = (t.to(dev) for t in qkv(B, Hq, Hkv, L, L, D, dtype=torch.bfloat16, seed=len(name), with_do=True))
    keep = _keep_masks(L, L, B)[name]
    md = keep.to(dev)[:, None]
    verdict = amd.ops.mask_verdict(md, B, Hq, L, L)
    kind, window, sinks, lens = _expected_verdict(keep, B, L)
    assert (kind == 3) == (name.startswith("window") and not name.endswith("holed"))
    out, lse = amd.sdpa_forward(q, k, v, attn_bias=md, mask_verdict=verdict, force_kernel=amd._lib.KERNEL_MFMA)
    grads = amd.sdpa_backward(go, q, k, v, out, lse, attn_bias=md, mask_verdict=verdict, force_kernel=amd._lib.KERNEL_MFMA)[:3]
    if kind in (1, 2):
        kw = dict(is_causal=kind == 2, kv_lens=torch.tensor(lens, dtype=torch.int32, device=dev))
    elif kind == 3:
        kw = dict(is_causal=True, window=window, sink_keys=sinks, kv_lens=torch.tensor(lens, dtype=torch.int32, device=dev))
    else:
        kw = dict(attn_bias=md)
    ro, rl = amd.sdpa_forward(q, k, v, **kw)
    rg = amd.sdpa_backward(go, q, k, v, ro, rl, **kw)[:3]
    # (the variant with a bias and the one with key counts are different instantiations of one kernel: the
    # forward does the same arithmetic in the same order; the dK/dV kernel folds the bias slot into the
    # exponent's multiply-add, which rounds differently in the last place)
    assert max_abs(out, ro) <= 1e-6 and max_abs(lse, rl) <= 1e-6, name
    for a, b in zip(grads, rg):
        assert max_abs(a, b) <= 8e-3 * max(1.0, b.abs().max().item()) and rel_err(a, b) <= 2e-3, name
    # ... and the oracle on the explicit mask
    keep4 = keep[:, None].expand(B, 1, keep.shape[1], L) if keep.shape[0] == B else keep[None].expand(B, 1, keep.shape[1], L)
    oo, ol = om.sdpa_forward(q.float().cpu(), k.float().cpu(), v.float().cpu(), attn_mask=keep4)
    assert max_abs(out, oo) <= 2e-2 and max_abs(lse, ol) <= 5e-3


@pytest.mark.gpu
@pytest.mark.parametrize("pdrop", [0.0, 0.2])
@pytest.mark.parametrize("name", ["padding_one_row", "padding", "causal_padding", "all", "random", "window_padding"])
def test_verdicts_for_masks_per_key_and_for_calls_with_dropout(amd, gpu_device, name, pdrop):
    """A `(B,1,1,S)` key-padding mask (one row for every query) takes its verdict too, and so do calls with
    dropout: forward and backward with mask + verdict (+ keep-mask) equal the calls with key counts (for
    keep-everything and causal patterns; a window has no dropout variant and stays a mask) and agree with
    the oracle on the explicit mask."""
    dev = gpu_device
    B, Hq, Hkv, L, D = 3, 4, 2, 640, 64
    q, k, v, go = (t.to(dev) for t in qkv(B, Hq, Hkv, L, L, D, dtype=torch.bfloat16, seed=len(name) + 3, with_do=True))
    keep = _keep_masks(L, L, B)[name]  # (Bm, Lm, S)
    md = torch.where(keep, 0.0, float("-inf")).to(torch.bfloat16).to(dev)[:, None]
    verdict = amd.ops.mask_verdict(md, B, Hq, L, L)
    kind, _, _, lens = _expected_verdict(keep, B, L)
    MFMA = amd._lib.KERNEL_MFMA
    drop = {}
    dk_cpu = None
    if pdrop:
        dk_cpu = torch.rand(B, Hq, L, L, generator=torch.Generator().manual_seed(5)) >= pdrop
        drop = dict(dropout_p=pdrop, dropout_keep=dk_cpu.to(dev))
    out, lse = amd.sdpa_forward(q, k, v, attn_bias=md, mask_verdict=verdict, force_kernel=MFMA, **drop)
    grads = amd.sdpa_backward(go, q, k, v, out, lse, attn_bias=md, mask_verdict=verdict, force_kernel=MFMA, **drop)[:3]
    if kind in (1, 2):
        kw = dict(is_causal=kind == 2, kv_lens=torch.tensor(lens, dtype=torch.int32, device=dev))
    else:
        assert kind == 0 or (kind == 3 and name == "window_padding")
        kw = dict(attn_bias=md)
    ro, rl = amd.sdpa_forward(q, k, v, force_kernel=MFMA, **kw, **drop)
    rg = amd.sdpa_backward(go, q, k, v, ro, rl, force_kernel=MFMA, **kw, **drop)[:3]
    if kind == 3 and not pdrop:  # (without dropout the window verdict is used: compared with the functor call elsewhere)
        pass
    else:
        assert max_abs(out, ro) <= 1e-6 and max_abs(lse, rl) <= 1e-6, name
        for a, b_ in zip(grads, rg):
            assert max_abs(a, b_) <= 8e-3 * max(1.0, b_.abs().max().item()) and rel_err(a, b_) <= 2e-3, name
    keep4 = keep[:, None].expand(keep.shape[0], 1, keep.shape[1], L).expand(B, 1, keep.shape[1], L).expand(B, Hq, L, L)
    bias = torch.where(keep4, 0.0, float("-inf"))
    rep = Hq // Hkv
    qc, gc = q.float().cpu(), go.float().cpu()
    kc, vc = k.float().cpu().repeat_interleave(rep, 1), v.float().cpu().repeat_interleave(rep, 1)
    oo, ol = om.compute_attention(qc, kc, vc, bias, dk_cpu, D**-0.5, False, pdrop)
    live = torch.isfinite(ol)
    assert max_abs(out, oo) <= 2e-2 and max_abs(lse.cpu()[live], ol[live]) <= 5e-3
    odq, odk, odv, _ = om.compute_attention_backward(gc, qc, kc, vc, bias, dk_cpu, oo, ol, D**-0.5, False, pdrop)
    odk, odv = odk.view(B, Hkv, rep, L, D).sum(2), odv.view(B, Hkv, rep, L, D).sum(2)
    for a, b_ in zip(grads, (odq, odk, odv)):
        assert max_abs(a, b_) <= 5e-2 * max(1.0, b_.abs().max().item()) and rel_err(a, b_) <= 3e-2, name


@pytest.mark.gpu
def test_fresh_bool_masks_run_at_the_speed_of_the_causal_flag(amd, gpu_device):
    # F.scaled_dot_product_attention(attn_mask=bool) hands the op a new additive tensor on every call: no
    # cache can know it, the verdict on the device does.  Ten calls in a row, against is_causal=True:
    # measured 1.11 to 1.15 times its time, of which upstream's own conversion of the bool mask is a
    # third (a mask that is read costs 2.4 times); the bound leaves room for the box and the allocator.
    dev = gpu_device
    B, H, L, D = 4, 32, 4096, 128
    q, k, v = (torch.randn(B, H, L, D, device=dev, dtype=torch.bfloat16) for _ in range(3))
    tril = torch.ones(L, L, dtype=torch.bool, device=dev).tril()
    amd.mask_patterns.clear_cache()
    with torch.no_grad():
        ref = F.scaled_dot_product_attention(q, k, v, is_causal=True)
        got = F.scaled_dot_product_attention(q, k, v, attn_mask=tril)
        assert max_abs(got, ref) <= 4e-3
        ok, seen = _within(lambda: F.scaled_dot_product_attention(q, k, v, attn_mask=tril),
                           lambda: F.scaled_dot_product_attention(q, k, v, is_causal=True), 1.2)
    assert ok, seen


@pytest.mark.gpu
def test_training_steps_with_a_mask_that_is_new_every_step(amd, gpu_device, monkeypatch):
    # forward and backward through autograd with a bool mask: upstream makes a new additive tensor per
    # step, the forward takes its verdict on the device, and the backward of the same step finds that
    # verdict again instead of reading the mask a second time; after a few steps no copy to the host either
    dev = gpu_device
    B, H, L, D = 2, 8, 1024, 64
    q, k, v, go = (t.to(dev) for t in qkv(B, H, H, L, L, D, dtype=torch.bfloat16, seed=9, with_do=True))
    tril = torch.ones(L, L, dtype=torch.bool, device=dev).tril()
    seen_b = []
    b0 = amd.ops.sdpa_backward
    monkeypatch.setattr(amd.ops, "sdpa_backward", lambda *a, **kw: (seen_b.append(kw), b0(*a, **kw))[1])
    qc, kc, vc = (t.clone().requires_grad_(True) for t in (q, k, v))
    F.scaled_dot_product_attention(qc, kc, vc, is_causal=True).backward(go)
    amd.mask_patterns.clear_cache()
    looked0, launched = amd.mask_patterns.stats["looked"], []
    real = amd.mask_patterns._launch_verdict
    monkeypatch.setattr(amd.mask_patterns, "_launch_verdict", lambda *a: (launched.append(1), real(*a))[1])
    for step in range(6):
        qm, km, vm = (t.clone().requires_grad_(True) for t in (q, k, v))
        F.scaled_dot_product_attention(qm, km, vm, attn_mask=tril).backward(go)
        kw = seen_b[-1]  # (the verdict on the device, or - its copy has arrived meanwhile - the pattern itself)
        assert kw.get("mask_verdict") is not None or (kw["attn_bias"] is None and kw["is_causal"])
        for a, b in ((qm.grad, qc.grad), (km.grad, kc.grad), (vm.grad, vc.grad)):
            assert max_abs(a, b) <= 2e-2 and rel_err(a, b) <= 5e-3
    assert len(launched) == 6  # one verdict per step: the backward reuses the forward's
    assert amd.mask_patterns.stats["looked"] - looked0 == 3  # ... and a copy to the host for the first three only


@pytest.mark.gpu
def test_a_verdict_found_from_another_stream_is_waited_for(amd, gpu_device):
    # two independent calls with one mask tensor on two streams: the second finds the first one's
    # verdict still on its way and must not read it before the first stream has written it
    dev = gpu_device
    B, H, L, D = 1, 8, 1024, 64
    q, k, v = (t.to(dev) for t in qkv(B, H, H, L, L, D, dtype=torch.bfloat16, seed=21))
    ref = F.scaled_dot_product_attention(q, k, v, is_causal=True)
    s1, s2 = torch.cuda.Stream(), torch.cuda.Stream()
    torch.cuda.synchronize()
    for make in (lambda: torch.ones(L, L, dtype=torch.bool, device=dev).tril(),                                  # the host copy is made
                 lambda: torch.where(torch.ones(L, L, dtype=torch.bool, device=dev).tril(), 0.0, float("-inf")).to(torch.bfloat16)):  # ... and when it is not
        for rounds in range(5 if make().dtype != torch.bool else 1):  # (the float mask: until its signature is left without a host copy)
            mask = make()
            torch.cuda.synchronize()
            with torch.cuda.stream(s1):
                o1 = F.scaled_dot_product_attention(q, k, v, attn_mask=mask)
            with torch.cuda.stream(s2):
                o2 = F.scaled_dot_product_attention(q, k, v, attn_mask=mask)
            torch.cuda.synchronize()
            assert max_abs(o1, ref) <= 1e-6 and max_abs(o2, ref) <= 1e-6


@pytest.mark.gpu
def test_a_captured_call_takes_its_verdict_on_every_replay(amd, gpu_device):
    # inside a stream capture nothing is cached and nothing waits: the verdict is part of the graph, so a
    # replay follows the mask as it then is - causal at the causal kernel's speed, anything else as a mask
    dev = gpu_device
    B, H, L, D = 4, 32, 4096, 128
    q, k, v = (torch.randn(B, H, L, D, device=dev, dtype=torch.bfloat16) for _ in range(3))
    tril = torch.ones(L, L, dtype=torch.bool, device=dev).tril()
    mask = torch.zeros(1, 1, L, L, device=dev, dtype=torch.bfloat16).masked_fill(~tril, float("-inf"))
    fused = torch.ops.aten._scaled_dot_product_fused_attention_overrideable
    amd.mask_patterns.clear_cache()
    with torch.no_grad():
        ref_c = fused(q, k, v, None, 0.0, True)[0]
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            fused(q, k, v, mask)  # (warm-up outside the capture, as captures want it)
        torch.cuda.current_stream().wait_stream(side)
        torch.cuda.synchronize()
        amd.mask_patterns.clear_cache()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            out = fused(q, k, v, mask)[0]
        graph.replay()
        torch.cuda.synchronize()
        assert max_abs(out, ref_c) <= 4e-3
        # the mask changes in place, by something no version counter sees from inside the graph
        g = torch.Generator(device="cpu").manual_seed(5)
        rnd = (torch.rand(L, L, generator=g) < 0.7) | torch.eye(L, dtype=torch.bool)
        mask.copy_(torch.zeros(L, L, dtype=torch.bfloat16).masked_fill(~rnd, float("-inf")).to(dev))
        graph.replay()
        torch.cuda.synchronize()
        with amd.mask_patterns.left_alone():
            ref_r = fused(q, k, v, mask)[0]
        assert max_abs(out, ref_r) <= 1e-6 and not max_abs(out, ref_c) <= 4e-3
        # ... and back, with right padding folded in
        pad = tril.clone()
        pad[:, 3000:] = False
        mask.copy_(torch.zeros(L, L, dtype=torch.bfloat16, device=dev).masked_fill(~pad, float("-inf")))
        graph.replay()
        torch.cuda.synchronize()
        ref_p = fused(q[:, :, :, :], k[:, :, :3000], v[:, :, :3000], None, 0.0, True)[0]
        assert max_abs(out, ref_p) <= 4e-3
        # eager work and synchronisations between replays; every replay checked, and timed against the flag
        mask.copy_(torch.zeros(L, L, dtype=torch.bfloat16, device=dev).masked_fill(~tril, float("-inf")))
        for _ in range(3):
            graph.replay()
            torch.cuda.synchronize()
            assert max_abs(out, ref_c) <= 4e-3
        ok, seen_t = _within(graph.replay, lambda: fused(q, k, v, None, 0.0, True), 1.15)
    assert ok, seen_t


@pytest.mark.gpu
def test_sliding_window_mask_takes_the_window_kernel(amd, gpu_device, monkeypatch):
    dev = gpu_device
    B, Hq, Hkv, L, D, W = 1, 4, 4, 4096, 128, 1024
    q, k, v, go = qkv(B, Hq, Hkv, L, L, D, dtype=torch.bfloat16, seed=4, with_do=True)
    keep = om.window_keep_mask(L, L, W)
    maskd = keep.to(dev)[None, None]
    maskd = torch.zeros(L, L, dtype=torch.bfloat16, device=dev).masked_fill(~maskd[0, 0], float("-inf"))  # kept by the caller
    amd.mask_patterns.clear_cache()
    seen = []
    f0 = amd.ops.sdpa_forward
    monkeypatch.setattr(amd.ops, "sdpa_forward", lambda *a, **kw: (seen.append(kw), f0(*a, **kw))[1])
    qd, kd, vd = (t.to(dev).requires_grad_(True) for t in (q, k, v))
    with torch.no_grad():  # first sight: the verdict's copy is on its way to the host; the calls below find it
        F.scaled_dot_product_attention(qd, kd, vd, attn_mask=maskd)
    torch.cuda.synchronize()
    out = F.scaled_dot_product_attention(qd, kd, vd, attn_mask=maskd)
    out.backward(go.to(dev))
    assert seen[-1]["attn_bias"] is None and seen[-1]["is_causal"] is True and seen[-1]["window"] == W
    # parity with the oracle on the explicit mask, forward and backward (head subset: the oracle is a CPU program)
    hs = slice(0, 2)
    ro, rl = om.sdpa_forward(q[:, hs].float(), k[:, hs].float(), v[:, hs].float(), attn_mask=keep)
    assert max_abs(out[:, hs], ro) <= 2e-2
    rdq, rdk, rdv = om.sdpa_backward(go[:, hs].float(), q[:, hs].float(), k[:, hs].float(), v[:, hs].float(), ro, rl,
                                     attn_mask=keep, reduce_in_fp32=True)
    assert max_abs(qd.grad[:, hs], rdq) <= 5e-2 and rel_err(qd.grad[:, hs], rdq) <= 3e-2
    assert rel_err(kd.grad[:, hs], rdk) <= 3e-2 and rel_err(vd.grad[:, hs], rdv) <= 3e-2
    # rate on the scores the window keeps
    Bp = 4
    qb, kb, vb = (torch.randn(Bp, 32, L, D, device=dev, dtype=torch.bfloat16) for _ in range(3))
    with torch.no_grad():
        ms = _best_ms(lambda: F.scaled_dot_product_attention(qb, kb, vb, attn_mask=maskd))
    live = int(keep.sum())
    tflops = 4.0 * Bp * 32 * D * live / (ms * 1e-3) / 1e12
    assert tflops >= 600.0, tflops


@pytest.mark.gpu
def test_sliding_window_mask_at_head_dim_256_takes_the_window_kernels(amd, gpu_device, monkeypatch):
    """Head dims above 128 have the window functor in their matrix-op kernels too (the forward's functor
    variant at width 256, the wide backward kernels' functor mode): a recognised window mask becomes the
    functor there as well, forward and backward, and never reaches the generic kernels."""
    dev = gpu_device
    B, H, L, D, W = 1, 2, 1024, 256, 256
    q, k, v, go = qkv(B, H, H, L, L, D, dtype=torch.bfloat16, seed=6, with_do=True)
    keep = om.window_keep_mask(L, L, W)
    maskd = torch.zeros(L, L, dtype=torch.bfloat16, device=dev).masked_fill(~keep.to(dev), float("-inf"))
    amd.mask_patterns.clear_cache()
    seen, seen_b = [], []
    f0, b0 = amd.ops.sdpa_forward, amd.ops.sdpa_backward
    MFMA = amd._lib.KERNEL_MFMA  # forced: the call fails if the matrix-op kernels cannot take it
    monkeypatch.setattr(amd.ops, "sdpa_forward", lambda *a, **kw: (seen.append(kw), f0(*a, **{**kw, "force_kernel": MFMA}))[1])
    monkeypatch.setattr(amd.ops, "sdpa_backward", lambda *a, **kw: (seen_b.append(kw), b0(*a, **{**kw, "force_kernel": MFMA}))[1])
    qd, kd, vd = (t.to(dev).requires_grad_(True) for t in (q, k, v))
    with torch.no_grad():  # first sight: the verdict's copy is on its way to the host; the calls below find it
        F.scaled_dot_product_attention(qd, kd, vd, attn_mask=maskd)
    torch.cuda.synchronize()
    assert amd.mask_patterns.classify(maskd) == ("window", W, 0)
    out = F.scaled_dot_product_attention(qd, kd, vd, attn_mask=maskd)
    out.backward(go.to(dev))
    for kw in (seen[-1], seen_b[-1]):
        assert kw["attn_bias"] is None and kw["is_causal"] is True and kw["window"] == W
    ro, rl = om.sdpa_forward(q.float(), k.float(), v.float(), attn_mask=keep)
    assert max_abs(out, ro) <= 2e-2
    rdq, rdk, rdv = om.sdpa_backward(go.float(), q.float(), k.float(), v.float(), ro, rl, attn_mask=keep, reduce_in_fp32=True)
    assert rel_err(qd.grad, rdq) <= 3e-2 and rel_err(kd.grad, rdk) <= 3e-2 and rel_err(vd.grad, rdv) <= 3e-2


@pytest.mark.gpu
@pytest.mark.parametrize("D", [128, 256])
def test_sliding_window_and_padding_mask_becomes_the_window_with_key_counts(amd, gpu_device, monkeypatch, D):
    """The (B,1,L,S) mask that the code of a sliding-window model builds from a right-padded batch
    (causal & window & key < len[b]).  A new tensor per forward pass, as that code makes them: the calls
    carry the verdict and run the window kernels with key counts (eight layers that share one new mask:
    measured 1.33x the time of eight functor calls at head dim 128 - the one pass over the 128 MB of
    mask, the second kernel of each pair, and workgroups sized without knowing the window - and bounded
    by 1.5x; as a bias each layer takes more than twice as long).  A tensor the caller keeps: once the
    verdict has reached the host, the functor call itself, forward and backward.  Both against the oracle
    on the explicit mask."""
    dev = gpu_device
    B, H, L, W = 3, 4, 2048, 256
    q, k, v, go = (t.to(dev) for t in qkv(B, H, H, L, L, D, dtype=torch.bfloat16, seed=8, with_do=True))
    lens = torch.tensor([L, 1300, 77])
    keep = om.window_keep_mask(L, L, W)[None, None] & (torch.arange(L)[None] < lens[:, None])[:, None, None, :]
    amd.mask_patterns.clear_cache()
    seen = []
    f0, b0 = amd.ops.sdpa_forward, amd.ops.sdpa_backward
    MFMA = amd._lib.KERNEL_MFMA  # forced: the call fails if the matrix-op kernels cannot take it
    monkeypatch.setattr(amd.ops, "sdpa_forward", lambda *a, **kw: (seen.append(kw), f0(*a, **{**kw, "force_kernel": MFMA}))[1])
    monkeypatch.setattr(amd.ops, "sdpa_backward", lambda *a, **kw: (seen.append(kw), b0(*a, **{**kw, "force_kernel": MFMA}))[1])
    fused = torch.ops.aten._scaled_dot_product_fused_attention_overrideable
    fused_bwd = torch.ops.aten._scaled_dot_product_fused_attention_overrideable_backward
    qc, kc, vc, gc = (t.float().cpu() for t in (q, k, v, go))
    ro, rl = om.sdpa_forward(qc, kc, vc, attn_mask=keep)
    rg = om.sdpa_backward(gc, qc, kc, vc, ro, rl, attn_mask=keep, reduce_in_fp32=True)

    def check(r, grads):
        assert max_abs(r[0], ro) <= 2e-2 and max_abs(r[1], rl) <= 5e-3
        for a, b_ in zip(grads[:3], rg):
            assert rel_err(a, b_) <= 3e-2 and max_abs(a, b_) <= 5e-2 * max(1.0, float(b_.abs().max()))

    fresh = lambda: torch.where(keep, 0.0, float("-inf")).to(torch.bfloat16).to(dev)
    if D == 128:  # (the verdict on the device serves head dims up to 128 in the backward)
        mask = fresh()
        r = fused(q, k, v, mask)
        grads = fused_bwd(go, q, k, v, mask, [True, True, True, False], r[0], r[1], None, None, L, L, 0.0, False, r[6], r[7])
        assert seen[0]["attn_bias"] is not None and seen[0].get("mask_verdict") is not None
        # (the backward carries the verdict too, unless its copy has reached the host by then)
        assert seen[1].get("mask_verdict") is not None or (seen[1]["attn_bias"] is None and seen[1]["window"] == W)
        v0 = seen[0]["mask_verdict"].cpu().tolist()
        assert v0[:4] == [3, W, 0, 1] and v0[8:8 + B] == lens.tolist()
        check(r, grads)
        # time, at a size where the kernels and not the host set it: new masks against the functor call
        Bt, Ht, Lt, Wt = 4, 16, 4096, 512
        qt, kt, vt = (torch.randn(Bt, Ht, Lt, D, device=dev, dtype=torch.bfloat16) for _ in range(3))
        lens_t = torch.tensor([Lt, 3000, 2000, 500])
        keep_t = (om.window_keep_mask(Lt, Lt, Wt)[None, None] & (torch.arange(Lt)[None] < lens_t[:, None])[:, None, None, :]).to(dev)
        mask_t = torch.where(keep_t, 0.0, float("-inf")).to(torch.bfloat16)
        kv = lens_t.to(torch.int32).to(dev)

        def layers_with_a_new_mask():  # (what a model's forward pass does: one new mask, used by every layer)
            amd.mask_patterns.clear_cache()
            for _ in range(8):
                fused(qt, kt, vt, mask_t)

        def layers_with_the_functor():
            for _ in range(8):
                amd.sdpa_forward(qt, kt, vt, is_causal=True, window=Wt, kv_lens=kv)

        with torch.no_grad():
            ok, seen_t = _within(layers_with_a_new_mask, layers_with_the_functor, 1.5)
        assert ok, seen_t
    # a mask the caller keeps: the host learns the pattern and makes the functor call
    mask = fresh()
    amd.mask_patterns.clear_cache()
    with torch.no_grad():
        fused(q, k, v, mask)
    torch.cuda.synchronize()
    pat = amd.mask_patterns.classify(mask)
    assert pat[:3] == ("window", W, 0) and pat[3].cpu().tolist() == lens.tolist()
    del seen[:]
    r = fused(q, k, v, mask)
    grads = fused_bwd(go, q, k, v, mask, [True, True, True, False], r[0], r[1], None, None, L, L, 0.0, False, r[6], r[7])
    for kw in seen:
        assert kw["attn_bias"] is None and kw["is_causal"] is True and kw["window"] == W and kw["kv_lens"].cpu().tolist() == lens.tolist()
    check(r, grads)


@pytest.mark.gpu
@pytest.mark.parametrize("D", [128, 256])
def test_causal_and_padding_mask_becomes_causal_with_key_counts(amd, gpu_device, monkeypatch, D):
    # the additive (B,1,L,S) mask that model code builds from causality and right padding: served by the
    # causal kernels with per-batch key counts, no mask read, forward and backward
    dev = gpu_device
    B, H, L = 3, 4, 1024
    q, k, v, go = (t.to(dev) for t in qkv(B, H, H, L, L, D, dtype=torch.bfloat16, seed=4, with_do=True))
    lens = torch.tensor([L, 600, 131])
    keep = torch.tril(torch.ones(L, L, dtype=torch.bool))[None, None] & (torch.arange(L)[None] < lens[:, None])[:, None, None, :]
    mask = torch.where(keep, 0.0, float("-inf")).to(torch.bfloat16).to(dev)
    amd.mask_patterns.clear_cache()
    seen = []
    f0, b0 = amd.ops.sdpa_forward, amd.ops.sdpa_backward
    monkeypatch.setattr(amd.ops, "sdpa_forward", lambda *a, **kw: (seen.append(kw), f0(*a, **kw))[1])
    monkeypatch.setattr(amd.ops, "sdpa_backward", lambda *a, **kw: (seen.append(kw), b0(*a, **kw))[1])
    fused = torch.ops.aten._scaled_dot_product_fused_attention_overrideable
    fused_bwd = torch.ops.aten._scaled_dot_product_fused_attention_overrideable_backward
    r = fused(q, k, v, mask)  # first sight: mask and verdict
    assert seen[-1]["attn_bias"] is not None and seen[-1].get("mask_verdict") is not None
    ro, rl = om.sdpa_forward(q.float().cpu(), k.float().cpu(), v.float().cpu(), attn_mask=keep)
    assert max_abs(r[0], ro) <= 2e-2 and max_abs(r[1], rl) <= 5e-3
    torch.cuda.synchronize()
    r = fused(q, k, v, mask)  # ... and once its copy has arrived
    assert seen[-1]["attn_bias"] is None and seen[-1]["is_causal"] is True and seen[-1]["kv_lens"].tolist() == [L, 600, 131]
    g = fused_bwd(go, q, k, v, mask, [True, True, True, False], r[0], r[1], None, None, L, L, 0.0, False, r[6], r[7])
    assert seen[-1]["attn_bias"] is None and seen[-1]["kv_lens"].tolist() == [L, 600, 131]
    rg = om.sdpa_backward(go.float().cpu(), q.float().cpu(), k.float().cpu(), v.float().cpu(), ro, rl, attn_mask=keep, reduce_in_fp32=True)
    assert max_abs(r[0], ro) <= 2e-2 and max_abs(r[1], rl) <= 5e-3
    for a, b_ in zip(g[:3], rg[:3]):
        assert max_abs(a, b_) <= 5e-2 and rel_err(a, b_) <= 2e-2
    # padding alone, as a bool (B,1,1,S) mask: key counts without the causal flag
    pad = (torch.arange(L)[None] < lens[:, None])[:, None, None, :].to(dev)
    fused(q, k, v, pad)
    torch.cuda.synchronize()
    r2 = fused(q, k, v, pad)
    assert seen[-1]["attn_bias"] is None and seen[-1]["is_causal"] is False and seen[-1]["kv_lens"].tolist() == [L, 600, 131]
    ro2, _ = om.sdpa_forward(q.float().cpu(), k.float().cpu(), v.float().cpu(), attn_mask=pad.cpu())
    assert max_abs(r2[0], ro2) <= 2e-2
    # left padding is no key count: the mask stays a mask
    left = (torch.arange(L)[None] >= (L - lens)[:, None])[:, None, None, :].to(dev)
    fused(q, k, v, left)
    assert seen[-1]["attn_bias"] is not None
