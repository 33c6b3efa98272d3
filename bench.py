#!/usr/bin/env python3
"""Benchmark of the fused SDPA hot path on one MI355X.

    python bench.py --gpus 1 --steps K --warmup W [--workload c3_fwd|c4_fwd_bwd|c5_decode|c2_fwd|masked_fwd|mqa_fwd_bwd]

A step is one pass of the hot path over one batch of synthetic input that is already resident
in HBM.  The default workload is the one the headline metric is quoted on: causal GQA bf16
forward at the Llama-3-8B layer shape (B=1, Hq=32, Hkv=8, S=8192, D=128).  One JSON line is
printed; `roofline` is for the dominant kernel of the workload (kernel time from HIP events on
the launch stream), `cpu_baseline` is the CPU oracle timed on a bounded sample of the same
workload on this box's host cores, `extras` carries the other workloads of the metric.

Before the W warmup steps the workload runs untimed for 0.3 s so that the GPU's clocks have
settled; the K timed steps are bracketed by torch.cuda.synchronize() on both sides.
"""

from __future__ import annotations

import argparse
import json
import math
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
for _p in (ROOT, os.path.join(ROOT, "torch-neuronx_amd")):
    if _p not in sys.path:
        sys.path.insert(0, _p)

import torch  # noqa: E402

PEAK_BF16_TFLOPS = 2500.0  # MI355X dense bf16 MFMA
PEAK_HBM_GBS = 8000.0      # MI355X HBM3E

METRIC = "SDPA fwd/bwd TFLOP/s & % MFMA peak (Llama-3-8B shape); fp8-KV decode HBM GB/s"


def causal_pairs(L, S):
    """Number of (query, key) pairs a top-left causal mask keeps."""
    return sum(min(i + 1, S) for i in range(L)) if L != S else L * (L + 1) // 2


def seeded(shapes, seed, dtype, dev):
    g = torch.Generator(device="cpu").manual_seed(seed)
    return [torch.randn(s, generator=g).to(dtype).to(dev) for s in shapes]


def spin_up(fn, seconds=0.3):
    """Untimed load before the warmup steps: the GPU's clocks climb over the first tens of
    milliseconds of work (the same kernel runs ~25 % slower right after idle), and a handful of
    warmup launches of a sub-millisecond kernel does not get there."""
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    while time.perf_counter() - t0 < seconds:
        for _ in range(10):
            fn()
        torch.cuda.synchronize()


SPIN = True


def event_time_ms(fn, steps, warmup):
    """Run warmup + steps launches; returns (wall ms per step, event ms per step)."""
    if SPIN:
        spin_up(fn)
    for _ in range(warmup):
        fn()
    torch.cuda.synchronize()
    start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    t0 = time.perf_counter()
    start.record()
    for _ in range(steps):
        fn()
    stop.record()
    torch.cuda.synchronize()
    wall = (time.perf_counter() - t0) * 1e3 / steps
    return wall, start.elapsed_time(stop) / steps


# ------------------------------------------------------------------------------------------
# workloads
# ------------------------------------------------------------------------------------------


def wl_fwd(amd, dev, B, Hq, Hkv, S, D, seed, name):
    q, k, v = seeded([(B, Hq, S, D), (B, Hkv, S, D), (B, Hkv, S, D)], seed, torch.bfloat16, dev)
    flops = 4.0 * B * Hq * D * causal_pairs(S, S)
    nbytes = 2.0 * (2 * B * Hq * S * D + 2 * B * Hkv * S * D) + 4.0 * B * Hq * S

    def step():
        amd.sdpa_forward(q, k, v, is_causal=True)

    cfg = {"workload": name, "B": B, "Hq": Hq, "Hkv": Hkv, "S": S, "D": D, "causal": True,
           "algorithmic_flops": flops, "dense_convention_flops": 4.0 * B * Hq * S * S * D,
           "algorithmic_bytes": nbytes}
    return step, flops, cfg, (q, k, v)


def wl_masked_fwd(amd, dev):
    """Forward with an additive bias shared by batch and heads (relative-position style),
    B=4 Hq=32 Hkv=8 L=S=4096 D=128 bf16, non-causal: the path the reference leaves to its
    unfused implementation whenever a mask is present (decompositions.py:2203)."""
    B, Hq, Hkv, S, D = 4, 32, 8, 4096, 128
    q, k, v = seeded([(B, Hq, S, D), (B, Hkv, S, D), (B, Hkv, S, D)], 1006, torch.bfloat16, dev)
    bias = torch.randn(1, 1, S, S, generator=torch.Generator().manual_seed(1007)).to(torch.bfloat16).to(dev)
    flops = 4.0 * B * Hq * D * S * S
    nbytes = 2.0 * (2 * B * Hq * S * D + 2 * B * Hkv * S * D) + 4.0 * B * Hq * S + 2.0 * S * S

    def step():
        amd.sdpa_forward(q, k, v, attn_bias=bias)

    cfg = {"workload": "masked_noncausal_gqa_bf16_fwd_shared_bias", "B": B, "Hq": Hq, "Hkv": Hkv, "S": S, "D": D,
           "causal": False, "bias": "(1,1,L,S) bf16", "algorithmic_flops": flops, "algorithmic_bytes": nbytes}
    return step, flops, cfg


def wl_fwd_bwd(amd, dev, Hkv=8):
    B, Hq, S, D = 2, 32, 4096, 128
    q, k, v, do = seeded([(B, Hq, S, D), (B, Hkv, S, D), (B, Hkv, S, D), (B, Hq, S, D)], 1004,
                         torch.bfloat16, dev)
    pairs = causal_pairs(S, S)
    f_fwd, f_bwd = 4.0 * B * Hq * D * pairs, 10.0 * B * Hq * D * pairs
    out, lse = amd.sdpa_forward(q, k, v, is_causal=True)

    def step_fwd():
        amd.sdpa_forward(q, k, v, is_causal=True)

    def step_bwd():
        amd.sdpa_backward(do, q, k, v, out, lse, is_causal=True)

    return step_fwd, step_bwd, f_fwd, f_bwd


def wl_decode(amd, dev, sets=4):
    """Config 5.  `sets` rotating copies of the cache keep K/V cold in the last-level cache."""
    B, Hq, Hkv, S, D = 64, 32, 8, 8192, 128
    g = torch.Generator(device="cpu").manual_seed(1005)
    q = torch.randn(B, Hq, 1, D, generator=g).to(torch.bfloat16).to(dev)
    lens = torch.randint(512, 8193, (B,), generator=g).to(torch.int32)
    caches = []
    for _ in range(sets):
        # synthetic cache drawn on the GPU (same distribution); parity on the seeded CPU draw
        # is the job of tests/test_decode_gpu.py
        kf = torch.randn(B, Hkv, S, D, device=dev)
        vf = torch.randn(B, Hkv, S, D, device=dev)
        ks = (kf.abs().amax((-2, -1)) / 448.0).float()
        vs = (vf.abs().amax((-2, -1)) / 448.0).float()
        caches.append(((kf / ks[:, :, None, None]).to(torch.float8_e4m3fn), (vf / vs[:, :, None, None]).to(torch.float8_e4m3fn), ks, vs))
        del kf, vf
    lens_d = lens.to(dev)
    total = int(lens.sum())
    nbytes = 2.0 * Hkv * D * total + 2 * (B * Hq * D * 2) + 2 * B * Hkv * 4 + B * 4
    state = {"i": 0}

    def step():
        kq, vq, ks, vs = caches[state["i"] % sets]
        state["i"] += 1
        amd.decode_fp8kv(q, kq, vq, ks, vs, lens_d)

    cfg = {"workload": "c5_decode_fp8kv", "B": B, "Hq": Hq, "Hkv": Hkv, "S_padded": S, "D": D,
           "sum_kv_len": total, "algorithmic_bytes": nbytes,
           "padded_read_bytes": 2.0 * B * Hkv * S * D}
    return step, nbytes, cfg


def cpu_model():
    """Model name of the host CPU the baseline runs on."""
    try:
        for line in open("/proc/cpuinfo"):
            if line.startswith("model name"):
                return line.split(":", 1)[1].strip()
    except OSError:
        pass
    return "unknown"


def cpu_threads():
    """Threads the CPU baseline uses: torch's intra-op pool, which follows OMP_NUM_THREADS (the
    box's CPU share) rather than the number of cores the machine shows."""
    return torch.get_num_threads()


def cpu_baseline_fwd(B, Hq, Hkv, S, D, seed, heads=2):
    """CPU oracle on a bounded sample: `heads` query heads of the same problem."""
    from oracle import sdpa_math as om

    g = torch.Generator(device="cpu").manual_seed(seed)
    q = torch.randn(B, Hq, S, D, generator=g).to(torch.bfloat16)[:, :heads].float()
    kvh = max(1, heads * Hkv // Hq)
    k = torch.randn(B, Hkv, S, D, generator=g).to(torch.bfloat16)[:, :kvh].float()
    v = torch.randn(B, Hkv, S, D, generator=g).to(torch.bfloat16)[:, :kvh].float()
    t0 = time.perf_counter()
    om.sdpa_forward(q, k, v, is_causal=True)
    dt = time.perf_counter() - t0
    flops = 4.0 * B * heads * D * causal_pairs(S, S)
    return {"value": flops / dt / 1e12, "unit": "TFLOP/s", "cores": cpu_threads(), "threads": cpu_threads(), "host_cores": os.cpu_count(), "cpu_model": cpu_model(),
            "kind": "port",
            "sample": f"{heads} of {Hq} query heads of the same workload, full S={S}; "
                      f"algorithmic (unmasked-pair) FLOPs / wall time; {dt:.2f} s"}


def cpu_baseline_fwd_bwd(B, Hq, Hkv, S, D, seed, heads=32):
    """CPU oracle forward + backward on `heads` query heads of config 4 (one batch element)."""
    from oracle import sdpa_math as om

    g = torch.Generator(device="cpu").manual_seed(seed)
    q = torch.randn(B, Hq, S, D, generator=g).to(torch.bfloat16)[:1, :heads].float()
    kvh = max(1, heads * Hkv // Hq)
    k = torch.randn(B, Hkv, S, D, generator=g).to(torch.bfloat16)[:1, :kvh].float()
    v = torch.randn(B, Hkv, S, D, generator=g).to(torch.bfloat16)[:1, :kvh].float()
    do = torch.randn(B, Hq, S, D, generator=g).to(torch.bfloat16)[:1, :heads].float()
    t0 = time.perf_counter()
    out, lse = om.sdpa_forward(q, k, v, is_causal=True)
    om.sdpa_backward(do, q, k, v, out, lse, is_causal=True)
    dt = time.perf_counter() - t0
    flops = 14.0 * heads * D * causal_pairs(S, S)
    return {"value": flops / dt / 1e12, "unit": "TFLOP/s", "cores": cpu_threads(), "threads": cpu_threads(), "host_cores": os.cpu_count(), "cpu_model": cpu_model(),
            "kind": "port",
            "sample": f"{heads} of {B * Hq} (batch, query head) pairs of the same workload, full S={S}, "
                      f"forward + backward; algorithmic (unmasked-pair) FLOPs / wall time; {dt:.2f} s"}


def cpu_baseline_decode(batches=32):
    """CPU oracle decode on the first `batches` sequences of config 5."""
    from oracle import sdpa_math as om

    B, Hq, Hkv, S, D = 64, 32, 8, 8192, 128
    g = torch.Generator(device="cpu").manual_seed(1005)
    q = torch.randn(B, Hq, 1, D, generator=g).to(torch.bfloat16)[:batches]
    lens = torch.randint(512, 8193, (B,), generator=g).to(torch.int32)[:batches]
    kq, ks = om.quantize_kv_fp8(torch.randn(batches, Hkv, S, D, generator=g))
    vq, vs = om.quantize_kv_fp8(torch.randn(batches, Hkv, S, D, generator=g))
    t0 = time.perf_counter()
    om.decode_fp8kv(q, kq, vq, ks, vs, lens)
    dt = time.perf_counter() - t0
    nbytes = 2.0 * Hkv * D * int(lens.sum())
    return {"value": nbytes / dt / 1e9, "unit": "GB/s", "cores": cpu_threads(), "threads": cpu_threads(), "host_cores": os.cpu_count(), "cpu_model": cpu_model(), "kind": "port",
            "sample": f"first {batches} of {B} sequences of the same workload ({int(lens.sum())} live keys); "
                      f"fp8 K/V bytes of the live keys / wall time (dequantisation included); {dt:.2f} s"}


# ------------------------------------------------------------------------------------------
# extras: the widened rows, a few launches each
# ------------------------------------------------------------------------------------------


def _fwd_bwd_rates(amd, q, k, v, do, live_pairs, e, dv, **kw):
    """Forward / backward rates on the scores that the mask keeps (`live_pairs` per batch and head)."""
    B, Hq = q.shape[0], q.shape[1]
    out, lse = amd.sdpa_forward(q, k, v, **kw)
    _, evf = event_time_ms(lambda: amd.sdpa_forward(q, k, v, **kw), 10, 3)
    _, evb = event_time_ms(lambda: amd.sdpa_backward(do, q, k, v, out, lse, **kw), 5, 2)
    f_fwd = 2.0 * B * Hq * (e + dv) * live_pairs
    f_bwd = 2.0 * B * Hq * (3 * e + 2 * dv) * live_pairs
    return {"fwd_ms": evf, "bwd_ms": evb, "fwd_TFLOP/s_live": f_fwd / (evf * 1e-3) / 1e12,
            "bwd_TFLOP/s_live": f_bwd / (evb * 1e-3) / 1e12}


def extra_window(amd, dev):
    """Sliding window of 1024 keys over the causal pattern, generated from indices (no mask tensor):
    B=2 Hq=32 Hkv=8 S=4096 D=128 bf16."""
    B, Hq, Hkv, S, D, W = 2, 32, 8, 4096, 128, 1024
    q, k, v, do = seeded([(B, Hq, S, D), (B, Hkv, S, D), (B, Hkv, S, D), (B, Hq, S, D)], 1008, torch.bfloat16, dev)
    live = sum(min(i + 1, W) for i in range(S))
    r = _fwd_bwd_rates(amd, q, k, v, do, live, D, D, is_causal=True, window=W)
    r["shape"] = "B=2 Hq=32 Hkv=8 S=4096 D=128 bf16, window 1024"
    return r


def extra_documents(amd, dev):
    """Packed sequences (eight documents of 512 keys, each causal) given as a bool mask tensor; the
    kernels skip the tiles that the mask drops through its tile skip tables."""
    B, Hq, Hkv, S, D = 2, 32, 8, 4096, 128
    q, k, v, do = seeded([(B, Hq, S, D), (B, Hkv, S, D), (B, Hkv, S, D), (B, Hq, S, D)], 1009, torch.bfloat16, dev)
    doc = torch.arange(S, device=dev) // 512
    mask = ((doc[:, None] == doc[None, :]) & torch.tril(torch.ones(S, S, dtype=torch.bool, device=dev)))[None, None]
    maps = amd.ops.mask_tile_maps(mask, B, Hq, S, S)
    r = _fwd_bwd_rates(amd, q, k, v, do, int(mask.sum().item()), D, D, attn_bias=mask, live_tiles=maps)
    _, evt = event_time_ms(lambda: amd.ops.mask_tile_maps(mask, B, Hq, S, S), 5, 2)
    r["tables_ms"] = evt
    r["shape"] = "B=2 Hq=32 Hkv=8 S=4096 D=128 bf16, (1,1,S,S) bool mask of 8 causal documents"
    return r


def extra_alibi(amd, dev):
    """ALiBi under the causal mask, as a score functor (a slope per head, no bias tensor):
    B=2 Hq=32 Hkv=8 S=4096 D=128 bf16."""
    B, Hq, Hkv, S, D = 2, 32, 8, 4096, 128
    q, k, v, do = seeded([(B, Hq, S, D), (B, Hkv, S, D), (B, Hkv, S, D), (B, Hq, S, D)], 1013, torch.bfloat16, dev)
    slopes = torch.exp2(-(torch.arange(Hq, device=dev, dtype=torch.float32) + 1) * 8.0 / Hq)
    r = _fwd_bwd_rates(amd, q, k, v, do, causal_pairs(S, S), D, D, is_causal=True, alibi_slopes=slopes)
    r["shape"] = "B=2 Hq=32 Hkv=8 S=4096 D=128 bf16, causal + ALiBi slopes"
    return r


def extra_document_ids(amd, dev):
    """Packed sequences (eight documents of 512 keys, each causal) given as document ids: no mask
    tensor; the kernels find the key tiles of a row block's documents by themselves."""
    B, Hq, Hkv, S, D = 2, 32, 8, 4096, 128
    q, k, v, do = seeded([(B, Hq, S, D), (B, Hkv, S, D), (B, Hkv, S, D), (B, Hq, S, D)], 1009, torch.bfloat16, dev)
    doc = (torch.arange(S, device=dev) // 512).to(torch.int32)[None].expand(B, S).contiguous()
    live = 8 * causal_pairs(512, 512)
    r = _fwd_bwd_rates(amd, q, k, v, do, live, D, D, is_causal=True, doc_ids_q=doc, doc_ids_k=doc, doc_ids_sorted=True)
    r["shape"] = "B=2 Hq=32 Hkv=8 S=4096 D=128 bf16, causal + (B,S) document ids, 8 documents of 512"
    return r


def extra_wide(amd, dev):
    """Head dim 256, causal MHA, B=2 H=16 S=4096 bf16."""
    B, H, S, D = 2, 16, 4096, 256
    q, k, v, do = seeded([(B, H, S, D), (B, H, S, D), (B, H, S, D), (B, H, S, D)], 1010, torch.bfloat16, dev)
    r = _fwd_bwd_rates(amd, q, k, v, do, causal_pairs(S, S), D, D, is_causal=True)
    r["shape"] = "B=2 H=16 S=4096 D=256 bf16 causal"
    return r


def extra_wide_window_softcap(amd, dev):
    """Head dim 256 with a sliding window of 1024 keys and a tanh soft cap of 50 on the scores (the attention
    of a Gemma-2 layer), both as functors: B=2 H=16 S=4096 bf16.  Rates count the scores the window keeps."""
    B, H, S, D, W = 2, 16, 4096, 256, 1024
    q, k, v, do = seeded([(B, H, S, D)] * 4, 1014, torch.bfloat16, dev)
    live = sum(min(i + 1, W) for i in range(S))
    r = _fwd_bwd_rates(amd, q, k, v, do, live, D, D, is_causal=True, window=W, softcap=50.0)
    r["shape"] = "B=2 H=16 S=4096 D=256 bf16, causal window 1024 + soft cap 50"
    return r


def extra_fresh_bool_mask(amd, dev):
    """F.scaled_dot_product_attention(attn_mask=bool lower triangle): upstream hands the op a NEW additive
    tensor on every call, so no per-tensor cache can know it; the verdict about the mask is taken on the
    device in front of the call (two small kernels), and the attention kernels follow it.  Forward time per
    call over ten calls in a row, against is_causal=True: B=4 H=32 S=4096 D=128 bf16."""
    import torch.nn.functional as F

    B, H, S, D = 4, 32, 4096, 128
    q, k, v = seeded([(B, H, S, D)] * 3, 1015, torch.bfloat16, dev)
    tril = torch.ones(S, S, dtype=torch.bool, device=dev).tril()
    amd.mask_patterns.clear_cache()
    with torch.no_grad():
        _, ev_m = event_time_ms(lambda: F.scaled_dot_product_attention(q, k, v, attn_mask=tril), 10, 3)
        _, ev_c = event_time_ms(lambda: F.scaled_dot_product_attention(q, k, v, is_causal=True), 10, 3)
    flops = 4.0 * B * H * D * causal_pairs(S, S)
    return {"bool_mask_ms": ev_m, "is_causal_ms": ev_c, "ratio": ev_m / ev_c, "TFLOP/s_live": flops / (ev_m * 1e-3) / 1e12,
            "shape": "B=4 H=32 S=4096 D=128 bf16, F.scaled_dot_product_attention(attn_mask=tril bool)"}


def extra_dropout(amd, dev):
    """Dropout 0.1 with right padding, a BERT-base layer in training: B=32 H=12 S=512 D=64 bf16, key counts
    between S/2 and S, the (B,H,S,S) keep-mask drawn once.  Rates count the scores that the padding keeps."""
    B, H, S, D = 32, 12, 512, 64
    q, k, v, do = seeded([(B, H, S, D)] * 4, 1012, torch.bfloat16, dev)
    g = torch.Generator(device="cpu").manual_seed(1012)
    lens = torch.randint(S // 2, S + 1, (B,), generator=g, dtype=torch.int32)
    keep = (torch.rand(B, H, S, S, device=dev) >= 0.1).to(torch.uint8)
    kw = dict(kv_lens=lens.to(dev), dropout_p=0.1, dropout_keep=keep)
    out, lse = amd.sdpa_forward(q, k, v, **kw)
    _, evf = event_time_ms(lambda: amd.sdpa_forward(q, k, v, **kw), 10, 3)
    _, evb = event_time_ms(lambda: amd.sdpa_backward(do, q, k, v, out, lse, **kw), 5, 2)
    live = float(lens.sum().item()) * S * H  # kept (query, key) pairs over all batches and heads
    return {"fwd_ms": evf, "bwd_ms": evb, "fwd_TFLOP/s_live": 4.0 * D * live / (evf * 1e-3) / 1e12,
            "bwd_TFLOP/s_live": 10.0 * D * live / (evb * 1e-3) / 1e12,
            "shape": "B=32 H=12 S=512 D=64 bf16, dropout 0.1, right padding (key counts)"}


def extra_decode_bf16(amd, dev):
    """A decode step over a bf16 K/V cache through the ordinary forward (no fp8, no decode entry point):
    Hq=32 Hkv=8 D=128 L=1, a full batch (the heads of a kv group share a workgroup) and a single
    sequence (its keys are split over workgroups)."""
    Hq, Hkv, D = 32, 8, 128
    r = {}
    for name, B, S in (("B64_S8192", 64, 8192), ("B1_S32768", 1, 32768)):
        g = torch.Generator(device=dev).manual_seed(1013)  # (drawn on the device: the cache is 2 x 1 GB)
        q = torch.randn((B, Hq, 1, D), generator=g, device=dev, dtype=torch.bfloat16)
        k, v = (torch.randn((B, Hkv, S, D), generator=g, device=dev, dtype=torch.bfloat16) for _ in range(2))
        amd.sdpa_forward(q, k, v)
        _, ev = event_time_ms(lambda: amd.sdpa_forward(q, k, v), 20, 5)
        r[name] = {"ms": ev, "kv_GB/s": 2.0 * B * Hkv * S * D * 2 / (ev * 1e-3) / 1e9}
        del q, k, v
    r["shape"] = "Hq=32 Hkv=8 D=128 L=1 bf16 cache"
    return r


def extra_decode_fp8_one_sequence(amd, dev):
    """The fp8-cache decode entry point on one long sequence (interactive serving): Hq=32 Hkv=8 D=128 L=1,
    B=1 at 32768 and 131072 keys - every (batch, kv head) is cut into a hundred pieces and more."""
    Hq, Hkv, D = 32, 8, 128
    r = {}
    for name, B, S in (("B1_S32768", 1, 32768), ("B1_S131072", 1, 131072)):
        g = torch.Generator(device=dev).manual_seed(1017)
        q = torch.randn((B, Hq, 1, D), generator=g, device=dev, dtype=torch.bfloat16)
        kq, vq = (torch.randn((B, Hkv, S, D), generator=g, device=dev).to(torch.float8_e4m3fn) for _ in range(2))
        sc = torch.ones(B, Hkv, device=dev)
        amd.decode_fp8kv(q, kq, vq, sc, sc, None)
        _, ev = event_time_ms(lambda: amd.decode_fp8kv(q, kq, vq, sc, sc, None), 30, 5)
        r[name] = {"ms": ev, "kv_GB/s": 2.0 * B * Hkv * S * D / (ev * 1e-3) / 1e9}
        del q, kq, vq
    r["shape"] = "Hq=32 Hkv=8 D=128 L=1 fp8 e4m3 cache"
    return r


def extra_few_kv_heads(amd, dev):
    """Backward with few key blocks, where the dK/dV kernel deals a block's query tiles to several
    workgroups: one kv head for 32 query heads (B=2 S=4096) and a 32/8 model at batch 1 (S=2048), D=128 causal."""
    r = {}
    for name, B, Hq, Hkv, S in (("mqa_32_1_B2_S4096", 2, 32, 1, 4096), ("gqa_32_8_B1_S2048", 1, 32, 8, 2048)):
        q, k, v, do = seeded([(B, Hq, S, 128), (B, Hkv, S, 128), (B, Hkv, S, 128), (B, Hq, S, 128)], 1015, torch.bfloat16, dev)
        r[name] = _fwd_bwd_rates(amd, q, k, v, do, causal_pairs(S, S), 128, 128, is_causal=True)
    r["shape"] = "D=128 bf16 causal"
    return r


def extra_f32(amd, dev):
    """float32 inputs on the float32 matrix op (peak 157.3 TFLOP/s), B=2 Hq=32 Hkv=8 S=4096 D=128 causal."""
    B, Hq, Hkv, S, D = 2, 32, 8, 4096, 128
    q, k, v, do = seeded([(B, Hq, S, D), (B, Hkv, S, D), (B, Hkv, S, D), (B, Hq, S, D)], 1011, torch.float32, dev)
    r = _fwd_bwd_rates(amd, q, k, v, do, causal_pairs(S, S), D, D, is_causal=True)
    r["fwd_frac_of_f32_peak"] = r["fwd_TFLOP/s_live"] / 157.3
    r["bwd_frac_of_f32_peak"] = r["bwd_TFLOP/s_live"] / 157.3
    r["shape"] = "B=2 Hq=32 Hkv=8 S=4096 D=128 float32 causal"
    return r


def known_size_copy(dev, mib=256):
    """One plain device-to-device copy of `mib` MiB: the yardstick that the HBM traffic counters
    (FETCH_SIZE / WRITE_SIZE) of a profiled run are scaled by."""
    src = torch.empty(mib << 20, dtype=torch.uint8, device=dev).fill_(1)
    dst = torch.empty_like(src)
    torch.cuda.synchronize()
    dst.copy_(src)
    torch.cuda.synchronize()
    del src, dst
    torch.cuda.empty_cache()


# HBM bytes per launch of the dominant kernel come from `rocprofv3 --pmc FETCH_SIZE` and
# `--pmc WRITE_SIZE` runs of this script (--pmc-copy), scaled by the same counters' reading for the
# known-size copy.  A counter run cannot be made from inside a timed run, so the figure is read from
# the committed summary of those runs (its `hbm_bytes_per_launch:` line); no summary, no figure.
TRAFFIC_SUMMARIES = {
    "c3_fwd": "fwd_w32_kernel_c3_causal_gqa_bf16_fwd.txt",
    "c4_fwd_bwd": "bwd_kernels_c4_causal_gqa_bf16_fwd_bwd.txt",
    "c5_decode": "decode_kernel_c5_decode_fp8kv.txt",
}


def measured_traffic_bytes(workload):
    name = TRAFFIC_SUMMARIES.get(workload)
    if not name:
        return None
    try:
        with open(os.path.join(ROOT, "profiles", name)) as f:
            for line in f:
                if line.startswith("hbm_bytes_per_launch:"):
                    return float(line.split(":", 1)[1].split()[0])
    except OSError:
        pass
    return None


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=100)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--workload", default="c3_fwd", choices=["c3_fwd", "c2_fwd", "c4_fwd_bwd", "c5_decode", "masked_fwd", "mqa_fwd_bwd"])
    ap.add_argument("--no-extras", action="store_true")
    ap.add_argument("--no-cpu", action="store_true")
    ap.add_argument("--no-spin", action="store_true", help="skip the untimed clock spin-up (profiled runs)")
    ap.add_argument("--pmc-copy", action="store_true",
                    help="also run one 256 MiB device copy (counter yardstick for profiled runs)")
    args = ap.parse_args()
    if args.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        print("bench.py: this build runs on ONE GPU; --gpus N with N > 1 is not supported "
              "(no collectives or sharding are part of it).", file=sys.stderr)
        sys.exit(2)
    if not torch.cuda.is_available():
        print("bench.py: no GPU visible", file=sys.stderr)
        sys.exit(1)

    import torch_neuronx_amd as amd

    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    extras = {}
    global SPIN
    SPIN = not args.no_spin
    if args.pmc_copy:
        known_size_copy(dev)

    if args.workload in ("c3_fwd", "c2_fwd"):
        if args.workload == "c3_fwd":
            step, flops, cfg, _ = wl_fwd(amd, dev, 1, 32, 8, 8192, 128, 1003, "c3_causal_gqa_bf16_fwd_llama3_8b")
        else:
            step, flops, cfg, _ = wl_fwd(amd, dev, 4, 12, 12, 1024, 64, 1002, "c2_causal_mha_bf16_fwd_gpt2_small")
        wall, ev = event_time_ms(step, args.steps, args.warmup)
        value = flops / (wall * 1e-3) / 1e12
        ach = flops / (ev * 1e-3) / 1e12
        roof = {"bound": "mfma", "achieved": ach, "peak": PEAK_BF16_TFLOPS, "unit": "TFLOP/s",
                "frac": ach / PEAK_BF16_TFLOPS, "traffic": None, "kernel": "fwd_w32_kernel",
                "kernel_ms": ev}
        unit, dtype = "TFLOP/s", "bf16"
        cpu = None
        if not args.no_cpu:
            if args.workload == "c3_fwd":
                cpu = cpu_baseline_fwd(1, 32, 8, 8192, 128, 1003, heads=32)
            else:
                cpu = cpu_baseline_fwd(4, 12, 12, 1024, 64, 1002, heads=12)
    elif args.workload == "masked_fwd":
        step, flops, cfg = wl_masked_fwd(amd, dev)
        wall, ev = event_time_ms(step, args.steps, args.warmup)
        value = flops / (wall * 1e-3) / 1e12
        ach = flops / (ev * 1e-3) / 1e12
        roof = {"bound": "mfma", "achieved": ach, "peak": PEAK_BF16_TFLOPS, "unit": "TFLOP/s",
                "frac": ach / PEAK_BF16_TFLOPS, "traffic": None, "kernel": "fwd_w32_kernel (masked variant)",
                "kernel_ms": ev}
        unit, dtype = "TFLOP/s", "bf16"
        cpu = None  # the oracle's rate on this shape is the forward baseline of c3_fwd
    elif args.workload in ("c4_fwd_bwd", "mqa_fwd_bwd"):  # (mqa: config 4 with one kv head for the 32 query heads)
        hkv = 8 if args.workload == "c4_fwd_bwd" else 1
        sf, sb, f_fwd, f_bwd = wl_fwd_bwd(amd, dev, hkv)
        _, ev_f = event_time_ms(sf, args.steps, args.warmup)

        def both():
            sf()
            sb()

        wall, ev = event_time_ms(both, args.steps, args.warmup)
        _, ev_b = event_time_ms(sb, args.steps, args.warmup)
        flops = f_fwd + f_bwd
        value = flops / (wall * 1e-3) / 1e12
        ach = f_bwd / (ev_b * 1e-3) / 1e12
        roof = {"bound": "mfma", "achieved": ach, "peak": PEAK_BF16_TFLOPS, "unit": "TFLOP/s",
                "frac": ach / PEAK_BF16_TFLOPS, "traffic": None, "kernel": "backward (all kernels of one call)",
                "kernel_ms": ev_b}
        cfg = {"workload": "c4_causal_gqa_bf16_fwd_bwd" if hkv == 8 else "causal_mqa_bf16_fwd_bwd", "B": 2, "Hq": 32, "Hkv": hkv, "S": 4096, "D": 128,
               "fwd_tflops": f_fwd / (ev_f * 1e-3) / 1e12, "bwd_tflops": ach,
               "algorithmic_flops": flops}
        unit, dtype = "TFLOP/s", "bf16"
        cpu = None if args.no_cpu or hkv != 8 else cpu_baseline_fwd_bwd(2, 32, 8, 4096, 128, 1004, heads=32)
    else:
        step, nbytes, cfg = wl_decode(amd, dev)
        wall, ev = event_time_ms(step, args.steps, args.warmup)
        value = nbytes / (wall * 1e-3) / 1e9
        ach = nbytes / (ev * 1e-3) / 1e9
        roof = {"bound": "hbm", "achieved": ach, "peak": PEAK_HBM_GBS, "unit": "GB/s",
                "frac": ach / PEAK_HBM_GBS, "traffic": None, "kernel": "decode_kernel + decode_merge_kernel (one call)",
                "kernel_ms": ev}
        unit, dtype = "GB/s", "fp8_e4m3 (K/V), bf16 (Q/O), f32 accumulate"
        cpu = None if args.no_cpu else cpu_baseline_decode(batches=32)

    if not args.no_extras and args.workload == "c3_fwd":
        try:
            step5, nbytes5, cfg5 = wl_decode(amd, dev)
            _, ev5 = event_time_ms(step5, 40, 8)
            gbs = nbytes5 / (ev5 * 1e-3) / 1e9
            extras["c5_decode_fp8kv"] = {"GB/s": gbs, "frac_of_hbm_peak": gbs / PEAK_HBM_GBS,
                                         "kernel_ms": ev5, "algorithmic_bytes": nbytes5}
            del step5
            torch.cuda.empty_cache()
        except Exception as e:  # reported, never hidden
            extras["c5_decode_fp8kv"] = {"error": repr(e)}
        try:
            sf, sb, f_fwd, f_bwd = wl_fwd_bwd(amd, dev)
            _, evf = event_time_ms(sf, 10, 3)
            _, evb = event_time_ms(sb, 5, 2)
            extras["c4_fwd_bwd"] = {"fwd_TFLOP/s": f_fwd / (evf * 1e-3) / 1e12,
                                    "bwd_TFLOP/s": f_bwd / (evb * 1e-3) / 1e12,
                                    "fwd_ms": evf, "bwd_ms": evb,
                                    "bwd_frac_of_bf16_peak": f_bwd / (evb * 1e-3) / 1e12 / PEAK_BF16_TFLOPS}
        except Exception as e:
            extras["c4_fwd_bwd"] = {"error": repr(e)}
        try:
            stepm, flopsm, cfgm = wl_masked_fwd(amd, dev)
            _, evm = event_time_ms(stepm, 10, 3)
            extras["masked_fwd_shared_bias"] = {"TFLOP/s": flopsm / (evm * 1e-3) / 1e12, "kernel_ms": evm,
                                                "frac_of_bf16_peak": flopsm / (evm * 1e-3) / 1e12 / PEAK_BF16_TFLOPS}
        except Exception as e:
            extras["masked_fwd_shared_bias"] = {"error": repr(e)}
        for name, fn in (("window_1024_fwd_bwd", extra_window), ("document_mask_tables_fwd_bwd", extra_documents),
                         ("alibi_causal_fwd_bwd", extra_alibi), ("document_ids_fwd_bwd", extra_document_ids),
                         ("head_dim_256_fwd_bwd", extra_wide), ("head_dim_256_window_softcap_fwd_bwd", extra_wide_window_softcap),
                         ("fresh_bool_mask_fwd", extra_fresh_bool_mask), ("dropout_padding_fwd_bwd", extra_dropout), ("decode_bf16_cache_fwd", extra_decode_bf16),
                         ("decode_fp8_one_sequence", extra_decode_fp8_one_sequence),
                         ("few_kv_heads_fwd_bwd", extra_few_kv_heads), ("float32_fwd_bwd", extra_f32)):
            try:
                extras[name] = fn(amd, dev)
            except Exception as e:
                extras[name] = {"error": repr(e)}
            torch.cuda.empty_cache()

    roof["traffic"] = measured_traffic_bytes(args.workload)
    line = {
        "metric": METRIC, "value": value, "unit": unit, "n_gpus": 1, "steps": args.steps,
        "warmup": args.warmup, "ms_per_step": wall, "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": dtype, "data": "synthetic", "config": cfg,
        "roofline": roof, "cpu_baseline": cpu, "extras": extras,
    }
    print(json.dumps(line))


if __name__ == "__main__":
    main()
