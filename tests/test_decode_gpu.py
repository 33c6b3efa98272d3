"""GPU parity of the fp8-KV decode kernel against the CPU oracle, through the C ABI.

The reference has no fp8 attention path: the oracle's definition (dequantise, then the
reference's forward math with a key-padding bias) is the contract.  PARITY UNPINNED by the
reference's own tests.
"""

import pytest
import torch

from helpers import max_abs
from oracle import sdpa_math as om

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def amd(gpu_device):
    import torch_neuronx_amd as amd

    return amd


def _case(B, Hq, Hkv, Lq, S, lens, seed, qdtype=torch.bfloat16, D=128):
    g = torch.Generator().manual_seed(seed)
    q = torch.randn(B, Hq, Lq, D, generator=g).to(qdtype)
    k = torch.randn(B, Hkv, S, D, generator=g)
    v = torch.randn(B, Hkv, S, D, generator=g)
    kq, ks = om.quantize_kv_fp8(k)
    vq, vs = om.quantize_kv_fp8(v)
    return q, kq, vq, ks, vs, lens


def _check(amd, dev, case, tol=2e-2, **kw):
    q, kq, vq, ks, vs, lens = case
    out, lse = amd.decode_fp8kv(q.to(dev), kq.to(dev), vq.to(dev), ks.to(dev), vs.to(dev),
                                None if lens is None else lens.to(dev), **kw)
    torch.cuda.synchronize()
    S = kq.shape[2]
    ro, rl = om.decode_fp8kv(q, kq, vq, ks, vs, lens if lens is not None else torch.full((q.shape[0],), S),
                             scale=kw.get("scale"))
    assert out.dtype == q.dtype
    assert max_abs(out, ro) <= tol
    assert max_abs(lse, rl) <= 5e-3
    return out, lse


@pytest.mark.parametrize("Hq,Hkv,Lq", [(32, 8, 1), (8, 8, 1), (16, 2, 1), (8, 2, 2), (4, 4, 3)])
def test_decode_small(amd, gpu_device, Hq, Hkv, Lq):
    lens = torch.tensor([700, 1, 33, 512, 513], dtype=torch.int32)
    _check(amd, gpu_device, _case(5, Hq, Hkv, Lq, 700, lens, seed=Hq + Lq))


def test_decode_no_lens_and_split_choices(amd, gpu_device):
    case = _case(2, 32, 8, 1, 1536, None, seed=3)
    a, la = _check(amd, gpu_device, case)
    b, lb = _check(amd, gpu_device, case, num_splits=1)
    c, lc = _check(amd, gpu_device, case, num_splits=12)
    assert max_abs(a, b) <= 4e-3 and max_abs(a, c) <= 4e-3


def test_decode_zero_length_sequence(amd, gpu_device):
    lens = torch.tensor([0, 5], dtype=torch.int32)
    q, kq, vq, ks, vs, _ = _case(2, 8, 2, 1, 256, lens, seed=5)
    out, lse = amd.decode_fp8kv(q.to(gpu_device), kq.to(gpu_device), vq.to(gpu_device),
                                ks.to(gpu_device), vs.to(gpu_device), lens.to(gpu_device))
    assert torch.equal(out[0].float().cpu(), torch.zeros(8, 1, 128))
    assert torch.isinf(lse[0]).all() and (lse[0] < 0).all()


def test_decode_fp32_and_fp16_queries(amd, gpu_device):
    lens = torch.tensor([300, 129], dtype=torch.int32)
    for dt in (torch.float32, torch.float16):
        _check(amd, gpu_device, _case(2, 8, 2, 1, 300, lens, seed=11, qdtype=dt))


def test_decode_many_batches_with_empty_and_short_sequences(amd, gpu_device):
    # more than 64 batches (the kernel scans lengths 64 at a time), empty sequences between
    # live ones, and sequences so short that one wavefront's share spans several of them
    B = 150
    g = torch.Generator().manual_seed(77)
    lens = torch.randint(0, 97, (B,), generator=g).to(torch.int32)
    lens[0] = 0
    lens[63:66] = 0
    lens[-1] = 0
    lens[70] = 300
    case = _case(B, 8, 2, 1, 300, lens, seed=78)
    out, lse = _check(amd, gpu_device, case)
    dead = lens == 0
    assert torch.equal(out[dead].float().cpu(), torch.zeros(int(dead.sum()), 8, 1, 128))
    assert torch.isinf(lse[dead]).all()
    # one piece per sequence at most (plus alignment) gives the same answer
    out1, _ = _check(amd, gpu_device, case, num_splits=1)
    assert max_abs(out, out1) <= 4e-3


def test_decode_all_sequences_empty(amd, gpu_device):
    lens = torch.zeros(3, dtype=torch.int32)
    q, kq, vq, ks, vs, _ = _case(3, 8, 2, 1, 64, lens, seed=9)
    out, lse = amd.decode_fp8kv(q.to(gpu_device), kq.to(gpu_device), vq.to(gpu_device),
                                ks.to(gpu_device), vs.to(gpu_device), lens.to(gpu_device))
    assert torch.equal(out.float().cpu(), torch.zeros(3, 8, 1, 128))
    assert torch.isinf(lse).all() and (lse < 0).all()


def test_config5_full_size(amd, gpu_device):
    # benchmark configuration 5: B=64,Hq=32,Hkv=8,D=128,q_len=1, kv_len ~ U[512,8192] padded to 8192
    B, Hq, Hkv, S = 64, 32, 8, 8192
    g = torch.Generator().manual_seed(1005)
    q = torch.randn(B, Hq, 1, 128, generator=g).to(torch.bfloat16)
    lens = torch.randint(512, 8193, (B,), generator=g).to(torch.int32)
    kq = torch.empty(B, Hkv, S, 128, dtype=torch.float8_e4m3fn)
    vq = torch.empty(B, Hkv, S, 128, dtype=torch.float8_e4m3fn)
    ks = torch.empty(B, Hkv)
    vs = torch.empty(B, Hkv)
    for b in range(B):  # batch by batch keeps the fp32 staging small
        kb = torch.randn(1, Hkv, S, 128, generator=g)
        vb = torch.randn(1, Hkv, S, 128, generator=g)
        kq[b : b + 1], ks[b : b + 1] = om.quantize_kv_fp8(kb)
        vq[b : b + 1], vs[b : b + 1] = om.quantize_kv_fp8(vb)
    _check(amd, gpu_device, (q, kq, vq, ks, vs, lens))


# Queries that are not bf16 carry more significant bits than two or three e4m3 terms hold (float16: 11,
# float32: 24).  The configurations below - float16 / float32 queries at scales 0.2 and 1.0 on N(0,1)
# data, logits of +-10 and more, one key up to 2048 - are the ones a randomised sweep found outside
# 2e-2 / 5e-3 when such queries were cut to 8 or 12 bits; the kernel now gives them 12 to 16.
_SHARP = [
    # (dtype, B, Hq, Hkv, Lq, S, lens, scale, splits)
    (torch.float32, 130, 4, 2, 4, 1, "short", 0.2, 1),
    (torch.float32, 2, 16, 8, 4, 31, "none", 1.0, 0),
    (torch.float16, 2, 16, 8, 3, 2048, "none", 1.0, 0),
    (torch.float32, 1, 12, 2, 1, 31, "full", 1.0, 0),
    (torch.float16, 2, 3, 1, 2, 100, "rand", 1.0, 1),
    (torch.float32, 3, 2, 1, 4, 500, "none", 1.0, 0),
    (torch.float32, 1, 8, 1, 1, 500, "rand", 1.0, 7),
    (torch.float32, 2, 2, 1, 3, 33, "short", 1.0, 2),
    (torch.float32, 5, 2, 1, 3, 32, "short", 1.0, 0),
    (torch.float16, 17, 48, 8, 1, 1, "rand", 1.0, 7),
    (torch.float16, 130, 48, 8, 1, 576, "rand", 0.2, 7),
    (torch.float16, 2, 16, 8, 4, 2048, "full", 1.0, 7),
    (torch.float16, 2, 16, 8, 3, 1000, "short", 1.0, 7),
    (torch.float16, 5, 16, 8, 3, 32, "rand", 1.0, 0),
    (torch.float16, 5, 24, 8, 2, 128, "short", 1.0, 0),
    (torch.float32, 64, 64, 8, 1, 32, "none", 1.0, 0),
    (torch.float16, 5, 48, 8, 1, 500, "none", 1.0, 1),
    (torch.float32, 5, 48, 8, 1, 1000, "rand", 1.0, 0),
    (torch.float16, 2, 64, 8, 1, 128, "short", 1.0, 2),
    (torch.float32, 5, 6, 2, 2, 32, "none", 1.0, 7),
    (torch.float16, 1, 2, 1, 3, 2048, "full", 1.0, 7),
    (torch.float32, 64, 8, 1, 1, 128, "rand", 1.0, 7),
    (torch.float16, 5, 6, 2, 2, 2048, "none", 1.0, 1),
]


@pytest.mark.parametrize("cfg", _SHARP, ids=lambda c: f"{str(c[0])[6:]}-B{c[1]}-{c[2]}x{c[3]}-Lq{c[4]}-S{c[5]}-{c[6]}-{c[7]}")
def test_decode_keeps_the_precision_of_float16_and_float32_queries(amd, gpu_device, cfg):
    dt, B, Hq, Hkv, Lq, S, mode, scale, splits = cfg
    g = torch.Generator().manual_seed(B * 1000 + S)
    lens = {"rand": torch.randint(0, S + 1, (B,), generator=g), "full": torch.full((B,), S), "none": None,
            "short": torch.randint(0, min(S, 40) + 1, (B,), generator=g)}[mode]
    lens = None if lens is None else lens.to(torch.int32)
    _check(amd, gpu_device, _case(B, Hq, Hkv, Lq, S, lens, seed=S + Hq, qdtype=dt), scale=scale, num_splits=splits)


def test_decode_float32_query_with_one_key(amd, gpu_device):
    # one key: the output is that key's value row and lse is the logit itself, so its error is the
    # error of the query's representation alone (8 bits would give about 6e-3 here)
    dev = gpu_device
    q, kq, vq, ks, vs, _ = _case(130, 4, 2, 4, 1, None, seed=5, qdtype=torch.float32)
    out, lse = amd.decode_fp8kv(q.to(dev), kq.to(dev), vq.to(dev), ks.to(dev), vs.to(dev), None, scale=0.2)
    ro, rl = om.decode_fp8kv(q, kq, vq, ks, vs, torch.full((130,), 1), scale=0.2)
    assert max_abs(lse, rl) <= 1e-3 and max_abs(out, ro) <= 1e-3


@pytest.mark.parametrize("qdtype", [torch.bfloat16, torch.float16, torch.float32])
@pytest.mark.parametrize("Hq,Hkv,Lq", [(12, 1, 1), (16, 1, 1), (8, 2, 4), (24, 2, 1), (3, 1, 5)])
def test_decode_up_to_sixteen_query_rows_per_kv_head(amd, gpu_device, qdtype, Hq, Hkv, Lq):
    lens = torch.tensor([700, 1, 33, 0], dtype=torch.int32)
    _check(amd, gpu_device, _case(4, Hq, Hkv, Lq, 700, lens, seed=Hq + Lq, qdtype=qdtype))


@pytest.mark.parametrize("D", [64, 256])
@pytest.mark.parametrize("qdtype", [torch.bfloat16, torch.float16, torch.float32])
@pytest.mark.parametrize("Hq,Hkv,Lq", [(32, 8, 1), (8, 8, 1), (8, 1, 1), (16, 1, 1), (4, 2, 3)])
def test_decode_head_dims_64_and_256(amd, gpu_device, D, qdtype, Hq, Hkv, Lq):
    # the same kernel laid out for 64- and 256-byte cache rows, every group size (terms x passes) of each query dtype
    lens = torch.tensor([700, 1, 33, 0, 513], dtype=torch.int32)
    case = _case(5, Hq, Hkv, Lq, 700, lens, seed=D + Hq + Lq, qdtype=qdtype, D=D)
    out, _ = _check(amd, gpu_device, case)
    assert torch.equal(out[3].float().cpu(), torch.zeros(Hq, Lq, D))  # the empty sequence
    _check(amd, gpu_device, case, scale=0.3)  # larger logits (the default scale at 256 is 1/16)


def test_decode_head_dims_64_and_256_long_and_split(amd, gpu_device):
    # sequences that several wavefronts share, with and without a cap on the pieces per sequence
    for D in (64, 256):
        case = _case(2, 32, 8, 1, 4096, torch.tensor([4096, 3001], dtype=torch.int32), seed=D, D=D)
        a, _ = _check(amd, gpu_device, case)
        b, _ = _check(amd, gpu_device, case, num_splits=1)
        assert max_abs(a, b) <= 4e-3


@pytest.mark.parametrize("D", [64, 128, 256])
def test_decode_of_one_long_sequence(amd, gpu_device, D):
    # a single sequence is cut into one piece per wavefront slot: more than a hundred partials per (batch,
    # kv head), which the merge reads a thread each and eight rows at a time
    case = _case(1, 8, 2, 1, 20000, torch.tensor([19977], dtype=torch.int32), seed=D + 1, D=D)
    a, la = _check(amd, gpu_device, case)
    b, lb = _check(amd, gpu_device, case, num_splits=4)  # ... against a few long pieces
    assert max_abs(a, b) <= 4e-3 and max_abs(la, lb) <= 1e-3


def test_decode_refuses_other_head_dims(amd, gpu_device):
    dev = gpu_device
    q, kq, vq, ks, vs, _ = _case(1, 8, 8, 1, 64, None, seed=1, D=96)
    with pytest.raises(RuntimeError, match="64, 128 or 256"):
        amd.decode_fp8kv(q.to(dev), kq.to(dev), vq.to(dev), ks.to(dev), vs.to(dev), None)


def test_decode_refuses_more_than_sixteen_rows(amd, gpu_device):
    dev = gpu_device
    q, kq, vq, ks, vs, _ = _case(1, 17, 1, 1, 64, None, seed=1)
    with pytest.raises(RuntimeError, match=r"\[1, 16\]"):
        amd.decode_fp8kv(q.to(dev), kq.to(dev), vq.to(dev), ks.to(dev), vs.to(dev), None)
