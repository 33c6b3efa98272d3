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


def _case(B, Hq, Hkv, Lq, S, lens, seed, qdtype=torch.bfloat16):
    g = torch.Generator().manual_seed(seed)
    q = torch.randn(B, Hq, Lq, 128, generator=g).to(qdtype)
    k = torch.randn(B, Hkv, S, 128, generator=g)
    v = torch.randn(B, Hkv, S, 128, generator=g)
    kq, ks = om.quantize_kv_fp8(k)
    vq, vs = om.quantize_kv_fp8(v)
    return q, kq, vq, ks, vs, lens


def _check(amd, dev, case, tol=2e-2, **kw):
    q, kq, vq, ks, vs, lens = case
    out, lse = amd.decode_fp8kv(q.to(dev), kq.to(dev), vq.to(dev), ks.to(dev), vs.to(dev),
                                None if lens is None else lens.to(dev), **kw)
    torch.cuda.synchronize()
    S = kq.shape[2]
    ro, rl = om.decode_fp8kv(q, kq, vq, ks, vs, lens if lens is not None else torch.full((q.shape[0],), S))
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
