"""GPU test of the decode entry point that allocates nothing (mi355_sdpa_decode_fp8kv_static):
its results equal, bit for bit, those of mi355_sdpa_decode_fp8kv with a caller's workspace, on
two calls in a row (the second on a smaller input, so that what the first left in the static
scratch is stale), and against the CPU oracle; a call that needs more scratch than the static
array holds is refused.  Everything goes through the C ABI."""

import ctypes as C

import pytest
import torch

from helpers import max_abs
from oracle import sdpa_math as om

pytestmark = pytest.mark.gpu


def _inputs(dev, B, Hq, Hkv, Lq, S, lens, seed, D=128):
    g = torch.Generator().manual_seed(seed)
    q = torch.randn(B, Hq, Lq, D, generator=g).to(torch.bfloat16)
    kq, ks = om.quantize_kv_fp8(torch.randn(B, Hkv, S, D, generator=g))
    vq, vs = om.quantize_kv_fp8(torch.randn(B, Hkv, S, D, generator=g))
    cpu = (q, kq, vq, ks, vs, lens)
    gpu = tuple(None if t is None else t.to(dev) for t in (q, kq, vq, ks.float().contiguous(), vs.float().contiguous(), lens))
    return cpu, gpu


def test_static_scratch_decode_matches_the_workspace_entry_point(gpu_device):
    import torch_neuronx_amd as amd

    dev = gpu_device
    big_lens = torch.tensor([2048, 517, 1, 1999, 1024, 33, 777, 1500], dtype=torch.int32)
    small_lens = torch.tensor([300, 64, 5], dtype=torch.int32)
    cases = [_inputs(dev, 8, 32, 8, 1, 2048, big_lens, 11), _inputs(dev, 3, 8, 2, 2, 320, small_lens, 12),
             _inputs(dev, 3, 16, 2, 1, 320, small_lens, 13, D=256), _inputs(dev, 3, 8, 8, 1, 320, small_lens, 14, D=64)]  # (the other head dims)
    # outputs are the caller's: allocated here, before the calls under test
    outs = [(torch.empty(c[1][0].shape, dtype=torch.bfloat16, device=dev),
             torch.empty(c[1][0].shape[:3], dtype=torch.float32, device=dev)) for c in cases]
    refs = [amd.decode_fp8kv(*c[1]) for c in cases]  # the existing entry point, workspace from the caller
    torch.cuda.synchronize()
    for rnd in range(2):  # two passes: the second starts from the scratch the first left behind
        for (cpu, gpu), (out, lse), (ro, rl) in zip(cases, outs, refs):
            out.fill_(float("nan")), lse.fill_(float("nan"))
            before = torch.cuda.memory_allocated(dev)
            o, l = amd.decode_fp8kv(*gpu, out=out, lse=lse, static_scratch=True)
            assert torch.cuda.memory_allocated(dev) == before
            torch.cuda.synchronize()
            assert o is out and l is lse
            assert torch.equal(out, ro) and torch.equal(lse, rl), (rnd, max_abs(out, ro), max_abs(lse, rl))
            wo, wl = om.decode_fp8kv(*cpu)
            assert max_abs(out, wo) <= 2e-2 and max_abs(lse, wl) <= 5e-3


def test_static_scratch_decode_refuses_what_does_not_fit(gpu_device):
    import torch_neuronx_amd as amd
    from torch_neuronx_amd import _lib

    dev = gpu_device
    # scratch grows with batch * kv heads * query rows per kv head: find a size beyond the array
    B, Hq, Hkv, Lq, S = 4096, 16, 2, 1, 64
    q = torch.zeros(B, Hq, Lq, 128, dtype=torch.bfloat16, device=dev)
    kq = torch.zeros(B, Hkv, S, 128, dtype=torch.float8_e4m3fn, device=dev)
    sc = torch.ones(B, Hkv, dtype=torch.float32, device=dev)
    out = torch.empty_like(q)
    p = _lib.DecodeParams()
    p.q, p.k, p.v, p.out = (_lib.tensor4(t) for t in (q, kq, kq, out))
    p.k_scale = p.v_scale = sc.data_ptr()
    p.q_dtype, p.scale = _lib.BF16, 0.1
    lib = _lib.load()
    need = lib.mi355_sdpa_decode_workspace_bytes(C.byref(p))
    assert need > _lib.DECODE_STATIC_SCRATCH_BYTES
    rc = lib.mi355_sdpa_decode_fp8kv_static(C.byref(p), _lib.current_stream(dev))
    assert rc == _lib.ERR_UNSUPPORTED and "static scratch" in _lib.last_error()
    with pytest.raises(NotImplementedError, match="static scratch"):
        amd.decode_fp8kv(q, kq, kq, sc, sc, out=out, static_scratch=True)
    # the same call with a workspace of the caller's is served
    o2, _ = amd.decode_fp8kv(q, kq, kq, sc, sc)
    torch.cuda.synchronize()
    assert torch.equal(o2, torch.zeros_like(o2))
