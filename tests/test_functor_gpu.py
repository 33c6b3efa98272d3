"""GPU parity of the mask / score functors (sliding window, sink keys, sink logit) against the CPU
oracle, forward and backward, through the C ABI.  The functors stand in for the specialisations the
reference renders into its templated kernel (flex_attention.py.jinja:74-117); no mask tensor is read."""

import pytest
import torch

from helpers import max_abs, qkv, rel_err
from oracle import sdpa_math as om

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def amd(gpu_device):
    import torch_neuronx_amd as amd

    return amd


def _run(amd, dev, B, Hq, Hkv, L, E, dtype, window, sink_keys, with_sink, seed, force=0, scale=None):
    q, k, v, go = qkv(B, Hq, Hkv, L, L, E, dtype=dtype, seed=seed, with_do=True)
    z = None
    if with_sink:
        z = torch.randn(B, Hq, generator=torch.Generator().manual_seed(seed + 1)) * 2
    kw = dict(is_causal=True, window=window, sink_keys=sink_keys, sink_logit=None if z is None else z.to(dev), scale=scale)
    qd, kd, vd, god = (t.to(dev) for t in (q, k, v, go))
    out, lse = amd.sdpa_forward(qd, kd, vd, force_kernel=force, **kw)
    res = amd.sdpa_backward(god, qd, kd, vd, out, lse, force_kernel=force, **kw)
    torch.cuda.synchronize()
    ro, rl = om.sdpa_forward_functor(q.float(), k.float(), v.float(), is_causal=True, scale=scale, window=window,
                                     sink_keys=sink_keys, sink_logit=z)
    rdq, rdk, rdv, rdz = om.sdpa_backward_functor(go.float(), q.float(), k.float(), v.float(), ro, rl, is_causal=True,
                                                  scale=scale, window=window, sink_keys=sink_keys, sink_logit=z)
    half = dtype is not torch.float32
    assert max_abs(out, ro) <= (2e-2 if half else 1e-5)
    assert max_abs(lse, rl) <= (5e-3 if half else 1e-5)
    for a, r in zip(res[:3], (rdq, rdk, rdv)):
        assert a.shape == r.shape
        assert max_abs(a, r) <= (5e-2 if half else 5e-5)
        if r.abs().max() > 1e-3:  # (a window of one key has dQ = dK = 0 exactly)
            assert rel_err(a, r) <= (3e-2 if half else 1e-5)
    if with_sink:
        assert max_abs(res[4], rdz) <= (5e-2 if half else 1e-4) and rel_err(res[4], rdz) <= (3e-2 if half else 1e-5)
    else:
        assert len(res) == 4
    return out, lse, res


@pytest.mark.parametrize("window,sink_keys,with_sink", [(5, 0, False), (40, 3, False), (0, 0, True), (17, 2, True), (1, 0, False)])
def test_functors_float32(amd, gpu_device, window, sink_keys, with_sink):
    _run(amd, gpu_device, 2, 4, 2, 77, 32, torch.float32, window, sink_keys, with_sink, seed=window + 3)


@pytest.mark.parametrize("L,E,window,sink_keys,with_sink", [
    (77, 32, 5, 0, False),
    (300, 64, 40, 3, True),
    (512, 128, 100, 40, True),    # several tiles below the window are dropped whole, the sink tiles are not
    (260, 96, 0, 0, True),        # sink logit alone, a narrow head dim
    (130, 16, 1000, 0, False),    # window longer than the sequence
    (200, 256, 70, 5, True),      # the width-256 instances
])
def test_functors_float32_in_the_matrix_op_kernels(amd, gpu_device, L, E, window, sink_keys, with_sink):
    # (forced: the call fails if the float32 matrix-op kernels refuse it)
    _run(amd, gpu_device, 2, 4, 2, L, E, torch.float32, window, sink_keys, with_sink, seed=L + window, force=amd._lib.KERNEL_MFMA)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("L,E,window,sink_keys,with_sink", [
    (512, 128, 128, 0, False),
    (512, 128, 100, 4, False),
    (777, 128, 256, 40, True),
    (1024, 64, 96, 0, True),
    (300, 128, 1000, 0, False),   # window longer than the sequence: plain causal
    (512, 128, 0, 0, True),       # sink logit alone
    (640, 96, 130, 33, True),     # padded head dim
])
def test_functors_half_precision(amd, gpu_device, dtype, L, E, window, sink_keys, with_sink):
    _run(amd, gpu_device, 2, 8, 2, L, E, dtype, window, sink_keys, with_sink, seed=L + window)


@pytest.mark.parametrize("L,E,window,sink_keys,with_sink", [
    (1024, 256, 256, 0, False),   # several tiles below the window dropped whole in every kernel
    (777, 256, 100, 40, True),    # sink keys, a sink logit, ragged tiles
    (640, 192, 130, 33, True),    # a head dim between 128 and 256
    (300, 256, 1000, 0, False),   # window longer than the sequence: plain causal
])
def test_functors_at_head_dims_above_128(amd, gpu_device, L, E, window, sink_keys, with_sink):
    # the forward's functor variant at width 256 and the wide backward kernels' functor mode, forced
    _run(amd, gpu_device, 2, 4, 2, L, E, torch.bfloat16, window, sink_keys, with_sink, seed=L + window, force=amd._lib.KERNEL_MFMA)


def test_window_equals_the_same_mask_as_a_tensor(amd, gpu_device):
    # the functor and the explicit boolean mask of the same pattern give the same result
    dev = gpu_device
    L, W, N = 512, 160, 5
    q, k, v = (t.to(dev) for t in qkv(1, 8, 2, L, L, 128, dtype=torch.bfloat16, seed=9))
    a, la = amd.sdpa_forward(q, k, v, is_causal=True, window=W, sink_keys=N)
    keep = om.window_keep_mask(L, L, W, N).to(dev)
    b, lb = amd.sdpa_forward(q, k, v, attn_bias=keep[None, None])
    assert max_abs(a, b) <= 4e-3 and max_abs(la, lb) <= 1e-4


def test_functor_argument_errors(amd, gpu_device):
    q, k, v = (t.to(gpu_device) for t in qkv(1, 2, 2, 64, 64, 64, dtype=torch.bfloat16, seed=1))
    with pytest.raises(RuntimeError, match="needs is_causal"):
        amd.sdpa_forward(q, k, v, window=8)
    with pytest.raises(RuntimeError, match="negative"):
        amd.sdpa_forward(q, k, v, is_causal=True, window=-1)
    with pytest.raises(RuntimeError, match="sink_keys needs"):
        amd.sdpa_forward(q, k, v, is_causal=True, sink_keys=4)
