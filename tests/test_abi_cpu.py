"""CPU-side checks of the C ABI and the host logic: the library loads, exports every symbol
the header declares, the ctypes mirror matches the C structs, and the boundary rules
(validation messages, backend choice, output layout, kernel gates) hold.  No kernel runs."""

import ctypes as C
import os
import re
import subprocess
import sys

import pytest
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "mi355_sdpa.h")


@pytest.fixture(scope="module")
def amd():
    import torch_neuronx_amd as amd
    from torch_neuronx_amd import _build

    if not os.path.exists(_build.LIB_PATH):
        _build.build()
    return amd


def _declared_symbols():
    text = open(HEADER).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(mi355_sdpa_[a-z0-9_]+)\s*\(", text)))


def test_library_exports_every_declared_symbol(amd):
    lib = amd._lib.load()
    names = _declared_symbols()
    assert len(names) >= 12
    for n in names:
        assert hasattr(lib, n), n
    assert set(names) == set(amd._lib.EXPORTS)
    assert lib.mi355_sdpa_abi_version() == 6


def test_ctypes_structs_match_c_layout(amd, tmp_path):
    src = tmp_path / "sizes.c"
    src.write_text(
        '#include <stdio.h>\n#include <stddef.h>\n#include "mi355_sdpa.h"\n'
        "int main(void){\n"
        'printf("%zu %zu %zu %zu %zu\\n", sizeof(mi355_sdpa_tensor), sizeof(mi355_sdpa_desc),'
        " sizeof(mi355_sdpa_fwd_params), sizeof(mi355_sdpa_bwd_params), sizeof(mi355_sdpa_decode_params));\n"
        'printf("%zu %zu %zu %zu\\n", offsetof(mi355_sdpa_fwd_params, scale), offsetof(mi355_sdpa_bwd_params, workspace),'
        " offsetof(mi355_sdpa_decode_params, workspace), offsetof(mi355_sdpa_desc, q_last_stride));\n"
        'printf("%zu %zu %zu %zu\\n", sizeof(mi355_sdpa_mask_spec), offsetof(mi355_sdpa_fwd_params, mask),'
        " offsetof(mi355_sdpa_bwd_params, mask), offsetof(mi355_sdpa_bwd_params, grad_sink_logit));\n"
        "return 0;}\n"
    )
    exe = tmp_path / "sizes"
    subprocess.run(["gcc", "-I", os.path.join(ROOT, "include"), str(src), "-o", str(exe)], check=True)
    out = subprocess.run([str(exe)], capture_output=True, text=True, check=True).stdout.split()
    L = amd._lib
    got = [C.sizeof(L.Tensor4), C.sizeof(L.Desc), C.sizeof(L.FwdParams), C.sizeof(L.BwdParams), C.sizeof(L.DecodeParams),
           L.FwdParams.scale.offset, L.BwdParams.workspace.offset, L.DecodeParams.workspace.offset,
           L.Desc.q_last_stride.offset,
           C.sizeof(L.MaskSpec), L.FwdParams.mask.offset, L.BwdParams.mask.offset, L.BwdParams.grad_sink_logit.offset]
    assert [int(x) for x in out] == got


def _desc(amd, q, k, v, **kw):
    return amd.ops.make_desc(q, k, v, **kw)


def _meta(*shape, dtype=torch.bfloat16, device="meta"):
    return torch.empty(*shape, dtype=dtype, device=device)


def test_validation_messages_match_the_operator_contract(amd):
    # messages: torch_neuronx/csrc/core/dispatch/NeuronDispatcher.cpp:2377-2459
    q, k, v = _meta(2, 8, 16, 64), _meta(2, 2, 16, 64), _meta(2, 2, 16, 64)
    amd.ops.validate(_desc(amd, q, k, v))
    cases = [
        (dict(return_debug_mask=True), (q, k, v), "return_debug_mask=True is not supported"),
        (dict(attn_bias=_meta(16, 16), is_causal=True), (q, k, v),
         "Explicit attn_mask should not be set when is_causal=True"),
        ({}, (_meta(2, 8, 16, 64, dtype=torch.int32), k, v), "query dtype must be float32, float16, or bfloat16, got"),
        ({}, (q, k.float(), v), "query, key, value must have the same dtype"),
        ({}, (_meta(8, 16, 64), k, v), "must be 4D tensors (B, H, S, D)"),
        ({}, (q, _meta(3, 2, 16, 64), _meta(3, 2, 16, 64)), "batch sizes must match"),
        ({}, (q, k, _meta(2, 4, 16, 64)), "key and value must have the same number of heads"),
        ({}, (q, k, _meta(2, 2, 17, 64)), "key and value must have the same sequence length"),
        ({}, (q, _meta(2, 3, 16, 64), _meta(2, 3, 16, 64)),
         "Number of heads in key and value must divide the number of heads in query"),
        (dict(dropout_p=1.5), (q, k, v), "is outside [0, 1]"),
    ]
    for kw, (qq, kk, vv), msg in cases:
        with pytest.raises(RuntimeError) as e:
            amd.ops.validate(_desc(amd, qq, kk, vv, **kw))
        assert msg in str(e.value), (msg, str(e.value))
    # float64 is accepted at the boundary (computed as float32)
    amd.ops.validate(_desc(amd, q.double(), k.double(), v.double()))
    # a float64 query makes the reference downcast every float64 operand before it compares dtypes
    # (NeuronDispatcher.cpp:2418-2432): float32 key / value pass with it, the reverse does not
    amd.ops.validate(_desc(amd, q.double(), k.float(), v.float()))
    amd.ops.validate(_desc(amd, q.double(), k.double(), v.float()))
    with pytest.raises(RuntimeError, match="must have the same dtype"):
        amd.ops.validate(_desc(amd, q.float(), k.double(), v.double()))
    with pytest.raises(RuntimeError, match="must have the same dtype"):
        amd.ops.validate(_desc(amd, q.double(), k, v))


def test_backend_choice_rules(amd):
    # rules: torch_neuronx/csrc/aten/SdpBackendSelection.cpp:29-67
    L = amd._lib

    def choice(q, k, v, on_device=True):
        d = _desc(amd, q, k, v)
        d.on_device = int(on_device)
        return amd.ops.choose_backend(d)

    q, k, v = _meta(2, 8, 16, 64), _meta(2, 2, 16, 64), _meta(2, 2, 16, 64)
    assert choice(q, k, v) == L.BACKEND_OVERRIDEABLE == 4
    assert choice(q, k, v, on_device=False) == L.BACKEND_MATH == 0
    assert choice(_meta(8, 16, 64), k, v) == 0
    assert choice(_meta(2, 8, 16, 0), _meta(2, 2, 16, 0), v) == 0  # zero-size head dim
    assert choice(q, _meta(2, 2, 0, 64), _meta(2, 2, 0, 64)) == 0  # no keys
    assert choice(q, k, _meta(2, 2, 16, 0)) == 0
    d = _desc(amd, q, k, v)
    d.on_device, d.has_symbolic_shape = 1, 1
    assert amd.ops.choose_backend(d) == 0


@pytest.mark.parametrize("make", [
    lambda: torch.empty(2, 4, 16, 8),
    lambda: torch.empty(2, 16, 4, 8).transpose(1, 2),
    lambda: torch.empty(2, 16, 4, 24).transpose(1, 2)[..., 8:16],
    lambda: torch.empty(16, 2, 4, 8).permute(1, 2, 0, 3),
    lambda: torch.empty(2, 1, 16, 8).expand(2, 4, 16, 8),
    lambda: torch.empty(1, 4, 16, 8).expand(2, 4, 16, 8),
    lambda: torch.empty(1, 1, 16, 8).expand(2, 4, 16, 8),      # strides (0, 0, 8, 1)
    lambda: torch.empty(16, 8).expand(2, 4, 16, 8).transpose(1, 2).transpose(1, 2),
    lambda: torch.empty(2, 16, 1, 8).expand(2, 16, 4, 8).transpose(1, 2),  # stride 0 in the middle of a permuted view
    lambda: torch.empty(2, 4, 40, 8)[:, :, ::2][:, :, :16],
    lambda: torch.empty(2, 4, 1, 8).expand(2, 4, 16, 8),       # ties between real strides
    lambda: torch.empty(2, 4, 16, 1).expand(2, 4, 16, 8),
])
def test_out_strides_follow_alloc_with_matching_layout(amd, make):
    # the rule of torch._meta_registrations.alloc_with_matching_layout, which the reference uses for
    # outputs and gradients (scaled_dot_product_fused_attention.py:357, :601-603): empty_like when the
    # shapes agree, else dense strides in the reference tensor's dimension order
    from torch._meta_registrations import alloc_with_matching_layout

    ref = make()
    for shape in [(2, 4, 16, 8), (2, 4, 16, 5), (2, 4, 16, 0), (2, 4, 3, 8)]:
        want = alloc_with_matching_layout(ref, shape)
        got = amd.ops.out_strides(ref.shape, ref.stride(), shape)
        assert got == want.stride(), (ref.stride(), shape)
        t = amd.ops.empty_like_layout(ref, shape)
        assert t.shape == shape and t.stride() == want.stride()


def test_kernel_gates(amd):
    # this library's own gate table, the analogue of decompositions.py:2161-2207 / :2371-2424
    L = amd._lib

    def gate(q, k, v, **kw):
        d = _desc(amd, q, k, v, **kw)
        return amd.ops.can_use_fused_fwd(d), amd.ops.can_use_fused_bwd(d)

    q, k, v = _meta(1, 32, 8192, 128), _meta(1, 8, 8192, 128), _meta(1, 8, 8192, 128)
    assert gate(q, k, v, is_causal=True) == (L.KERNEL_MFMA, L.KERNEL_MFMA)
    assert gate(q.half(), k.half(), v.half()) == (L.KERNEL_MFMA, L.KERNEL_MFMA)
    assert gate(q.float(), k.float(), v.float()) == (L.KERNEL_MFMA, L.KERNEL_MFMA)  # float32 matrix op
    assert gate(q.float(), k.float(), v.float(), attn_bias=_meta(8192, 8192)) == (L.KERNEL_MFMA, L.KERNEL_MFMA)
    assert gate(q, k, v, attn_bias=_meta(8192, 8192)) == (L.KERNEL_MFMA, L.KERNEL_MFMA)  # masked calls too
    q64, k64 = _meta(1, 8, 512, 64), _meta(1, 8, 512, 64)
    assert gate(q64, k64, k64, attn_bias=_meta(512, 512)) == (L.KERNEL_MFMA, L.KERNEL_MFMA)
    assert gate(q, k, v, dropout_p=0.1) == (L.KERNEL_MFMA, L.KERNEL_MFMA)  # dropout: 16-bit, head dims up to 128, no bias
    assert gate(q, k, v, dropout_p=0.1, attn_bias=_meta(8192, 8192)) == (L.KERNEL_MFMA, L.KERNEL_MFMA)  # ... with a bias too
    assert gate(q.float(), k.float(), v.float(), dropout_p=0.1) == (L.KERNEL_MFMA, L.KERNEL_MFMA)
    assert gate(q.float(), k.float(), v.float(), dropout_p=0.1, attn_bias=_meta(8192, 8192)) == (L.KERNEL_MFMA, L.KERNEL_MFMA)
    assert gate(q, k, v, scale=0.0) == (L.KERNEL_GENERIC, L.KERNEL_GENERIC)
    assert gate(q, k, v, scale=0.25) == (L.KERNEL_MFMA, L.KERNEL_MFMA)
    q96 = _meta(2, 8, 512, 96)  # narrow head dims (multiples of 8) run padded in the next wider kernel
    assert gate(q96, q96, q96, is_causal=True) == (L.KERNEL_MFMA, L.KERNEL_MFMA)
    q256 = _meta(2, 8, 512, 256)  # head dims up to 256, forward and backward
    assert gate(q256, q256, q256) == (L.KERNEL_MFMA, L.KERNEL_MFMA)
    assert gate(q256, q256, q256, dropout_p=0.1) == (L.KERNEL_MFMA, L.KERNEL_MFMA)  # dropout at every width
    q100 = _meta(2, 8, 512, 100)
    assert gate(q100, q100, q100) == (L.KERNEL_GENERIC, L.KERNEL_GENERIC)
    q2, k2 = _meta(1, 4, 64, 192), _meta(1, 4, 64, 192)
    assert gate(q2, k2, _meta(1, 4, 64, 128)) == (L.KERNEL_MFMA, L.KERNEL_MFMA)  # D_qk > D_v (192 / 128)
    assert gate(_meta(1, 4, 64, 64), _meta(1, 4, 64, 64), _meta(1, 4, 64, 128)) == (L.KERNEL_GENERIC, L.KERNEL_GENERIC)
    assert gate(_meta(1, 4, 64, 640), _meta(1, 4, 64, 640), _meta(1, 4, 64, 640)) == (L.KERNEL_NONE, L.KERNEL_NONE)
    assert gate(q, _meta(1, 3, 8192, 128), _meta(1, 3, 8192, 128)) == (L.KERNEL_NONE, L.KERNEL_NONE)
    assert gate(_meta(1, 4, 0, 64), _meta(1, 4, 16, 64), _meta(1, 4, 16, 64)) == (L.KERNEL_NONE, L.KERNEL_NONE)
    assert gate(q, k, v, return_debug_mask=True) == (L.KERNEL_NONE, L.KERNEL_NONE)


def test_entry_points_reject_bad_arguments_without_a_gpu(amd):
    lib = amd._lib.load()
    assert lib.mi355_sdpa_fwd(None, None) == amd._lib.ERR_INVALID
    assert "null" in amd._lib.last_error()
    p = amd._lib.FwdParams()
    assert lib.mi355_sdpa_fwd(C.byref(p), None) == amd._lib.ERR_INVALID
    assert "query" in amd._lib.last_error()
    assert lib.mi355_sdpa_bwd(None, None) == amd._lib.ERR_INVALID
    assert lib.mi355_sdpa_decode_fp8kv(None, None) == amd._lib.ERR_INVALID
    assert lib.mi355_sdpa_bwd_workspace_bytes(None) == 0


def test_host_ops_refuse_cpu_tensors(amd):
    q = torch.randn(1, 2, 4, 8)
    with pytest.raises(ValueError):
        amd.sdpa_forward(q, q, q)
    with pytest.raises(ValueError):
        amd.python_ops.scaled_dot_product_fused_attention_overrideable(q, q, q)
    with pytest.raises(ValueError):
        amd.native_multi_head_attn_mid(q, q, q)


def test_registered_operator_surface(amd):
    names = amd.registered_ops()
    for n in ("_scaled_dot_product_fused_attention_overrideable",
              "_scaled_dot_product_fused_attention_overrideable_backward",
              "_scaled_dot_product_flash_attention", "_scaled_dot_product_flash_attention_backward"):
        assert n in names
    s = torch.ops.mi355_kernels.scaled_dot_product_attention_kernel.default._schema
    assert [a.name for a in s.arguments] == ["q", "k", "v", "is_causal", "dropout_p", "scale", "training", "seed", "lse"]
    s = torch.ops.mi355_kernels.scaled_dot_product_attention_backward_kernel.default._schema
    assert [a.name for a in s.arguments] == ["grad_out", "q", "k", "v", "out", "lse", "is_causal", "dropout_p", "scale", "seed"]
    assert hasattr(torch.ops.mi355_kernels, "sdpa_decode_fp8kv")


def test_missing_library_fails_loudly(amd, monkeypatch):
    from torch_neuronx_amd import _lib

    monkeypatch.setattr(_lib, "_lib", None)
    monkeypatch.setattr(_lib, "LIB_PATH", "/nonexistent/libmi355_sdpa.so")
    with pytest.raises(RuntimeError, match="no fallback"):
        _lib.load()


def _resource_usage():
    """Per-kernel figures the compiler reported when the library was built."""
    from torch_neuronx_amd import _build

    if not os.path.exists(_build.RESOURCE_PATH):
        _build.build()
    rows = {}
    for line in open(_build.RESOURCE_PATH):
        src, name, *kv = line.split()
        rows[name] = dict(src=src, **{k: v for k, v in (x.split("=", 1) for x in kv)})
    return rows


def test_hot_kernels_use_no_scratch_and_keep_their_occupancy():
    # The hand-scheduled MFMA kernels count on every value living in a register: a spill puts
    # scratch loads/stores (vector memory ops the hand-counted waits know nothing of) into their
    # loops.  Checked on what the compiler reported for the library that the tests load.
    import re

    rows = _resource_usage()
    assert len(rows) > 50
    fwd = {n: r for n, r in rows.items() if "fwd_w32_kernel" in n}
    assert len(fwd) >= 30
    # the full-width wide dK/dV kernel holds 512 registers as it is: with a mask it is known to spill
    # a few, and without one the compiler parks some accumulators in scratch while it writes the
    # results out, after the loops (seen in the generated code: no scratch access before the last barrier);
    # its functor mode keeps a second packed copy of the probabilities and spills more.  That file
    # waits for every load at once (no counted waits), so a spill there costs time, not correctness.
    known = re.compile(r"bwd_wide_dkdv_kernelIDF16[b_]Li256ELi256ELi([0123])ELb([01])EE")
    for name, r in rows.items():
        if r["src"] not in ("fwd_mfma_w32.hip", "bwd_dq_w32.hip", "bwd_dkdv_w32.hip", "bwd_wide.hip", "decode_fp8kv.hip"):
            continue
        scratch = int(r["ScratchSize_[bytes/lane]"])
        if "decode_kernelIfLi256ELi1ELi3EE" in name:  # float32 queries at head dim 256, 9-16 rows: a dozen bytes, no counted waits there
            assert scratch <= 16, (name, scratch)
            continue
        if re.search(r"bwd_dkdv_w32_kernelIDF16[b_]Li128ELi5E", name):
            # dropout together with a bias at head dim 128: 32 bias elements and 32 keep bytes of a tile in
            # flight at once; the counted waits of that file stay valid under extra scratch traffic (a
            # wait that allows N loads in flight covers everything older, whatever the N youngest are)
            assert scratch <= 112, (name, scratch)
            continue
        m = known.search(name)
        if m:
            # (masked with skip tables and no split: the spill in the loop alone; the instances that
            # split: the write-out's as well)
            mode, tables = int(m.group(1)), int(m.group(2))
            # (functor and dropout modes: a second packed copy of the probabilities, the functors' operands or the keep bits)
            assert scratch <= (288 if mode >= 2 else 64 if (mode == 1 and tables == 1) else 96), (name, scratch)
            continue
        assert scratch == 0, (name, scratch)
        assert r["Dynamic_Stack"] == "False"
    for name, r in fwd.items():
        d = int(re.search(r"Li(\d+)ELi\d+ELi\d+E(?:Lb[01]E)?E", name).group(1))
        assert int(r["Occupancy_[waves/SIMD]"]) >= (1 if d > 128 else 2), name
