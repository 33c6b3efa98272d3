"""Host side of the fused attention path: marshals torch tensors into the C ABI.

Everything here is plumbing - allocation of outputs with the layout rules of the operator
contract, argument normalisation and error mapping.  All arithmetic happens in the HIP
kernels behind ``libmi355_sdpa.so``.
"""

from __future__ import annotations

import ctypes as C
import math

import torch

from . import _lib


def _require_cuda(t: torch.Tensor, name: str) -> None:
    if t.device.type != "cuda":
        raise ValueError(f"Expected a GPU tensor for {name}, got {t.device}")


def make_desc(query, key, value, attn_bias=None, dropout_p=0.0, is_causal=False,
              return_debug_mask=False, scale=None, requires_lse=True) -> _lib.Desc:
    """Shape/dtype descriptor for the host-logic entry points (works for meta/CPU tensors)."""
    d = _lib.Desc()
    d.q_dim, d.k_dim, d.v_dim = query.dim(), key.dim(), value.dim()
    symbolic = False
    for arr, t in ((d.q_size, query), (d.k_size, key), (d.v_size, value)):
        for i in range(min(4, t.dim())):
            s = t.shape[i]
            if isinstance(s, int):
                arr[i] = s
            else:
                symbolic = True
                arr[i] = 1
    d.q_dtype, d.k_dtype, d.v_dtype = (_lib.dtype_id(t.dtype) for t in (query, key, value))
    d.on_device = int(all(t.device.type == "cuda" for t in (query, key, value)))
    d.has_symbolic_shape = int(symbolic)
    d.has_attn_bias = int(attn_bias is not None)
    d.is_causal = int(bool(is_causal))
    d.return_debug_mask = int(bool(return_debug_mask))
    d.has_scale = int(scale is not None)
    d.scale = float(scale) if scale is not None else 0.0
    d.dropout_p = float(dropout_p)
    d.requires_lse = int(requires_lse)
    strides = []
    for t in (query, key, value):
        st = t.stride(-1) if t.dim() > 0 and not symbolic else 1
        strides.append(int(st) if isinstance(st, int) else 1)
    d.q_last_stride, d.k_last_stride, d.v_last_stride = strides
    return d


def validate(desc: _lib.Desc) -> None:
    """Raise RuntimeError with the operator-boundary message if the call breaks the contract."""
    buf = C.create_string_buffer(512)
    if _lib.load().mi355_sdpa_validate(C.byref(desc), buf, 512) != 0:
        raise RuntimeError(buf.value.decode())


def choose_backend(desc: _lib.Desc) -> int:
    return _lib.load().mi355_sdpa_choose_backend(C.byref(desc))


def can_use_fused_fwd(desc: _lib.Desc) -> int:
    return _lib.load().mi355_sdpa_can_use_fused_fwd(C.byref(desc))


def can_use_fused_bwd(desc: _lib.Desc) -> int:
    return _lib.load().mi355_sdpa_can_use_fused_bwd(C.byref(desc))


def out_strides(ref_sizes, ref_strides, out_sizes):
    arr = lambda v: (C.c_int64 * 4)(*[int(x) for x in v])
    res = (C.c_int64 * 4)()
    _lib.load().mi355_sdpa_out_strides(arr(ref_sizes), arr(ref_strides), arr(out_sizes), res)
    return tuple(res)


def empty_like_layout(ref: torch.Tensor, shape, dtype=None) -> torch.Tensor:
    """New tensor of ``shape`` whose dimension order follows ``ref`` (stride-0 dims never alias)."""
    if ref.is_contiguous() and 0 not in ref.shape:  # the common case needs no stride arithmetic
        return torch.empty(tuple(shape), dtype=dtype or ref.dtype, device=ref.device)
    st = out_strides(ref.shape, ref.stride(), shape)
    return torch.empty_strided(tuple(shape), st, dtype=dtype or ref.dtype, device=ref.device)


def _unit_last(t: torch.Tensor) -> torch.Tensor:
    return t if t.stride(-1) == 1 or t.size(-1) <= 1 else t.contiguous()


def _bias_view(attn_bias, B, Hq, L, S, repack_for=None):
    """``attn_bias`` expanded to ``(B,Hq,L,S)`` (stride 0 on broadcast dims) and its dtype id.

    ``repack_for``: the dtype of the query, for calls that may run in the matrix-op kernels.  Those read
    the bias a dword at a time: a bias whose rows do not start on dwords or are not whole dwords (a
    16-bit bias over an odd number of keys, a slice that starts at an odd element, a bool mask over a
    number of keys that is no multiple of four) is copied once, over its own extents - broadcast dims
    stay broadcast - into a layout they take: the same dtype where that can be aligned, float32
    otherwise (an additive 0 / -inf tensor for a bool mask).  One pass over the bias, against a call
    that would otherwise leave the matrix-op kernels altogether."""
    if attn_bias is None:
        return None, 0
    b = attn_bias
    while b.dim() < 4:
        b = b.unsqueeze(0)
    b = b.expand(B, Hq, L, S)
    if repack_for is not None and not _dword_rows(b, S):
        own = b[tuple(slice(0, 1) if (b.stride(i) == 0 and b.size(i) > 1) else slice(None) for i in range(4))]
        if own.dtype == torch.bool:
            tgt = repack_for if (S % 2 == 0 and repack_for in (torch.float16, torch.bfloat16)) else torch.float32
            own = torch.zeros(own.shape, dtype=tgt, device=own.device).masked_fill_(~own, float("-inf"))
        else:
            gran = max(4 // own.element_size(), 1)
            own = own.contiguous() if S % gran == 0 else own.to(torch.float32).contiguous()
        b = own.expand(B, Hq, L, S)
    return b, _lib.dtype_id(b.dtype)


def padded_keep_mask(B, Hq, L, S, device, dtype=torch.uint8):
    """An uninitialised ``(B,Hq,L,S)`` keep-mask whose rows start on dwords (a view of rows padded to a
    multiple of four bytes where ``S`` is none): the layout that every kernel takes as it is."""
    S4 = -(-S // 4) * 4
    return torch.empty((B, Hq, L, S4), dtype=dtype, device=device)[..., :S]


def _keep_rows(keep, B, Hq, L, S, dtype):
    """The dropout keep-mask as bytes in a layout the kernels take: ``(B,Hq,L)`` rows densely packed at
    one pitch.  The matrix-op kernels for 16-bit inputs read the bytes a dword at a time, so for them a
    mask whose rows do not start on dwords (``S`` no multiple of four: 197 image patches, a batch padded
    to its longest sequence) is copied once into rows padded to one - against a call that would
    otherwise run in the generic kernels, a hundred times slower.  ``padded_keep_mask`` makes masks
    that need no copy."""
    keep = keep.expand(B, Hq, L, S)
    if keep.dtype != torch.uint8:
        keep = keep.to(torch.uint8)
    ld = keep.stride(2) if L > 1 else max(keep.stride(2), S)
    packed = (keep.stride(3) == 1 or S == 1) and ld >= S and keep.stride(1) == L * ld and keep.stride(0) == Hq * L * ld
    if packed and (dtype == torch.float32 or (ld % 4 == 0 and keep.data_ptr() % 4 == 0)):
        return keep if L > 1 or keep.stride(2) == ld else keep.as_strided(keep.shape, (Hq * L * ld, L * ld, ld, 1))
    if dtype == torch.float32 or S % 4 == 0:
        return keep.contiguous()
    out = padded_keep_mask(B, Hq, L, S, keep.device)
    out.copy_(keep)
    return out


def _dword_rows(b, S) -> bool:
    if b.dtype not in (torch.bool, torch.float16, torch.bfloat16, torch.float32):
        return True  # (not a dtype the matrix-op kernels take: nothing to gain)
    gran = max(4 // b.element_size(), 1)
    if S > 1 and b.stride(3) != 1:
        return False
    if b.data_ptr() % 4 != 0 or S % gran != 0:
        return False
    return all(b.size(i) <= 1 or b.stride(i) % gran == 0 for i in range(3))


def mask_tile_maps(attn_bias, B, Hq, L, S):
    """Tile skip tables of a bias / keep-mask (``mi355_sdpa_mask_tiles``): ``(live, live_t)`` int32
    device tensors, or ``None`` for a mask that cannot have them (a mask per key, more than 32768
    keys, rows that are not dword aligned).  Valid as long as the mask's contents are unchanged."""
    bias, bias_dt = _bias_view(attn_bias, B, Hq, L, S)
    if bias is None:
        return None
    lib = _lib.load()
    t4 = _lib.tensor4(bias)
    w, wt = C.c_size_t(0), C.c_size_t(0)
    _lib.check(lib.mi355_sdpa_mask_tiles_words(C.byref(t4), bias_dt, C.byref(w), C.byref(wt)))
    if w.value == 0:
        return None
    live = torch.empty((w.value,), dtype=torch.int32, device=bias.device)
    live_t = torch.empty((max(wt.value, 1),), dtype=torch.int32, device=bias.device)
    with _lib.on_device(bias.device):
        rc = lib.mi355_sdpa_mask_tiles(C.byref(t4), bias_dt, live.data_ptr(), live_t.data_ptr(),
                                       _lib.current_stream(bias.device))
    _lib.check(rc)
    return live, live_t


def mask_verdict(attn_bias, B, Hq, L, S):
    """The device-side verdict about a bias / keep-mask (``mi355_sdpa_mask_verdict``): an int32 device
    tensor for ``sdpa_forward(..., mask_verdict=)``, or ``None`` for a mask that cannot have one.
    ``[0]`` kind (0 no pattern, 1 keep-everything, 2 causal, 3 sliding window), ``[1]`` window,
    ``[2]`` sink keys, ``[3]`` 1 if a batch keeps fewer than ``S`` keys, ``[8 + b]`` keys of batch ``b``."""
    bias, bias_dt = _bias_view(attn_bias, B, Hq, L, S)
    if bias is None:
        return None
    lib = _lib.load()
    t4 = _lib.tensor4(bias)
    words = lib.mi355_sdpa_mask_verdict_words(C.byref(t4), bias_dt)
    if words == 0:
        return None
    verdict = torch.empty((words,), dtype=torch.int32, device=bias.device)
    with _lib.on_device(bias.device):
        _lib.check(lib.mi355_sdpa_mask_verdict(C.byref(t4), bias_dt, verdict.data_ptr(), _lib.current_stream(bias.device)))
    return verdict


def _mask_spec(spec, query, S, window, sink_keys, sink_logit, live_tiles=None, score_mods=None):
    """Fill the functor part of a parameter block; returns ``(sink logits as passed to the library or
    None, the tensors that must stay alive over the launch)``."""
    spec.window = int(window or 0)
    spec.sink_keys = int(sink_keys or 0)
    if live_tiles is not None:
        spec.live_tiles, spec.live_tiles_t = live_tiles[0].data_ptr(), live_tiles[1].data_ptr()
    B, Hq, L = query.shape[0], query.shape[1], query.shape[2]
    keep = []
    z = None
    if sink_logit is not None:
        # (Hq,), (B, Hq) or (B, Hq, n): n logits per head (flex_attention_bwd.py.jinja:103)
        z = sink_logit.to(device=query.device, dtype=torch.float32)
        if z.dim() <= 1 or (z.dim() == 2 and z.numel() == Hq):
            z = z.reshape(1, Hq)
        if z.dim() == 2:
            z = z.expand(B, Hq).contiguous()
        else:
            z = z.expand(B, Hq, z.shape[2]).contiguous()
            spec.n_sink_logits = int(z.shape[2])
        spec.sink_logit = z.data_ptr()
    if score_mods:
        f32 = lambda t, shape, name: _fixed(t, torch.float32, shape, name, query.device)
        i32 = lambda t, shape, name: _fixed(t, torch.int32, shape, name, query.device)
        m = score_mods
        if m.get("softcap"):
            spec.softcap = float(m["softcap"])
        if m.get("alibi_slopes") is not None:
            keep.append(f32(m["alibi_slopes"], (Hq,), "alibi_slopes"))
            spec.alibi_slopes = keep[-1].data_ptr()
        if m.get("key_bias") is not None:
            keep.append(f32(m["key_bias"], (Hq, S), "key_bias"))
            spec.key_bias = keep[-1].data_ptr()
        if m.get("key_weight") is not None:
            keep.append(f32(m["key_weight"], (Hq, S), "key_weight"))
            spec.key_weight = keep[-1].data_ptr()
        dq_, dk_ = m.get("doc_ids_q"), m.get("doc_ids_k")
        if (dq_ is None) != (dk_ is None):
            raise ValueError("doc_ids_q and doc_ids_k come together")
        if dq_ is not None:
            keep.append(i32(dq_, (B, L), "doc_ids_q"))
            spec.doc_ids_q = keep[-1].data_ptr()
            keep.append(i32(dk_, (B, S), "doc_ids_k"))
            spec.doc_ids_k = keep[-1].data_ptr()
            spec.doc_ids_sorted = int(bool(m.get("doc_ids_sorted")))
    return z, keep


def _fixed(t, dtype, shape, name, device):
    """``t`` as a contiguous device tensor of ``dtype`` and ``shape`` (a leading dim of 1, or a
    missing one, is broadcast)."""
    t = torch.as_tensor(t).to(device=device, dtype=dtype)
    while t.dim() < len(shape):
        t = t.unsqueeze(0)
    if t.dim() != len(shape) or any(a != b and a != 1 for a, b in zip(t.shape, shape)):
        raise ValueError(f"{name} must have shape {tuple(shape)}, got {tuple(t.shape)}")
    return t.expand(*shape).contiguous()


_SCORE_MOD_KEYS = ("alibi_slopes", "softcap", "key_bias", "key_weight", "doc_ids_q", "doc_ids_k", "doc_ids_sorted")


def _score_mods(kw):
    m = {k: kw.pop(k) for k in _SCORE_MOD_KEYS if k in kw}
    if kw:
        raise TypeError(f"unexpected arguments: {sorted(kw)}")
    live = any(m.get(k) is not None for k in _SCORE_MOD_KEYS if k not in ("softcap", "doc_ids_sorted"))
    return m if live or (m.get("softcap") or 0) > 0 else None


def sdpa_forward(query, key, value, attn_bias=None, is_causal=False, scale=None, dropout_p=0.0,
                 dropout_keep=None, kv_lens=None, need_lse=True, force_kernel=0,
                 window=None, sink_keys=0, sink_logit=None, live_tiles=None, mask_verdict=None,
                 seq_major_out=False, **score_mods):
    """Fused forward.  K/V arrive at ``Hkv`` heads.  Returns ``(out, lse)``; ``out`` keeps the
    dimension order of ``query`` and ``lse`` is contiguous float32 ``(B,Hq,L)``.

    ``live_tiles``: the ``(live, live_t)`` pair of ``mask_tile_maps`` for this ``attn_bias`` (or
    ``True`` to build it here): the kernels then skip the tiles that the mask drops whole.
    ``mask_verdict``: what ``mask_verdict`` below wrote about this ``attn_bias``: where the verdict
    names the causal or the keep-everything pattern, the kernels generate it and read no mask.

    ``window`` (with ``is_causal``): query ``i`` sees keys ``i-window+1 .. i`` and the first
    ``sink_keys`` keys; ``sink_logit`` ``(B,Hq)``, ``(Hq,)`` or ``(B,Hq,n)``: logits that join every
    row's softmax and carry no value.

    Score functors (keyword only), applied to ``s = scale * q.k`` in this order: ``key_weight``
    ``(Hq,S)`` multiplies, ``key_bias`` ``(Hq,S)`` is added, ``alibi_slopes`` ``(Hq,)`` adds
    ``slope[h] * (j - i)``, ``softcap`` turns ``s`` into ``softcap * tanh(s / softcap)``;
    ``doc_ids_q`` ``(B,L)`` / ``doc_ids_k`` ``(B,S)`` keep a score iff the two ids are equal
    (``doc_ids_sorted=True``: the caller's promise that both are non-decreasing along the sequence,
    which lets the kernels skip the key tiles of other documents).

    ``seq_major_out``: ``out`` is laid out ``(B,L,Hq,Dv)`` in memory whatever the query's layout, which
    is what upstream's memory-efficient operator promises its callers."""
    score_mods = _score_mods(score_mods)
    for t, n in ((query, "query"), (key, "key"), (value, "value")):
        _require_cuda(t, n)
    B, Hq, L, E = query.shape
    S, Dv = key.shape[2], value.shape[3]
    if scale is None:
        scale = 1.0 / math.sqrt(E)
    q, k, v = _unit_last(query), _unit_last(key), _unit_last(value)
    if seq_major_out:
        out = torch.empty((B, L, Hq, Dv), dtype=query.dtype, device=query.device).transpose(1, 2)
    else:
        out = empty_like_layout(query, (B, Hq, L, Dv))
        if out.stride(-1) != 1 and Dv > 1:
            out = torch.empty((B, Hq, L, Dv), dtype=query.dtype, device=query.device)
    lse = torch.empty((B, Hq, L), dtype=torch.float32, device=query.device) if need_lse else None
    bias, bias_dt = _bias_view(attn_bias, B, Hq, L, S, repack_for=None if force_kernel == _lib.KERNEL_GENERIC else query.dtype)
    p, P = _lib.FwdParams(), _lib.FwdParams
    for f, t in ((P.q, q), (P.k, k), (P.v, v), (P.out, out), (P.bias, bias)):
        _lib.put4(p, f, t)
    p.lse = lse.data_ptr() if lse is not None else None
    p.bias_dtype = bias_dt
    if kv_lens is not None:
        kv_lens = kv_lens.to(device=query.device, dtype=torch.int32).contiguous()
        p.kv_lens = kv_lens.data_ptr()
    if dropout_p > 0.0:
        if dropout_keep is None:
            raise ValueError("dropout_p > 0 needs dropout_keep")
        if not 0.0 <= dropout_p <= 1.0:
            raise ValueError(f"dropout_p={dropout_p} is outside [0, 1]. Pass a value in [0, 1].")
        if dropout_keep.numel() <= 1:
            dropout_p = 0.0  # a mask of one element is the reference's placeholder for none (torch_neuronx/_sdpa_math.py:42-45)
        else:
            dropout_keep = _keep_rows(dropout_keep, B, Hq, L, S, query.dtype)
            p.dropout_keep, p.dropout_keep_ld = dropout_keep.data_ptr(), dropout_keep.stride(2)
    p.dropout_p = float(dropout_p)
    p.dtype = _lib.dtype_id(query.dtype)
    p.is_causal, p.scale, p.force_kernel = int(bool(is_causal)), float(scale), int(force_kernel)
    if live_tiles is True:
        live_tiles = mask_tile_maps(attn_bias, B, Hq, L, S)
    _z = _mask_spec(p.mask, query, S, window, sink_keys, sink_logit, live_tiles, score_mods)  # noqa: F841 (kept alive over the launch)
    if mask_verdict is not None:
        p.mask.mask_verdict = mask_verdict.data_ptr()
    ws = None
    if L <= 128:
        # few query rows: the library may want to split the keys over more workgroups
        need = _lib.load().mi355_sdpa_fwd_workspace_bytes(C.byref(p))
        if need:
            ws = torch.empty(need, dtype=torch.uint8, device=query.device)
            p.workspace, p.workspace_bytes = ws.data_ptr(), need
    with _lib.on_device(query.device):
        rc = _lib.load().mi355_sdpa_fwd(C.byref(p), _lib.current_stream(query.device))
    _lib.check(rc)
    return out, lse


def sdpa_backward(grad_out, query, key, value, out, lse, attn_bias=None, is_causal=False,
                  scale=None, dropout_p=0.0, dropout_keep=None, kv_lens=None,
                  want_grad_bias=False, force_kernel=0, window=None, sink_keys=0, sink_logit=None,
                  live_tiles=None, mask_verdict=None, seq_major_grads=False, grad_bias_row_pad=4, **score_mods):
    """Fused backward.  Returns ``(dq, dk, dv, dbias-or-None)``; each gradient keeps the
    dimension order of its input, dk/dv come back at ``Hkv`` heads.  With a ``sink_logit`` a
    fifth element follows: its gradient, float32 ``(B,Hq)`` or ``(B,Hq,n)``.  Score functors as in
    ``sdpa_forward``: their derivative multiplies the gradient of the scores; the captured vectors
    get no gradient of their own.

    ``seq_major_grads``: dq, dk and dv are laid out ``(B,L,H,D)`` in memory whatever the inputs' layouts,
    and ``grad_bias_row_pad = 16`` leaves the bias gradient as a view of rows padded to 16 keys: the
    layouts upstream's memory-efficient backward promises its callers."""
    score_mods = _score_mods(score_mods)
    for t, n in ((grad_out, "grad_out"), (query, "query"), (key, "key"), (value, "value")):
        _require_cuda(t, n)
    B, Hq, L, E = query.shape
    Hkv, S, Dv = key.shape[1], key.shape[2], value.shape[3]
    if scale is None:
        scale = 1.0 / math.sqrt(E)
    go, q, k, v, o = (_unit_last(t) for t in (grad_out, query, key, value, out))
    lse = lse.to(torch.float32).contiguous()

    def grad_like(ref, shape):
        if seq_major_grads:
            return torch.empty((shape[0], shape[2], shape[1], shape[3]), dtype=ref.dtype, device=ref.device).transpose(1, 2)
        g = empty_like_layout(ref, shape)
        if g.stride(-1) != 1 and shape[-1] > 1:
            g = torch.empty(shape, dtype=ref.dtype, device=ref.device)
        return g

    dq, dk, dv = grad_like(query, (B, Hq, L, E)), grad_like(key, (B, Hkv, S, E)), grad_like(value, (B, Hkv, S, Dv))
    bias, bias_dt = _bias_view(attn_bias, B, Hq, L, S, repack_for=None if force_kernel == _lib.KERNEL_GENERIC else query.dtype)
    dbias = None
    if want_grad_bias and bias is not None:
        # (the matrix-op kernels for 16-bit inputs write the gradient four keys at a time: rows padded to that)
        S4 = S if (query.dtype == torch.float32 or L == 1) and grad_bias_row_pad <= 4 else -(-S // grad_bias_row_pad) * grad_bias_row_pad
        dbias = torch.empty((B, Hq, L, S4), dtype=query.dtype, device=query.device)[..., :S]
    p, P = _lib.BwdParams(), _lib.BwdParams
    for f, t in ((P.grad_out, go), (P.q, q), (P.k, k), (P.v, v), (P.out, o), (P.grad_q, dq), (P.grad_k, dk),
                 (P.grad_v, dv), (P.bias, bias), (P.grad_bias, dbias)):
        _lib.put4(p, f, t)
    p.lse = lse.data_ptr()
    p.bias_dtype = bias_dt
    if kv_lens is not None:
        kv_lens = kv_lens.to(device=query.device, dtype=torch.int32).contiguous()
        p.kv_lens = kv_lens.data_ptr()
    if dropout_p > 0.0:
        if dropout_keep is None:
            raise ValueError("dropout_p > 0 needs dropout_keep")
        if not 0.0 <= dropout_p <= 1.0:
            raise ValueError(f"dropout_p={dropout_p} is outside [0, 1]. Pass a value in [0, 1].")
        if dropout_keep.numel() <= 1:
            dropout_p = 0.0  # a mask of one element is the reference's placeholder for none (torch_neuronx/_sdpa_math.py:42-45)
        else:
            dropout_keep = _keep_rows(dropout_keep, B, Hq, L, S, query.dtype)
            p.dropout_keep, p.dropout_keep_ld = dropout_keep.data_ptr(), dropout_keep.stride(2)
    p.dropout_p = float(dropout_p)
    p.dtype = _lib.dtype_id(query.dtype)
    p.is_causal, p.scale, p.force_kernel = int(bool(is_causal)), float(scale), int(force_kernel)
    if live_tiles is True:
        live_tiles = mask_tile_maps(attn_bias, B, Hq, L, S)
    _z, _keep = _mask_spec(p.mask, query, S, window, sink_keys, sink_logit, live_tiles, score_mods)
    if mask_verdict is not None:
        p.mask.mask_verdict = mask_verdict.data_ptr()
    dsink = None
    if _z is not None:
        dsink = torch.empty(_z.shape, dtype=torch.float32, device=query.device)
        p.grad_sink_logit = dsink.data_ptr()
    lib = _lib.load()
    nbytes = lib.mi355_sdpa_bwd_workspace_bytes(C.byref(p))
    ws = torch.empty((max(nbytes, 1),), dtype=torch.uint8, device=query.device)
    p.workspace, p.workspace_bytes = ws.data_ptr(), nbytes
    with _lib.on_device(query.device):
        rc = lib.mi355_sdpa_bwd(C.byref(p), _lib.current_stream(query.device))
    _lib.check(rc)
    if dbias is not None and dbias.stride(2) != S and L > 1 and grad_bias_row_pad <= 4:
        dbias = dbias.contiguous()  # (rows were padded for the kernel)
    if _z is not None:
        return dq, dk, dv, dbias, dsink
    return dq, dk, dv, dbias


def decode_fp8kv(query, k_fp8, v_fp8, k_scale, v_scale, kv_lens=None, scale=None,
                 num_splits=0, need_lse=True, out=None, lse=None, static_scratch=False):
    """Decode-step attention over an fp8 e4m3 K/V cache.  Returns ``(out, lse)``.

    With ``static_scratch=True`` the call goes through ``mi355_sdpa_decode_fp8kv_static``, which
    allocates nothing: the caller passes ``out`` (and ``lse`` if wanted), ``k_scale`` / ``v_scale`` /
    ``kv_lens`` must already be contiguous float32 / int32 device tensors, and nothing is allocated
    here either."""
    for t, n in ((query, "query"), (k_fp8, "key"), (v_fp8, "value")):
        _require_cuda(t, n)
    if k_fp8.dtype != torch.float8_e4m3fn or v_fp8.dtype != torch.float8_e4m3fn:
        raise RuntimeError("decode_fp8kv: key and value must be float8_e4m3fn")
    B, Hq, Lq, D = query.shape
    if scale is None:
        scale = 1.0 / math.sqrt(D)
    if static_scratch:
        if out is None:
            raise ValueError("decode_fp8kv: static_scratch=True needs a preallocated out")
        for t, n, dt in ((k_scale, "k_scale", torch.float32), (v_scale, "v_scale", torch.float32),
                         (kv_lens, "kv_lens", torch.int32)):
            if t is not None and (t.dtype != dt or not t.is_contiguous() or t.device != query.device):
                raise ValueError(f"decode_fp8kv: with static_scratch=True {n} must be a contiguous {dt} tensor on the query's device")
        for t, n in ((query, "query"), (k_fp8, "key"), (v_fp8, "value"), (out, "out")):
            if t.stride(-1) != 1:
                raise ValueError(f"decode_fp8kv: with static_scratch=True {n} must have unit stride on the head dim")
        q, k, v, ks, vs = query, k_fp8, v_fp8, k_scale, v_scale
    else:
        q, k, v = _unit_last(query), _unit_last(k_fp8), _unit_last(v_fp8)
        if out is None:
            out = torch.empty((B, Hq, Lq, v.shape[3]), dtype=query.dtype, device=query.device)
        if lse is None and need_lse:
            lse = torch.empty((B, Hq, Lq), dtype=torch.float32, device=query.device)
        ks = k_scale.to(device=query.device, dtype=torch.float32).contiguous()
        vs = v_scale.to(device=query.device, dtype=torch.float32).contiguous()
        if kv_lens is not None:
            kv_lens = kv_lens.to(device=query.device, dtype=torch.int32).contiguous()
    if tuple(out.shape) != (B, Hq, Lq, v.shape[3]) or out.dtype != query.dtype:
        raise ValueError("decode_fp8kv: out must have shape (B, Hq, Lq, D) and the query's dtype")
    if lse is not None and (tuple(lse.shape) != (B, Hq, Lq) or lse.dtype != torch.float32 or not lse.is_contiguous()):
        raise ValueError("decode_fp8kv: lse must be a contiguous float32 (B, Hq, Lq) tensor")
    p, P = _lib.DecodeParams(), _lib.DecodeParams
    for f, t in ((P.q, q), (P.k, k), (P.v, v), (P.out, out)):
        _lib.put4(p, f, t)
    p.k_scale, p.v_scale = ks.data_ptr(), vs.data_ptr()
    if kv_lens is not None:
        p.kv_lens = kv_lens.data_ptr()
    p.lse = lse.data_ptr() if lse is not None else None
    p.q_dtype, p.scale, p.num_splits = _lib.dtype_id(query.dtype), float(scale), int(num_splits)
    lib = _lib.load()
    if static_scratch:
        with _lib.on_device(query.device):
            rc = lib.mi355_sdpa_decode_fp8kv_static(C.byref(p), _lib.current_stream(query.device))
        _lib.check(rc)
        return out, lse
    nbytes = lib.mi355_sdpa_decode_workspace_bytes(C.byref(p))
    ws = torch.empty((max(nbytes, 1),), dtype=torch.uint8, device=query.device)
    p.workspace, p.workspace_bytes = ws.data_ptr(), nbytes
    with _lib.on_device(query.device):
        rc = lib.mi355_sdpa_decode_fp8kv(C.byref(p), _lib.current_stream(query.device))
    _lib.check(rc)
    return out, lse
