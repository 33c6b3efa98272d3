"""CPU oracle for fused scaled-dot-product attention.  TEST INFRASTRUCTURE ONLY.

This module restates, with plain PyTorch CPU ops, the numerical definition the
reference uses for its attention path.  It is the checker for the HIP kernels:
only the tests, the smoke check and the CPU-baseline leg of the benchmark may
import it.  Nothing in the shipped package calls into it.

What each function follows in the reference (paths relative to the reference
tree):

* ``accumulator_dtype``            torch_neuronx/_sdpa_math.py:6-7
* ``masked_logits``                torch_neuronx/_sdpa_math.py:15-33 and :82-83
* ``compute_attention``            torch_neuronx/_sdpa_math.py:51-95
* ``compute_attention_backward``   torch_neuronx/_sdpa_math.py:98-176
* ``normalize_sdpa_args``          torch_neuronx/neuron_dynamo_backend/decompositions.py:2083-2104
* ``reduce_gqa_gradients``         torch_neuronx/neuron_dynamo_backend/decompositions.py:2569-2599
* ``sdpa_forward`` / ``sdpa_backward``  the eager wrapper order expand -> math -> reduce,
  torch_neuronx/python_ops/torch_mlir/ops/scaled_dot_product_attention.py:134-195,411-462

* ``apply_score_mods`` / ``functor_keep_mask`` / ``sdpa_forward_score_mod`` / ``sdpa_backward_score_mod``
  the order in which the reference's templated kernels apply what a caller's score_mod / mask_mod
  compute: scale * q.k, then score_mod, then the mask
  (torch_neuronx/neuron_dynamo_backend/flex_attention/flex_attention.py.jinja:74-92, :2495-2660),
  the backward with joint_mod, the derivative of score_mod, applied to the softmax gradient
  (flex_attention_bwd.py.jinja:958-988, :1250-1275), sink logits ``[bs, nheads]`` or
  ``[bs, nheads, num_sinks]`` (flex_attention_bwd.py.jinja:103, :316-320); the functors themselves
  are the ones of the reference's tests
  (tests/neuron_dynamo_backend/unit/fx/passes/test_flex_attention_legalization.py:1051-1066, :1207-1218)

Parity pins (tests/test_oracle.py): float64 ``F.scaled_dot_product_attention``,
float64 ``torch.logsumexp``, a pure-Python triple loop on tiny inputs, autograd
through the forward, row-sum identities of the backward, GQA == MHA on repeated
heads, fully-masked-row behaviour and the saturation invariants of the
reference's own CPU tests.

PARITY UNPINNED: ``quantize_kv_fp8`` / ``decode_fp8kv`` have no counterpart in
the reference (it has no fp8 attention path); they are pinned only by their own
definition (per-(batch, kv-head) scale = amax/448, ``torch.float8_e4m3fn`` cast)
plus the float64 SDPA check of the dequantised problem.
"""

from __future__ import annotations

import math

import torch

NEG_INF = float("-inf")


def accumulator_dtype(dtype: torch.dtype) -> torch.dtype:
    """Half-precision inputs accumulate in float32; everything else keeps its dtype."""
    if dtype is torch.float16 or dtype is torch.bfloat16:
        return torch.float32
    return dtype


def _bias_present_fwd(attn_bias) -> bool:
    # forward: an empty tensor means "no bias"  (_sdpa_math.py:30)
    return attn_bias is not None and attn_bias.numel() > 0


def _bias_present_bwd(attn_bias) -> bool:
    # backward: a single-element placeholder also means "no bias" (_sdpa_math.py:142)
    return attn_bias is not None and attn_bias.numel() > 1


def _dropout_active(dropout_mask, dropout_p: float) -> bool:
    if not 0.0 <= dropout_p <= 1.0:
        raise ValueError(f"dropout_p={dropout_p} is outside [0, 1]. Pass a value in [0, 1].")
    return dropout_p > 0.0 and dropout_mask is not None and dropout_mask.numel() > 1


def _dropout(x, dropout_mask, dropout_p: float):
    if not _dropout_active(dropout_mask, dropout_p):
        return x
    kept = x * dropout_mask
    return kept if dropout_p == 1.0 else kept / (1.0 - dropout_p)


def masked_logits(q_acc, k_acc, scale: float, attn_bias, is_causal: bool):
    """``(Q K^T) * scale`` in the accumulator dtype, causal fill first, bias added after.

    The causal pattern is the lower triangle of an ``L x S`` matrix anchored at the
    top-left corner, also when ``L != S``.
    """
    s = torch.matmul(q_acc, k_acc.transpose(-2, -1)) * scale
    if is_causal:
        L, S = s.shape[-2], s.shape[-1]
        row = torch.arange(L).unsqueeze(-1)
        col = torch.arange(S).unsqueeze(0)
        s = s.masked_fill(col > row, NEG_INF)
    if attn_bias is not None:
        s = s + attn_bias
    return s


def compute_attention(query, key, value, attn_bias, dropout_mask, scale, is_causal, dropout_p):
    """Forward for already head-expanded ``(B,H,L,E)/(B,H,S,E)/(B,H,S,Dv)`` operands.

    Returns ``(output in query.dtype, logsumexp float32 (B,H,L))``.  A row whose
    logits are all ``-inf`` yields a zero output row and ``lse = -inf``.
    """
    in_dtype = query.dtype
    acc = accumulator_dtype(in_dtype)
    bias = attn_bias if _bias_present_fwd(attn_bias) else None
    s = masked_logits(query.to(acc), key.to(acc), scale, bias, is_causal)

    row_max = s.amax(dim=-1, keepdim=True)
    dead = row_max == NEG_INF
    shift = torch.where(dead, torch.zeros_like(row_max), row_max)
    e = torch.exp(s - shift)
    denom = e.sum(dim=-1, keepdim=True)
    lse = (row_max + torch.log(denom)).squeeze(-1)
    p = e / torch.where(dead, torch.ones_like(denom), denom)
    p = _dropout(p, dropout_mask, dropout_p)
    out = torch.matmul(p.to(in_dtype), value)
    return out, lse.to(torch.float32)


def compute_attention_backward(
    grad_out, query, key, value, attn_bias, dropout_mask, out, lse, scale, is_causal, dropout_p,
    bias_present=None,
):
    """Backward for head-expanded operands; returns ``(dQ, dK, dV, dBias-or-None)``.

    Everything runs in the accumulator dtype and only the results are rounded.  The
    row term is ``sum_j dP_ij P_ij + sum_d dO_id (O_id - (P V)_id)``: with the true
    output it reduces to ``rowsum(dO * O)``; the second part matters when ``out`` is
    a globally merged output and this call sees one block of keys.
    """
    in_dtype = query.dtype
    acc = accumulator_dtype(in_dtype)
    go, q, k, v, o = (t.to(acc) for t in (grad_out, query, key, value, out))
    lse = lse.to(acc)
    # (bias_present: the decision of a caller that hands in one slice of a larger bias)
    with_bias = _bias_present_bwd(attn_bias) if bias_present is None else bias_present
    # a one-element bias is a lowering placeholder: ignored here, while the forward
    # (numel > 0) would still add it
    bias = attn_bias.to(acc) if with_bias else None
    s = masked_logits(q, k, scale, bias, is_causal)

    dead = (lse == NEG_INF).unsqueeze(-1)
    p = torch.exp(s - torch.where(dead, torch.zeros_like(lse.unsqueeze(-1)), lse.unsqueeze(-1)))
    p = torch.where(dead, torch.zeros_like(p), p)

    p_drop = _dropout(p, dropout_mask, dropout_p)
    d_v = torch.matmul(p_drop.transpose(-2, -1), go)
    d_p = _dropout(torch.matmul(go, v.transpose(-2, -1)), dropout_mask, dropout_p)
    block_out = torch.matmul(p_drop, v)
    row_term = (d_p * p).sum(-1, keepdim=True) + (go * (o - block_out)).sum(-1, keepdim=True)
    d_logits = p * (d_p - row_term)
    d_s = d_logits * scale
    d_q = torch.matmul(d_s, k)
    d_k = torch.matmul(d_s.transpose(-2, -1), q)
    d_bias = d_logits.to(in_dtype) if with_bias else None
    return d_q.to(in_dtype), d_k.to(in_dtype), d_v.to(in_dtype), d_bias


def normalize_sdpa_args(query, key, value, attn_mask, scale, enable_gqa=True):
    """Argument rules of the reference adapter: GQA expansion (query head ``h`` reads
    kv head ``h // rep``), default ``scale = 1/sqrt(E)``, boolean mask (True = attend)
    turned into an additive ``0 / -inf`` bias of the query dtype."""
    hq, hkv = query.shape[1], key.shape[1]
    if enable_gqa and hq > hkv and hq % hkv == 0:
        rep = hq // hkv
        key = key.repeat_interleave(rep, dim=1)
        value = value.repeat_interleave(rep, dim=1)
    if scale is None:
        scale = 1.0 / math.sqrt(query.shape[-1])
    if attn_mask is None:
        bias = None
    elif attn_mask.dtype == torch.bool:
        bias = torch.zeros(attn_mask.shape, dtype=query.dtype).masked_fill(~attn_mask, NEG_INF)
    else:
        bias = attn_mask
    return key, value, bias, scale


def reduce_gqa_gradients(grad_k, grad_v, hkv: int):
    """Sum key/value gradients over the query heads that share a kv head."""
    b, hq, s, e = grad_k.shape
    if hq == hkv:
        return grad_k, grad_v
    rep = hq // hkv
    dv = grad_v.shape[-1]
    return (
        grad_k.reshape(b, hkv, rep, s, e).sum(dim=2),
        grad_v.reshape(b, hkv, rep, s, dv).sum(dim=2),
    )


def _head_slices(hq: int, chunk: int):
    for h0 in range(0, hq, chunk):
        yield h0, min(hq, h0 + chunk)


def _as_4d(mask):
    """Masks broadcast from the right: pad leading dimensions up to (B, H, L, S)."""
    if mask is None:
        return None
    while mask.dim() < 4:
        mask = mask.unsqueeze(0)
    return mask


def _chunk_for(L: int, S: int, budget_bytes: int = 1 << 30) -> int:
    per_head = max(1, L * S * 4)
    return max(1, budget_bytes // per_head)


def sdpa_forward(query, key, value, attn_mask=None, is_causal=False, scale=None, head_chunk=None):
    """Whole forward at the operator boundary: K/V arrive at ``Hkv`` heads.

    Runs head-chunked per batch so the ``L x S`` temporaries stay bounded; the
    arithmetic per head is exactly ``compute_attention``.
    """
    B, Hq, L, _ = query.shape
    Hkv, S = key.shape[1], key.shape[2]
    rep = Hq // Hkv
    if scale is None:
        scale = 1.0 / math.sqrt(query.shape[-1])
    chunk = head_chunk or _chunk_for(L, S)
    attn_mask = _as_4d(attn_mask)
    out = torch.empty(B, Hq, L, value.shape[-1], dtype=query.dtype)
    lse = torch.empty(B, Hq, L, dtype=torch.float32)
    for b in range(B):
        for h0, h1 in _head_slices(Hq, chunk):
            heads = torch.arange(h0, h1)
            kb = key[b : b + 1, heads // rep]
            vb = value[b : b + 1, heads // rep]
            mask = None
            if attn_mask is not None:
                mask = attn_mask[b : b + 1] if attn_mask.shape[0] > 1 else attn_mask
                if mask.shape[1] > 1:
                    mask = mask[:, h0:h1]
            _, _, bias, _ = normalize_sdpa_args(query[b : b + 1, h0:h1], kb, vb, mask, scale, False)
            o, l_ = compute_attention(
                query[b : b + 1, h0:h1], kb, vb, bias, None, scale, is_causal, 0.0
            )
            out[b, h0:h1] = o[0]
            lse[b, h0:h1] = l_[0]
    return out, lse


def sdpa_backward(
    grad_out, query, key, value, out, lse, attn_mask=None, is_causal=False, scale=None,
    head_chunk=None, reduce_in_fp32=False,
):
    """Whole backward at the operator boundary; dK/dV come back at ``Hkv`` heads.

    The reference rounds per-head gradients to the input dtype and then sums the
    group (``reduce_in_fp32=False``).  ``reduce_in_fp32=True`` sums float32 per-head
    gradients instead, which is the float32 target the kernels are compared with.
    """
    B, Hq, L, E = query.shape
    Hkv, S = key.shape[1], key.shape[2]
    rep = Hq // Hkv
    if scale is None:
        scale = 1.0 / math.sqrt(E)
    chunk = head_chunk or _chunk_for(L, S)
    attn_mask = _as_4d(attn_mask)
    res_dtype = torch.float32 if reduce_in_fp32 else query.dtype
    dq = torch.empty(B, Hq, L, E, dtype=res_dtype)
    dk = torch.zeros(B, Hkv, S, E, dtype=res_dtype)
    dv = torch.zeros(B, Hkv, S, value.shape[-1], dtype=res_dtype)
    cast = (lambda t: t.float()) if reduce_in_fp32 else (lambda t: t)
    for b in range(B):
        for h0, h1 in _head_slices(Hq, chunk):
            heads = torch.arange(h0, h1)
            sel = lambda t: t[b : b + 1, h0:h1]
            kb = cast(key[b : b + 1, heads // rep])
            vb = cast(value[b : b + 1, heads // rep])
            mask = None
            if attn_mask is not None:
                mask = attn_mask[b : b + 1] if attn_mask.shape[0] > 1 else attn_mask
                if mask.shape[1] > 1:
                    mask = mask[:, h0:h1]
            _, _, bias, _ = normalize_sdpa_args(cast(sel(query)), kb, vb, mask, scale, False)
            # the one-element-placeholder rule applies to the bias of the whole call, not to the
            # slice of it that this chunk sees
            gq, gk, gv, _ = compute_attention_backward(
                cast(sel(grad_out)), cast(sel(query)), kb, vb, bias, None,
                cast(sel(out)), sel(lse), scale, is_causal, 0.0,
                bias_present=None if attn_mask is None else _bias_present_bwd(attn_mask),
            )
            dq[b, h0:h1] = gq[0]
            dk[b].index_add_(0, heads // rep, gk[0])
            dv[b].index_add_(0, heads // rep, gv[0])
    return dq, dk, dv


# --------------------------------------------------------------------------------------
# Mask / score functors: sliding window, sink keys, sink logit.  The reference takes
# ``sliding_window`` and ``sink`` as arguments of its templated kernel
# (torch_neuronx/neuron_dynamo_backend/flex_attention/flex_attention.py.jinja:94-117; the sink
# joins the row maximum :1921-1923 and the exponential sum :2134-2140), but the rendered mask
# function is not in the tree, so the window's boundary convention here is this build's:
# a window of ``window`` keys that ends at the query's own position.  PARITY UNPINNED by the
# reference's tests; pinned by float64 ``F.scaled_dot_product_attention`` on the explicit mask
# with the sink as one more key of value zero (tests/test_oracle.py).
# --------------------------------------------------------------------------------------


def window_keep_mask(L: int, S: int, window: int, sink_keys: int = 0) -> torch.Tensor:
    """Boolean ``(L, S)`` keep-mask: causal (top-left), and key ``j`` within the last
    ``window`` positions of query ``i`` or among the first ``sink_keys`` keys."""
    row = torch.arange(L).unsqueeze(-1)
    col = torch.arange(S).unsqueeze(0)
    keep = col <= row
    if window and window > 0:
        keep = keep & ((row - col < window) | (col < sink_keys))
    return keep


def _with_sink(query, key, value, bias, sink_logit):
    """The sink as one more key: zero key and value rows and a bias column holding the logit."""
    B, Hq, L, _ = query.shape
    S = key.shape[2]
    z = sink_logit.to(torch.float32).reshape(-1, Hq).expand(B, Hq)
    key = torch.cat([key, key.new_zeros(key.shape[0], key.shape[1], 1, key.shape[3])], dim=2)
    value = torch.cat([value, value.new_zeros(value.shape[0], value.shape[1], 1, value.shape[3])], dim=2)
    full = torch.zeros(B, Hq, L, S + 1, dtype=torch.float32)
    if bias is not None:
        full[..., :S] = bias
    full[..., S] = z[:, :, None]
    return key, value, full


def sdpa_forward_functor(query, key, value, is_causal=False, scale=None, window=0, sink_keys=0, sink_logit=None):
    """Forward with the mask functors; K/V at ``Hkv`` heads.  Returns ``(out, lse)``."""
    B, Hq, L, E = query.shape
    S = key.shape[2]
    rep = Hq // key.shape[1]
    if scale is None:
        scale = 1.0 / math.sqrt(E)
    k = key.repeat_interleave(rep, dim=1)
    v = value.repeat_interleave(rep, dim=1)
    bias = None
    if is_causal or window:
        keep = window_keep_mask(L, S, window, sink_keys) if window else (torch.arange(S)[None] <= torch.arange(L)[:, None])
        bias = torch.zeros(L, S, dtype=torch.float32).masked_fill(~keep, NEG_INF)
    if sink_logit is not None:
        k, v, bias = _with_sink(query, k, v, bias, sink_logit)
    return compute_attention(query, k, v, bias, None, scale, False, 0.0)


def sdpa_backward_functor(grad_out, query, key, value, out, lse, is_causal=False, scale=None, window=0,
                          sink_keys=0, sink_logit=None):
    """Backward with the mask functors: ``(dq, dk, dv, dsink-or-None)`` in float32, dk/dv at ``Hkv`` heads."""
    B, Hq, L, E = query.shape
    Hkv, S = key.shape[1], key.shape[2]
    rep = Hq // Hkv
    if scale is None:
        scale = 1.0 / math.sqrt(E)
    k = key.float().repeat_interleave(rep, dim=1)
    v = value.float().repeat_interleave(rep, dim=1)
    bias = None
    if is_causal or window:
        keep = window_keep_mask(L, S, window, sink_keys) if window else (torch.arange(S)[None] <= torch.arange(L)[:, None])
        bias = torch.zeros(1, 1, L, S, dtype=torch.float32).masked_fill(~keep, NEG_INF).expand(B, Hq, L, S)
    if sink_logit is not None:
        k, v, bias = _with_sink(query, k, v, None if bias is None else bias, sink_logit)
    gq, gk, gv, gb = compute_attention_backward(grad_out.float(), query.float(), k, v, bias, None, out.float(), lse,
                                                scale, False, 0.0, bias_present=bias is not None)
    dsink = None
    if sink_logit is not None:
        dsink = gb[..., S].sum(-1)
        gk, gv = gk[:, :, :S], gv[:, :, :S]
    gk, gv = reduce_gqa_gradients(gk, gv, Hkv)
    return gq, gk, gv, dsink


# --------------------------------------------------------------------------------------
# Score functors and index-computed masks (the score_mod / mask_mod / joint_mod of the
# reference's templated kernels), written out on the full L x S score matrix.
# --------------------------------------------------------------------------------------


def apply_score_mods(scores, alibi_slopes=None, softcap=0.0, key_bias=None, key_weight=None):
    """``scores`` = ``scale * q.k`` as ``(B,Hq,L,S)`` -> ``(modified scores, derivative of the
    modification with respect to the score)``.  Order: ``* key_weight[h,j]``, ``+ key_bias[h,j]``,
    ``+ alibi_slopes[h] * (j - i)``, ``softcap * tanh(. / softcap)``."""
    B, Hq, L, S = scores.shape
    s = scores
    d = torch.ones_like(scores)
    if key_weight is not None:
        w = key_weight.to(s.dtype).reshape(1, Hq, 1, S)
        s = s * w
        d = d * w
    if key_bias is not None:
        s = s + key_bias.to(s.dtype).reshape(1, Hq, 1, S)
    if alibi_slopes is not None:
        rel = (torch.arange(S)[None, :] - torch.arange(L)[:, None]).to(s.dtype)
        s = s + alibi_slopes.to(s.dtype).reshape(1, Hq, 1, 1) * rel
    if softcap and softcap > 0:
        th = torch.tanh(s / softcap)
        s = softcap * th
        d = d * (1.0 - th * th)
    return s, d


def functor_keep_mask(B, L, S, is_causal=False, window=0, sink_keys=0, doc_ids_q=None, doc_ids_k=None):
    """Boolean ``(B or 1, 1, L, S)`` keep-mask of the index-computed masks, or ``None`` for none."""
    keep = None
    if is_causal or window:
        keep = (window_keep_mask(L, S, window, sink_keys) if window
                else (torch.arange(S)[None] <= torch.arange(L)[:, None]))[None, None]
    if doc_ids_q is not None:
        same = (doc_ids_q.reshape(-1, L)[:, :, None] == doc_ids_k.reshape(-1, S)[:, None, :])[:, None]
        keep = same if keep is None else keep & same
    return keep


def _sink_columns(sink_logit, B, Hq):
    """``(B,Hq,n)`` float32 sink logits from ``(Hq,)``, ``(B,Hq)`` or ``(B,Hq,n)``."""
    z = sink_logit.to(torch.float32)
    if z.dim() <= 1 or (z.dim() == 2 and z.numel() == Hq):
        z = z.reshape(1, Hq)
    if z.dim() == 2:
        z = z[:, :, None]
    return z.expand(B, Hq, z.shape[2])


def sdpa_forward_score_mod(query, key, value, is_causal=False, scale=None, window=0, sink_keys=0, sink_logit=None,
                           alibi_slopes=None, softcap=0.0, key_bias=None, key_weight=None, doc_ids_q=None,
                           doc_ids_k=None):
    """Forward with score functors, index masks and sink logits; K/V at ``Hkv`` heads.  Float32
    accumulation, probabilities rounded to the input dtype before ``P V`` (as ``compute_attention``).
    Returns ``(out, lse)``."""
    B, Hq, L, E = query.shape
    S = key.shape[2]
    rep = Hq // key.shape[1]
    if scale is None:
        scale = 1.0 / math.sqrt(E)
    in_dtype = query.dtype
    acc = accumulator_dtype(in_dtype)
    k = key.repeat_interleave(rep, dim=1)
    v = value.repeat_interleave(rep, dim=1)
    s = torch.matmul(query.to(acc), k.to(acc).transpose(-2, -1)) * scale
    s, _ = apply_score_mods(s, alibi_slopes, softcap, key_bias, key_weight)
    keep = functor_keep_mask(B, L, S, is_causal, window, sink_keys, doc_ids_q, doc_ids_k)
    if keep is not None:
        s = s.masked_fill(~keep, NEG_INF)
    full = s if sink_logit is None else torch.cat([s, _sink_columns(sink_logit, B, Hq)[:, :, None, :].expand(B, Hq, L, -1).to(acc)], -1)
    row_max = full.amax(dim=-1, keepdim=True)
    dead = row_max == NEG_INF
    shift = torch.where(dead, torch.zeros_like(row_max), row_max)
    e = torch.exp(full - shift)
    denom = e.sum(dim=-1, keepdim=True)
    lse = (row_max + torch.log(denom)).squeeze(-1)
    p = (e / torch.where(dead, torch.ones_like(denom), denom))[..., :S]
    out = torch.matmul(p.to(in_dtype), v)
    return out, lse.to(torch.float32)


def sdpa_backward_score_mod(grad_out, query, key, value, out, lse, is_causal=False, scale=None, window=0, sink_keys=0,
                            sink_logit=None, alibi_slopes=None, softcap=0.0, key_bias=None, key_weight=None,
                            doc_ids_q=None, doc_ids_k=None):
    """Backward of ``sdpa_forward_score_mod``: ``(dq, dk, dv, dsink-or-None)`` in float32, dk/dv at
    ``Hkv`` heads.  ``dS = P (dP - rowsum(dO O))`` is the gradient of the MODIFIED scores; the
    derivative of the functors turns it into the gradient of ``scale * q.k``."""
    B, Hq, L, E = query.shape
    Hkv, S = key.shape[1], key.shape[2]
    rep = Hq // Hkv
    if scale is None:
        scale = 1.0 / math.sqrt(E)
    go, q, o = grad_out.float(), query.float(), out.float()
    k = key.float().repeat_interleave(rep, dim=1)
    v = value.float().repeat_interleave(rep, dim=1)
    s = torch.matmul(q, k.transpose(-2, -1)) * scale
    s, dfac = apply_score_mods(s, alibi_slopes, softcap, key_bias, key_weight)
    keep = functor_keep_mask(B, L, S, is_causal, window, sink_keys, doc_ids_q, doc_ids_k)
    if keep is not None:
        s = s.masked_fill(~keep, NEG_INF)
    l = lse.float().unsqueeze(-1)
    dead = l == NEG_INF
    p = torch.where(dead, torch.zeros_like(s), torch.exp(s - torch.where(dead, torch.zeros_like(l), l)))
    delta = (go * o).sum(-1, keepdim=True)
    d_v = torch.matmul(p.transpose(-2, -1), go)
    d_p = torch.matmul(go, v.transpose(-2, -1))
    d_s = p * (d_p - delta) * dfac * scale
    d_q = torch.matmul(d_s, k)
    d_k = torch.matmul(d_s.transpose(-2, -1), q)
    dsink = None
    if sink_logit is not None:
        z = _sink_columns(sink_logit, B, Hq)  # (B,Hq,n): p_sink = exp(z - lse), dP of a sink is 0
        pz = torch.where(dead, torch.zeros_like(l), torch.exp(z[:, :, None, :] - torch.where(dead, torch.zeros_like(l), l)))
        dsink = -(pz * delta).sum(2)
        if sink_logit.dim() < 3:
            dsink = dsink[..., 0]
    d_k, d_v = reduce_gqa_gradients(d_k, d_v, Hkv)
    return d_q, d_k, d_v, dsink


# --------------------------------------------------------------------------------------
# fp8 key/value cache decode.  No reference counterpart: PARITY UNPINNED (see header).
# --------------------------------------------------------------------------------------

FP8_E4M3_MAX = 448.0


def quantize_kv_fp8(x: torch.Tensor):
    """Per-(batch, kv-head) symmetric quantisation to OCP e4m3: ``scale = amax/448``.

    ``x`` is ``(B, Hkv, S, D)`` float32.  Returns ``(x_q float8_e4m3fn, scale (B,Hkv) float32)``.
    """
    amax = x.abs().amax(dim=(-2, -1))
    scale = (amax / FP8_E4M3_MAX).clamp_min(1e-12).to(torch.float32)
    xq = (x / scale[:, :, None, None]).to(torch.float8_e4m3fn)
    return xq, scale


def dequantize_kv_fp8(xq: torch.Tensor, scale: torch.Tensor):
    return xq.to(torch.float32) * scale[:, :, None, None]


def decode_fp8kv(query, k_q, v_q, k_scale, v_scale, kv_lens, scale=None, head_chunk=None):
    """Decode-step attention (``q_len`` small) over an fp8 cache with key padding.

    ``query`` ``(B,Hq,Lq,D)`` bf16/fp16/fp32; ``k_q``/``v_q`` ``(B,Hkv,S,D)`` float8_e4m3fn;
    ``kv_lens`` ``(B,)`` integer: key ``j`` of batch ``b`` takes part iff ``j < kv_lens[b]``.
    The definition is ``compute_attention`` on the dequantised float32 cache with a
    ``0/-inf`` key-padding bias; the output is returned in float32 together with lse.
    """
    B, Hq, Lq, D = query.shape
    Hkv, S = k_q.shape[1], k_q.shape[2]
    rep = Hq // Hkv
    if scale is None:
        scale = 1.0 / math.sqrt(D)
    out = torch.empty(B, Hq, Lq, v_q.shape[-1], dtype=torch.float32)
    lse = torch.empty(B, Hq, Lq, dtype=torch.float32)
    for b in range(B):
        n = int(kv_lens[b])
        if n == 0:  # every key padded away: the fully-masked-row rule of compute_attention
            out[b], lse[b] = 0.0, float("-inf")
            continue
        kb = dequantize_kv_fp8(k_q[b : b + 1, :, :n], k_scale[b : b + 1])
        vb = dequantize_kv_fp8(v_q[b : b + 1, :, :n], v_scale[b : b + 1])
        heads = torch.arange(Hq)
        o, l_ = compute_attention(
            query[b : b + 1].float(), kb[:, heads // rep], vb[:, heads // rep],
            None, None, scale, False, 0.0,
        )
        out[b], lse[b] = o[0], l_[0]
    return out, lse


# --------------------------------------------------------------------------------------
# Independent brute force for tiny inputs (pure Python loops, float64).
# --------------------------------------------------------------------------------------


def brute_force_attention(query, key, value, bias, scale, is_causal):
    """Triple-loop float64 softmax attention on one ``(L,E)/(S,E)/(S,Dv)`` head.

    ``bias`` is ``None`` or an ``(L,S)`` additive tensor.  Returns python lists
    ``(out[L][Dv], lse[L])``.
    """
    L, E = query.shape
    S, Dv = value.shape
    q, k, v = query.double().tolist(), key.double().tolist(), value.double().tolist()
    bb = bias.double().tolist() if bias is not None else None
    out, lses = [], []
    for i in range(L):
        logits = []
        for j in range(S):
            if is_causal and j > i:
                logits.append(NEG_INF)
                continue
            acc = 0.0
            for d in range(E):
                acc += q[i][d] * k[j][d]
            acc *= scale
            if bb is not None:
                acc += bb[i][j]
            logits.append(acc)
        m = max(logits)
        if m == NEG_INF:
            out.append([0.0] * Dv)
            lses.append(NEG_INF)
            continue
        w = [math.exp(x - m) for x in logits]
        z = sum(w)
        out.append([sum(w[j] * v[j][d] for j in range(S)) / z for d in range(Dv)])
        lses.append(m + math.log(z))
    return out, lses
