"""Recognise attention masks that a kernel can generate by itself.

The reference recovers causality at trace time: its graph pass proves that an explicit mask is
lower-triangular and rewrites the call to ``is_causal=True``, so that the fused kernel stays
eligible (torch_neuronx/neuron_dynamo_backend/fx/passes/sdpa_causal_mask.py:162-289); with a mask
its fused path is refused (decompositions.py:2203).  Here a mask only exists as a tensor, so it is
read on the device (``mi355_sdpa_mask_verdict``: four numbers per row, then one workgroup that
holds them against the patterns) and the verdict stays there: the attention call that follows is
given its address, and its kernels run as the causal / keep-everything kernels with per-batch key
counts when the verdict says so, and with the mask otherwise.  No step of that waits for the
host, so it also works inside a stream capture and for a mask that is new on every call.

A copy of the verdict travels to the host on the side.  Once it has arrived (a later call finds
that out with a query, never a wait) the decision is cached for as long as the tensor is
unchanged: a causal mask, a sliding window with sink keys and a keep-everything mask are then
served by the kernels that generate those patterns from indices and read no mask at all; so are
the masks that model code builds from right padding, with or without causality or a sliding window
folded in (per-batch key counts).
"""

from __future__ import annotations

import contextlib
import ctypes as C
import os
import threading
import weakref
from collections import OrderedDict

import numpy as np
import torch

from . import _lib

_CACHE_ENTRIES = 16
# key -> (entry, weak reference to the mask's storage); an entry is a verdict on its way to the host
# (_Pending) or ("known", pattern).  The cache never keeps a mask alive: an
# entry goes when the storage dies (so its memory cannot come back under the same key with other
# contents; views of one mask, which upstream makes afresh on every call, share the storage and its
# version counter), and what an entry itself holds is a pattern tuple and at most a (B,) tensor of
# key counts.
_cache: "OrderedDict[tuple, tuple]" = OrderedDict()
# A caller that hands in a NEW tensor on every call (upstream's functional API turns a boolean mask
# into a fresh additive one each time before it reaches the fused op) never hits the cache: after
# _MAX_MISSES misses in a row for one signature the masks of that signature get no cache entry (and
# no skip tables), with another try every _RETRY_EVERY calls.
_MAX_MISSES = 3
_RETRY_EVERY = 512
_misses: dict = {}
stats = {"looked": 0, "hits": 0, "left_alone": 0}


_switch = threading.local()


def enabled() -> bool:
    if getattr(_switch, "off", 0):
        return False
    return os.environ.get("TORCH_NEURONX_AMD_RECOVER_MASKS", "1").lower() not in ("0", "false", "off", "no")


@contextlib.contextmanager
def left_alone():
    """Calls made inside this block (on this thread) take their masks as they are: no look at the
    tensor, no cache, no skip tables.  For masks that are written by something torch's version
    counter does not see."""
    _switch.off = getattr(_switch, "off", 0) + 1
    try:
        yield
    finally:
        _switch.off -= 1


def _version(mask: torch.Tensor):
    """The tensor's version counter, or ``None`` for a tensor that has none (created under
    ``torch.inference_mode()``): nothing tells when such a tensor changes, so it is never cached
    and never looked at - it stays the mask it is."""
    if mask.is_inference():
        return None
    return mask._version


def _remember(cache: OrderedDict, key, value, mask: torch.Tensor) -> None:
    def drop(_ref, cache=cache, key=key):
        cache.pop(key, None)

    cache[key] = (value, weakref.ref(mask.untyped_storage(), drop))
    while len(cache) > _CACHE_ENTRIES:
        cache.popitem(last=False)


def _lookup(cache: OrderedDict, key):
    """``(True, value)`` for a live entry, ``(False, None)`` otherwise."""
    hit = cache.get(key)
    if hit is None:
        return False, None
    if hit[1]() is None:  # (the storage died and its callback has not run yet)
        cache.pop(key, None)
        return False, None
    cache.move_to_end(key)
    return True, hit[0]


def _back_off(sig) -> bool:
    """Counts a miss for this signature; True if the mask should be left alone this time."""
    streak = _misses.get(sig, 0)
    _misses[sig] = streak + 1
    return streak >= _MAX_MISSES and (streak - _MAX_MISSES) % _RETRY_EVERY != _RETRY_EVERY - 1


def pattern_from_rows(rows: np.ndarray, L: int, S: int):
    """``rows[i] = (last kept key, kept keys or -1, kept run from key 0, start of the run ending at
    the last kept key)`` -> ``("all",)``, ``("causal",)``, ``("window", W, N)`` or ``None``.

    Causal is anchored top-left (row ``i`` keeps keys ``0 .. min(i, S-1)``); a window keeps keys
    ``i-W+1 .. i`` and the first ``N`` keys.  A candidate is accepted only if the summary of every
    row equals what the pattern would give."""
    if L == 0 or S == 0 or rows.shape != (L, 4):
        return None
    hi, cnt, lead, lo = (rows[:, c].astype(np.int64) for c in range(4))
    if (cnt < 0).any():
        return None
    if (cnt == S).all():
        return ("all",)
    i = np.arange(L, dtype=np.int64)
    hi_c = np.minimum(i, S - 1)
    if not (hi == hi_c).all():
        return None
    lead_full = np.where(hi_c + 1 < S, hi_c + 1, S)
    if (cnt == hi_c + 1).all():
        return ("causal",) if (lead == lead_full).all() and (lo == 0).all() else None
    r = L - 1
    W = int(hi[r] - lo[r] + 1)
    N = int(lead[r]) if lead[r] < lo[r] else 0
    if W <= 0 or lo[r] == 0:
        return None
    lo_w = np.maximum(i - W + 1, 0)
    joined = lo_w <= N  # the window reaches into the sink keys (or to key 0): one run from key 0
    exp_lo = np.where(joined, 0, lo_w)
    exp_lead = np.where(joined, lead_full, N)
    exp_cnt = np.where(joined, hi_c + 1, hi_c - lo_w + 1 + N)
    if (i - W + 1 > hi_c).any():  # a row whose window lies past the last key is dead: not this pattern
        return None
    if (lo == exp_lo).all() and (lead == exp_lead).all() and (cnt == exp_cnt).all():
        return ("window", W, N)
    return None


def lens_pattern_from_rows(rows: np.ndarray, L: int, S: int, rows_broadcast: bool):
    """Masks that depend on the batch the way padding does: ``rows[b, i]`` as in ``pattern_from_rows``
    for every batch ``b`` -> ``("all", lens)`` (batch ``b`` keeps keys ``0 .. lens[b]-1`` in every row)
    or ``("causal", lens)`` (row ``i`` keeps keys ``0 .. min(i, lens[b]-1)``): what model code builds
    when it folds right padding, and causality, into one mask.  ``rows_broadcast``: the mask has one
    row per batch, valid for every query.  ``None`` if some row is anything else."""
    B = rows.shape[0]
    if B == 0 or S == 0 or rows.ndim != 3 or rows.shape[2] != 4:
        return None
    hi, cnt, lead, lo = (rows[:, :, c].astype(np.int64) for c in range(4))
    if (cnt < 0).any() or (lo != 0).any():
        return None
    n = hi[:, -1] + 1  # keys of the batch as its last row sees them
    if (hi == (n - 1)[:, None]).all() and (cnt == n[:, None]).all():  # every row the same run from key 0
        return ("all", n.astype(np.int32))
    if rows_broadcast:
        return None
    i = np.arange(rows.shape[1], dtype=np.int64)[None, :]
    full = hi[:, -1] == min(L - 1, S - 1)  # the last row reaches its diagonal: no key is known to be padding
    n = np.where(full, S, n)
    hi_c = np.minimum(np.minimum(i, S - 1), (n - 1)[:, None])
    if (hi == hi_c).all() and (cnt == hi_c + 1).all():
        return ("causal", n.astype(np.int32))
    return None


def window_lens_pattern_from_rows(rows: np.ndarray, L: int, S: int):
    """A sliding window with sink keys, with or without right padding, per batch: ``rows[b, i]`` as in
    ``pattern_from_rows`` -> ``("window", W, N, lens)`` (row ``i`` of batch ``b`` keeps those of the keys
    ``i-W+1 .. i`` and of the first ``N`` keys that lie below ``lens[b]``; a row whose window lies behind
    its batch's keys keeps the sink keys or nothing) or ``None``.  The keys of a batch are those up to
    the last one any of its rows keeps - all ``S`` when a row reaches the last diagonal element; ``W``
    and ``N`` are read in the last row with keys of its own of the batch with the most keys."""
    if rows.ndim != 3 or rows.shape[0] == 0 or rows.shape[1] != L or rows.shape[2] != 4 or L < 2 or S < 1:
        return None
    hi, cnt, lead, lo = (rows[:, :, c].astype(np.int64) for c in range(4))
    if (cnt < 0).any():
        return None
    top_b = hi.max(axis=1)
    n = np.where(top_b == min(L - 1, S - 1), S, top_b + 1)
    b_sel = int(np.argmax(n))
    if n[b_sel] <= 0:
        return None
    r = min(int(n[b_sel]), L) - 1
    W = int(hi[b_sel, r] - lo[b_sel, r] + 1)
    N = int(lead[b_sel, r]) if lead[b_sel, r] < lo[b_sel, r] else 0
    if W <= 0 or lo[b_sel, r] == 0:
        return None
    i = np.arange(L, dtype=np.int64)[None, :]
    top = np.minimum(np.minimum(i, S - 1), (n - 1)[:, None])
    lo_w = np.maximum(i - W + 1, 0)
    behind = lo_w > top
    joined = ~behind & (lo_w <= N)
    m = np.maximum(np.minimum(N, top + 1), 0)
    e_hi = np.where(behind, m - 1, top)
    e_cnt = np.where(behind, m, np.where(joined, top + 1, top - lo_w + 1 + N))
    e_lead = np.where(behind, m, np.where(joined, top + 1, N))
    e_lo = np.where(behind | joined, 0, lo_w)
    if (hi == e_hi).all() and (cnt == e_cnt).all() and (lead == e_lead).all() and (lo == e_lo).all():
        return ("window", W, N, n.astype(np.int32))
    return None


# A verdict is put to use on the device only where the mask's traffic matters; below, the mask is as
# cheap as the two extra launches (the copy to the host is still made, for the calls that follow).
_MIN_SCORES_ON_DEVICE = 256 * 256


class _Pending:
    """A verdict on the device whose copy to the host is under way (or was not asked for)."""

    __slots__ = ("verdict", "host", "event", "B", "stream")

    def __init__(self, verdict, host, event, B, stream):
        self.verdict, self.host, self.event, self.B, self.stream = verdict, host, event, B, stream

    def usable_on(self, stream) -> bool:
        """The verdict was computed on ``self.stream``: work on another stream has to wait for it
        (through the event, where one was recorded)."""
        if stream == self.stream:
            return True
        if self.event is None:
            return False
        stream.wait_event(self.event)
        return True

    def settled(self) -> bool:
        return self.event is not None and self.event.query()

    def pattern(self):
        """``("all" | "causal" [, key counts]) | ("window", W, N [, key counts]) | None`` from the host copy."""
        h = self.host
        kind, window, sinks, short = (int(x) for x in h[:4])
        if kind in (1, 2):
            name = "all" if kind == 1 else "causal"
            # (the key counts are used where they are: behind the verdict's header, on the device)
            return (name, self.verdict[8:8 + self.B]) if short else (name,)
        if kind == 3:
            return ("window", window, sinks, self.verdict[8:8 + self.B]) if short else ("window", window, sinks)
        return None


def _verdict_words(view: torch.Tensor, dtype_id: int) -> int:
    t4 = _lib.tensor4(view)
    return int(_lib.load().mi355_sdpa_mask_verdict_words(C.byref(t4), dtype_id))


def _launch_verdict(view: torch.Tensor, dtype_id: int, words: int) -> torch.Tensor:
    verdict = torch.empty((words,), dtype=torch.int32, device=view.device)
    t4 = _lib.tensor4(view)
    with _lib.on_device(view.device):
        _lib.check(_lib.load().mi355_sdpa_mask_verdict(C.byref(t4), dtype_id, verdict.data_ptr(), _lib.current_stream(view.device)))
    return verdict


def look(mask: torch.Tensor, B: int, Hq: int, L: int, S: int):
    """What is known about a device mask: ``(pattern, verdict)``.

    ``pattern`` (see ``pattern_from_rows`` / ``lens_pattern_from_rows``) is set when the host
    already knows it: the tensor was seen before, is unchanged (version counter included), and the
    verdict's copy has arrived.  Otherwise ``verdict`` may be an int32 device tensor for the
    attention call (``mask_verdict``): computed now, on the current stream, or found with the
    tensor's cache entry.  ``(None, None)``: a mask that cannot have a verdict (it depends on the
    head, its keys are not unit-stride), or a small one seen for the first time.

    Inside a stream capture, and for tensors without a version counter (made under
    ``torch.inference_mode()``), nothing is cached and nothing found in the cache is used: the
    verdict is computed by the captured work itself, on every replay, from the mask as it then is."""
    if mask.device.type != "cuda":
        return None, None
    dtype_id = _lib.dtype_id(mask.dtype)
    if dtype_id not in (_lib.BOOL, _lib.F32, _lib.F16, _lib.BF16) or L < 1 or S < 1 or B < 1:
        return None, None
    view = mask
    while view.dim() < 4:
        view = view.unsqueeze(0)
    view = view.expand(B, Hq, L, S)
    words = _verdict_words(view, dtype_id)
    if words == 0:
        return None, None
    on_device = L * S >= _MIN_SCORES_ON_DEVICE and L > 1
    version = _version(mask)
    if version is None or torch.cuda.is_current_stream_capturing():
        return None, (_launch_verdict(view, dtype_id, words) if on_device else None)
    key = (mask.data_ptr(), tuple(mask.shape), tuple(mask.stride()), mask.dtype, version, mask.device.index, B, L, S)
    sig = (B, L, S, mask.dtype, mask.device.index)
    found, entry = _lookup(_cache, key)
    if found:
        if isinstance(entry, _Pending):
            if not entry.settled():
                # (the backward of the step that made the entry, typically: no sign that the tensor lives on)
                stats["pending"] = stats.get("pending", 0) + 1
                if on_device and not entry.usable_on(torch.cuda.current_stream(mask.device)):
                    return None, _launch_verdict(view, dtype_id, words)
                return None, (entry.verdict if on_device else None)
            # (still possibly the backward of the step that made the entry: the miss streak stands)
            pat = entry.pattern()
            _remember(_cache, key, ("known", pat), mask)
            entry = ("known", pat)
        else:
            _misses.pop(sig, None)  # (found again after its pattern was known: the caller keeps its masks)
        stats["hits"] += 1
        return entry[1], None
    # A caller that hands in a NEW tensor on every call never finds its entry again: after a few such
    # misses in a row the copy to the host (a pinned buffer, an event) is no longer made for masks of
    # that signature; the verdict on the device still is, where the mask is large enough to matter.
    if _back_off(sig):
        stats["left_alone"] += 1
        if not on_device:
            return None, None
        # (remembered without a copy to the host: the backward of the same step finds it here)
        verdict = _launch_verdict(view, dtype_id, words)
        _remember(_cache, key, _Pending(verdict, None, None, B, torch.cuda.current_stream(mask.device)), mask)
        return None, verdict
    stats["looked"] += 1
    verdict = _launch_verdict(view, dtype_id, words)
    host = torch.empty((8 + B,), dtype=torch.int32, pin_memory=True)
    host.copy_(verdict[:8 + B], non_blocking=True)
    event = torch.cuda.Event()
    stream = torch.cuda.current_stream(mask.device)
    event.record(stream)
    _remember(_cache, key, _Pending(verdict, host, event, B, stream), mask)
    return None, (verdict if on_device else None)


def classify(mask: torch.Tensor, wait: bool = True):
    """Pattern of a device mask as the host knows it (``look`` without the shapes of a call: batch and
    heads are taken from the mask).  With ``wait`` the verdict's copy is awaited: for tools and
    tests, not for the attention calls."""
    view = mask
    while view.dim() < 4:
        view = view.unsqueeze(0)
    B, Hq, L, S = view.shape
    pat, verdict = look(mask, B, Hq, L, S)
    if pat is None and wait and not torch.cuda.is_current_stream_capturing() and _version(mask) is not None:
        torch.cuda.current_stream(mask.device).synchronize()
        pat, _ = look(mask, B, Hq, L, S)
    return pat


_tile_cache: "OrderedDict[tuple, tuple]" = OrderedDict()


def tile_maps(mask: torch.Tensor, B: int, Hq: int, L: int, S: int):
    """Tile skip tables of a mask that is no pattern (``ops.mask_tile_maps``), cached for as long as
    the tensor is unchanged.  The run-time counterpart of the reference's static tile elimination
    (neuron_dynamo_backend/flex_attention/flex_attention.py.jinja:15-33): one pass over the mask on
    the device, no trip to the host.  ``None`` for masks too small to matter, masks per key, tensors
    without a version counter, inside a graph capture, and for a caller that brings a new tensor on
    every call (a relative-position bias computed per step, upstream's per-call conversion of a bool
    mask): after a few misses in a row for one signature such tensors get no tables - a pass over the
    tensor per call costs more than the tables save - with another try every ``_RETRY_EVERY`` calls.
    The cache holds the small tables and a weak reference to the mask's storage, never the mask."""
    if not enabled() or mask is None or L < 256 or S < 256 or mask.dim() < 2 or mask.shape[-2] == 1:
        return None
    version = _version(mask)
    if version is None or torch.cuda.is_current_stream_capturing():
        return None
    from . import ops

    key = (mask.data_ptr(), tuple(mask.shape), tuple(mask.stride()), mask.dtype, version, mask.device.index, B, Hq)
    sig = ("tiles", tuple(mask.shape), mask.dtype, mask.device.index)
    found, maps = _lookup(_tile_cache, key)
    if found:
        _misses.pop(sig, None)
        stats["tile_hits"] = stats.get("tile_hits", 0) + 1
        return maps
    if _back_off(sig):
        stats["tile_left_alone"] = stats.get("tile_left_alone", 0) + 1
        return None
    maps = ops.mask_tile_maps(mask, B, Hq, L, S)
    stats["tile_builds"] = stats.get("tile_builds", 0) + 1
    _remember(_tile_cache, key, maps, mask)
    return maps


def clear_cache() -> None:
    """Forget every verdict and table.  Needed after a mask was changed by anything that does not
    bump the tensor's version counter (a kernel launched through its data pointer, a graph replay
    that writes the buffer): only writes through torch ops are seen."""
    _cache.clear()
    _misses.clear()
    _tile_cache.clear()
