"""ctypes binding of the C ABI declared in include/mi355_sdpa.h.

The library is loaded from the package's ``lib/`` directory.  There is no fallback: if it is
missing the import of any op raises, so a GPU run can never silently take another path.
"""

from __future__ import annotations

import ctypes as C
import struct
import os

import torch

from ._build import LIB_PATH

F32, F16, BF16, F64, BOOL, FP8_E4M3, OTHER = 0, 1, 2, 3, 4, 5, 99
KERNEL_NONE, KERNEL_GENERIC, KERNEL_MFMA, KERNEL_MFMA_T128, KERNEL_MFMA_T256 = 0, 1, 2, 3, 4
BACKEND_MATH, BACKEND_OVERRIDEABLE = 0, 4
OK, ERR_INVALID, ERR_UNSUPPORTED, ERR_LAUNCH = 0, -1, -2, -3
DECODE_STATIC_SCRATCH_BYTES = 32 << 20
ABI_VERSION = 6  # MI355_SDPA_ABI_VERSION of include/mi355_sdpa.h that the structures below follow

_DTYPES = {
    torch.float32: F32, torch.float16: F16, torch.bfloat16: BF16, torch.float64: F64,
    torch.bool: BOOL, torch.float8_e4m3fn: FP8_E4M3,
}


def dtype_id(dt: torch.dtype) -> int:
    return _DTYPES.get(dt, OTHER)


class Tensor4(C.Structure):
    _fields_ = [("data", C.c_void_p), ("size", C.c_int64 * 4), ("stride", C.c_int64 * 4)]


class Desc(C.Structure):
    _fields_ = [
        ("q_dim", C.c_int32), ("k_dim", C.c_int32), ("v_dim", C.c_int32),
        ("q_size", C.c_int64 * 4), ("k_size", C.c_int64 * 4), ("v_size", C.c_int64 * 4),
        ("q_dtype", C.c_int32), ("k_dtype", C.c_int32), ("v_dtype", C.c_int32),
        ("on_device", C.c_int32), ("has_symbolic_shape", C.c_int32), ("has_attn_bias", C.c_int32),
        ("is_causal", C.c_int32), ("return_debug_mask", C.c_int32), ("has_scale", C.c_int32),
        ("scale", C.c_float), ("dropout_p", C.c_float), ("requires_lse", C.c_int32),
        ("q_last_stride", C.c_int32), ("k_last_stride", C.c_int32), ("v_last_stride", C.c_int32),
    ]


class MaskSpec(C.Structure):
    _fields_ = [("window", C.c_int32), ("sink_keys", C.c_int32), ("sink_logit", C.c_void_p),
                ("live_tiles", C.c_void_p), ("live_tiles_t", C.c_void_p),
                ("n_sink_logits", C.c_int32), ("softcap", C.c_float), ("alibi_slopes", C.c_void_p),
                ("key_bias", C.c_void_p), ("key_weight", C.c_void_p), ("doc_ids_q", C.c_void_p),
                ("doc_ids_k", C.c_void_p), ("doc_ids_sorted", C.c_int32),
                ("mask_verdict", C.c_void_p)]


class FwdParams(C.Structure):
    _fields_ = [
        ("q", Tensor4), ("k", Tensor4), ("v", Tensor4), ("out", Tensor4),
        ("lse", C.c_void_p), ("bias", Tensor4), ("bias_dtype", C.c_int32),
        ("kv_lens", C.c_void_p), ("dropout_keep", C.c_void_p), ("dropout_p", C.c_float),
        ("dtype", C.c_int32), ("is_causal", C.c_int32), ("scale", C.c_float),
        ("force_kernel", C.c_int32), ("mask", MaskSpec),
        ("workspace", C.c_void_p), ("workspace_bytes", C.c_size_t), ("dropout_keep_ld", C.c_int64),
    ]


class BwdParams(C.Structure):
    _fields_ = [
        ("grad_out", Tensor4), ("q", Tensor4), ("k", Tensor4), ("v", Tensor4), ("out", Tensor4),
        ("lse", C.c_void_p), ("grad_q", Tensor4), ("grad_k", Tensor4), ("grad_v", Tensor4),
        ("bias", Tensor4), ("bias_dtype", C.c_int32), ("grad_bias", Tensor4),
        ("kv_lens", C.c_void_p), ("dropout_keep", C.c_void_p), ("dropout_p", C.c_float),
        ("dtype", C.c_int32), ("is_causal", C.c_int32), ("scale", C.c_float),
        ("workspace", C.c_void_p), ("workspace_bytes", C.c_size_t), ("force_kernel", C.c_int32),
        ("mask", MaskSpec), ("grad_sink_logit", C.c_void_p), ("dropout_keep_ld", C.c_int64),
    ]


class DecodeParams(C.Structure):
    _fields_ = [
        ("q", Tensor4), ("k", Tensor4), ("v", Tensor4),
        ("k_scale", C.c_void_p), ("v_scale", C.c_void_p), ("kv_lens", C.c_void_p),
        ("out", Tensor4), ("lse", C.c_void_p), ("q_dtype", C.c_int32), ("scale", C.c_float),
        ("num_splits", C.c_int32), ("workspace", C.c_void_p), ("workspace_bytes", C.c_size_t),
    ]


EXPORTS = {
    "mi355_sdpa_fwd": (C.c_int, [C.POINTER(FwdParams), C.c_void_p]),
    "mi355_sdpa_bwd": (C.c_int, [C.POINTER(BwdParams), C.c_void_p]),
    "mi355_sdpa_bwd_workspace_bytes": (C.c_size_t, [C.POINTER(BwdParams)]),
    "mi355_sdpa_fwd_workspace_bytes": (C.c_size_t, [C.POINTER(FwdParams)]),
    "mi355_sdpa_decode_fp8kv": (C.c_int, [C.POINTER(DecodeParams), C.c_void_p]),
    "mi355_sdpa_decode_workspace_bytes": (C.c_size_t, [C.POINTER(DecodeParams)]),
    "mi355_sdpa_decode_fp8kv_static": (C.c_int, [C.POINTER(DecodeParams), C.c_void_p]),
    "mi355_sdpa_mask_rows": (C.c_int, [C.c_void_p, C.c_int32, C.c_int64, C.c_int64, C.c_int64, C.c_void_p, C.c_void_p]),
    "mi355_sdpa_mask_tiles_words": (C.c_int, [C.c_void_p, C.c_int32, C.POINTER(C.c_size_t), C.POINTER(C.c_size_t)]),
    "mi355_sdpa_mask_verdict_words": (C.c_size_t, [C.c_void_p, C.c_int32]),
    "mi355_sdpa_mask_verdict": (C.c_int, [C.c_void_p, C.c_int32, C.c_void_p, C.c_void_p]),
    "mi355_sdpa_mask_tiles": (C.c_int, [C.c_void_p, C.c_int32, C.c_void_p, C.c_void_p, C.c_void_p]),
    "mi355_sdpa_choose_backend": (C.c_int, [C.POINTER(Desc)]),
    "mi355_sdpa_validate": (C.c_int, [C.POINTER(Desc), C.c_char_p, C.c_size_t]),
    "mi355_sdpa_out_strides": (C.c_int, [C.POINTER(C.c_int64), C.POINTER(C.c_int64),
                                         C.POINTER(C.c_int64), C.POINTER(C.c_int64)]),
    "mi355_sdpa_can_use_fused_fwd": (C.c_int, [C.POINTER(Desc)]),
    "mi355_sdpa_can_use_fused_bwd": (C.c_int, [C.POINTER(Desc)]),
    "mi355_sdpa_last_error": (C.c_char_p, []),
    "mi355_sdpa_abi_version": (C.c_int, []),
}

_lib = None


def load() -> C.CDLL:
    """Load the shared library (once).  Raises if it has not been built."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise RuntimeError(
                f"{LIB_PATH} is missing: build the HIP extension first "
                "(python -m torch_neuronx_amd._build, or __graft_entry__.build()). "
                "There is no fallback path."
            )
        lib = C.CDLL(LIB_PATH)
        for name, (res, args) in EXPORTS.items():
            fn = getattr(lib, name)
            fn.restype, fn.argtypes = res, args
        if lib.mi355_sdpa_abi_version() != ABI_VERSION:
            raise RuntimeError(
                f"{LIB_PATH} has ABI version {lib.mi355_sdpa_abi_version()}, this binding is for {ABI_VERSION}: "
                "rebuild the HIP extension (python -m torch_neuronx_amd._build)")
        _lib = lib
    return _lib


def last_error() -> str:
    return load().mi355_sdpa_last_error().decode()


_I64x4 = C.c_int64 * 4


def tensor4(t) -> Tensor4:
    if t is None:
        return Tensor4()
    assert t.dim() == 4
    return Tensor4(t.data_ptr(), _I64x4(*t.shape), _I64x4(*t.stride()))


_T4 = struct.Struct("@P4q4q")
assert _T4.size == C.sizeof(Tensor4)


def put4(params, field, t) -> None:
    """Write tensor ``t`` (4-D, or None: left zero) into the Tensor4 member ``field`` (a descriptor such
    as ``FwdParams.q``) of the parameter block ``params``: one packed write, a third of the time of
    building a Tensor4 and assigning it, which counts on calls whose kernels take microseconds."""
    if t is None:
        return
    sh, st = t.shape, t.stride()
    if len(sh) != 4:
        raise ValueError("expected a 4-D tensor")
    _T4.pack_into(params, field.offset, t.data_ptr(), sh[0], sh[1], sh[2], sh[3], st[0], st[1], st[2], st[3])


_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)


def current_stream(device) -> int:
    """Handle of torch's current stream on ``device`` (a hipStream_t as an integer)."""
    if _raw_stream is not None and device.index is not None:
        return _raw_stream(device.index)
    return torch.cuda.current_stream(device).cuda_stream


class _NoSwitch:
    def __enter__(self):
        return None

    def __exit__(self, *exc):
        return False


_NO_SWITCH = _NoSwitch()


def on_device(device):
    """Context that makes ``device`` current for the launch; free when it already is."""
    if device.index is None or torch.cuda.current_device() == device.index:
        return _NO_SWITCH
    return torch.cuda.device(device)


def check(rc: int) -> None:
    """Turn a status code into the exception type the operator contract asks for."""
    if rc == OK:
        return
    msg = last_error()
    if rc == ERR_UNSUPPORTED:
        raise NotImplementedError(msg)
    raise RuntimeError(msg)
