"""ctypes binding of libsqattn_hip.so: DLPack capsules in, error codes out.

The library is the only compute path of this package.  If it is missing, or a call fails, an exception
is raised -- there is no eager/PyTorch fallback.
"""
from __future__ import annotations

import ctypes
import os
from typing import Optional

import torch

_PKG_DIR = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_PKG_DIR, "libsqattn_hip.so")

ABI_VERSION = 3   # SQ_ABI_VERSION of include/sqattn.h
SQ_OK, SQ_EINVAL, SQ_ESHAPE, SQ_EDEVICE, SQ_EDTYPE, SQ_EUNSUPPORTED, SQ_EHIP, SQ_EWORKSPACE = 0, -1, -2, -3, -4, -5, -6, -7
LAYOUT = {"HND": 0, "NHD": 1}
P_NONE, P_E4M3_STATIC, P_E4M3_BLOCK, P_E4M3_STATIC_FAST, P_E4M3_FP8_PV, P_E4M3_MX_FP8_PV = 0, 1, 2, 3, 4, 5
WINDOW_NONE, WINDOW_SIZES = 0, 1
KMEANS_STATELESS, KMEANS_KEEP_SUMS, KMEANS_APPLY_CHANGES = 0, 1, 2
QTYPE = {"int": 0, "e4m3": 1, "e5m2": 2}


class DLDevice(ctypes.Structure):
    _fields_ = [("device_type", ctypes.c_int32), ("device_id", ctypes.c_int32)]


class DLDataType(ctypes.Structure):
    _fields_ = [("code", ctypes.c_uint8), ("bits", ctypes.c_uint8), ("lanes", ctypes.c_uint16)]


class DLTensor(ctypes.Structure):
    _fields_ = [
        ("data", ctypes.c_void_p),
        ("device", DLDevice),
        ("ndim", ctypes.c_int32),
        ("dtype", DLDataType),
        ("shape", ctypes.POINTER(ctypes.c_int64)),
        ("strides", ctypes.POINTER(ctypes.c_int64)),
        ("byte_offset", ctypes.c_uint64),
    ]


class PrefillParams(ctypes.Structure):
    _fields_ = [
        ("layout", ctypes.c_int32),
        ("p_quant", ctypes.c_int32),
        ("head_dim_og", ctypes.c_int32),
        ("q_offset", ctypes.c_int64),
        ("window_mode", ctypes.c_int32),
        ("block_m", ctypes.c_int32),
        ("sink", ctypes.c_int32),
        ("num_heads_w", ctypes.c_int32),
        ("w8", ctypes.POINTER(ctypes.c_int32)),
        ("w4", ctypes.POINTER(ctypes.c_int32)),
        ("q_quant", ctypes.c_int32),
    ]


class DecodeParams(ctypes.Structure):
    _fields_ = [
        ("layout", ctypes.c_int32),
        ("p_quant", ctypes.c_int32),
        ("num_splits", ctypes.c_int32),
        ("head_dim_og", ctypes.c_int32),
    ]


class HistogramParams(ctypes.Structure):
    _fields_ = [
        ("kind", ctypes.c_int32),
        ("bins", ctypes.c_int32),
        ("sink", ctypes.c_int32),
        ("softmax_scale", ctypes.c_float),
    ]


HIST_ABSOLUTE, HIST_RELATIVE, HIST_RELATIVE_SINK = 0, 1, 2

_P = ctypes.POINTER(DLTensor)

# every symbol include/sqattn.h declares: name -> (restype, argtypes)
SYMBOLS = {
    "sq_abi_version": (ctypes.c_int, []),
    "sq_last_error": (ctypes.c_char_p, []),
    "sq_prefill_workspace_bytes": (ctypes.c_size_t, [ctypes.c_int64] * 4),
    "sq_prefill_fwd": (ctypes.c_int, [_P, _P, _P, _P, _P, _P, _P, _P, ctypes.POINTER(PrefillParams), ctypes.c_void_p]),
    "sq_decode_num_splits": (ctypes.c_int32, [ctypes.c_int64] * 3),
    "sq_decode_workspace_bytes": (ctypes.c_size_t, [ctypes.c_int64, ctypes.c_int64, ctypes.c_int64, ctypes.c_int32]),
    "sq_decode_fwd": (ctypes.c_int, [_P, _P, _P, _P, _P, _P, _P, ctypes.POINTER(DecodeParams), ctypes.c_void_p]),
    "sq_decode_noalloc_scratch_bytes": (ctypes.c_size_t, []),
    "sq_decode_noalloc_init": (ctypes.c_int, []),
    "sq_decode_fwd_noalloc": (ctypes.c_int, [_P, _P, _P, _P, _P, _P, ctypes.POINTER(DecodeParams), ctypes.c_void_p]),
    "sq_decode_selected_fwd": (ctypes.c_int, [_P] * 8 + [ctypes.POINTER(DecodeParams), ctypes.c_void_p]),
    "sq_kmeans_workspace_bytes": (ctypes.c_size_t, [ctypes.c_int64] * 4),
    "sq_kmeans_train": (ctypes.c_int, [_P, _P, _P, _P, _P, ctypes.c_int32, ctypes.c_void_p]),
    "sq_kmeans_train_stateful": (ctypes.c_int, [_P, _P, _P, _P, _P, ctypes.c_int32, ctypes.c_int32, ctypes.c_void_p]),
    "sq_reverse_index": (ctypes.c_int, [_P, _P, _P, _P, ctypes.c_void_p]),
    "sq_index_add": (ctypes.c_int, [_P, _P, _P, _P, ctypes.c_void_p]),
    "sq_topk_select": (ctypes.c_int, [_P, _P, _P, _P, _P, _P, ctypes.c_int32, ctypes.c_void_p]),
    "sq_fake_quant_prepass_workspace_bytes": (ctypes.c_size_t, [ctypes.c_int64] * 3),
    "sq_fake_quant_prepass": (ctypes.c_int, [_P] * 9 + [ctypes.c_int32, ctypes.c_void_p]),
    "sq_fake_quant_prepass_typed": (ctypes.c_int, [_P] * 9 + [ctypes.c_int32, ctypes.c_int32, ctypes.c_int32, ctypes.c_void_p]),
    "sq_rmsnorm": (ctypes.c_int, [_P, _P, _P, ctypes.c_float, ctypes.c_void_p]),
    "sq_silu_and_mul": (ctypes.c_int, [_P, _P, ctypes.c_void_p]),
    "sq_rope": (ctypes.c_int, [_P] * 6 + [ctypes.c_int32, ctypes.c_void_p]),
    "sq_linear_rows": (ctypes.c_int, [_P] * 5 + [ctypes.c_void_p]),
    "sq_linear_rows_silu_and_mul": (ctypes.c_int, [_P] * 4 + [ctypes.c_void_p]),
    "sq_linear_rows_rope": (ctypes.c_int, [_P] * 5 + [ctypes.c_int32, ctypes.c_int32] + [_P] * 5 + [ctypes.c_void_p]),
    "sq_rmsnorm_linear_rows": (ctypes.c_int, [_P, _P, ctypes.c_float] + [_P] * 4 + [ctypes.c_void_p]),
    "sq_rmsnorm_linear_rows_silu_and_mul": (ctypes.c_int, [_P, _P, ctypes.c_float] + [_P] * 3 + [ctypes.c_void_p]),
    "sq_rmsnorm_linear_rows_rope": (ctypes.c_int, [_P, _P, ctypes.c_float] + [_P] * 4 + [ctypes.c_int32, ctypes.c_int32] + [_P] * 5 + [ctypes.c_void_p]),
    "sq_prefill_int8qk_fwd": (ctypes.c_int, [_P] * 7 + [ctypes.POINTER(PrefillParams), ctypes.c_void_p]),
    "sq_fake_quant_prepass_int8qk": (ctypes.c_int, [_P] * 7 + [ctypes.c_int32, ctypes.c_void_p]),
    "sq_kv_cache_store": (ctypes.c_int, [_P] * 4 + [ctypes.c_int32, ctypes.c_int64, ctypes.c_void_p]),
    "sq_kv_cache_append": (ctypes.c_int, [_P] * 6 + [ctypes.c_int32, ctypes.c_void_p]),
    "sq_kv_cache_reorder": (ctypes.c_int, [_P] * 5 + [ctypes.c_void_p]),
    "sq_attention_histogram": (ctypes.c_int, [_P, _P, _P, ctypes.POINTER(HistogramParams), ctypes.c_void_p]),
}

# libsqattn_probe.so: a measurement aid (the rate of a loop of nothing but MFMAs), not part of the product's C ABI
PROBE_LIB_PATH = os.path.join(_PKG_DIR, "libsqattn_probe.so")
PROBE_SYMBOLS = {
    "sq_last_error": (ctypes.c_char_p, []),
    "sq_probe_mfma_operand_bytes": (ctypes.c_size_t, []),
    "sq_probe_mfma_flops": (ctypes.c_int64, [ctypes.c_int32, ctypes.c_int32]),
    "sq_probe_mfma_rate": (ctypes.c_int, [ctypes.c_int32, _P, _P, ctypes.c_int32, ctypes.c_void_p]),
}

_lib: Optional[ctypes.CDLL] = None
_probe_lib: Optional[ctypes.CDLL] = None


def lib() -> ctypes.CDLL:
    """Load the shared library once; raise if it has not been built."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise RuntimeError(
                f"{LIB_PATH} is missing: build it with `python -m longcontext_sqattn_paddle_amd.build` "
                "(there is no fallback path)")
        handle = ctypes.CDLL(LIB_PATH)
        for name, (res, args) in SYMBOLS.items():
            fn = getattr(handle, name)
            fn.restype = res
            fn.argtypes = args
        if handle.sq_abi_version() != ABI_VERSION:
            raise RuntimeError("libsqattn_hip.so ABI version mismatch")
        _lib = handle
    return _lib


def probe_lib() -> ctypes.CDLL:
    """The measurement-aid library (bench.py and its test); errors of its calls go through `check(code, probe_lib())`."""
    global _probe_lib
    if _probe_lib is None:
        if not os.path.exists(PROBE_LIB_PATH):
            raise RuntimeError(f"{PROBE_LIB_PATH} is missing: build it with `python -m longcontext_sqattn_paddle_amd.build`")
        handle = ctypes.CDLL(PROBE_LIB_PATH)
        for name, (res, args) in PROBE_SYMBOLS.items():
            fn = getattr(handle, name)
            fn.restype = res
            fn.argtypes = args
        _probe_lib = handle
    return _probe_lib


_capsule_ptr = ctypes.pythonapi.PyCapsule_GetPointer
_capsule_ptr.restype = ctypes.c_void_p
_capsule_ptr.argtypes = [ctypes.py_object, ctypes.c_char_p]


class Borrowed:
    """A DLTensor borrowed from a torch tensor through its DLPack capsule.

    The capsule is kept alive (and never consumed) for the lifetime of this object; dropping it runs
    the producer's deleter, so the library only ever sees borrowed memory.
    """

    def __init__(self, t: torch.Tensor):
        self.tensor = t
        self.capsule = torch.utils.dlpack.to_dlpack(t)
        addr = _capsule_ptr(self.capsule, b"dltensor")
        self.ptr = ctypes.cast(addr, _P)  # DLManagedTensor starts with its DLTensor


def dl(t: Optional[torch.Tensor]):
    return None if t is None else Borrowed(t)


def ptr(b: Optional[Borrowed]):
    return None if b is None else b.ptr


def check(code: int, library: Optional[ctypes.CDLL] = None) -> None:
    """Map a library error code to the exception type the reference raises for the same mistake."""
    if code == SQ_OK:
        return
    msg = (library or lib()).sq_last_error().decode("utf-8", "replace")
    if code in (SQ_EINVAL, SQ_EUNSUPPORTED, SQ_EDTYPE):
        raise ValueError(msg)
    if code == SQ_ESHAPE:
        raise AssertionError(msg)
    raise RuntimeError(f"libsqattn_hip error {code}: {msg}")


def current_stream(device) -> ctypes.c_void_p:
    return ctypes.c_void_p(torch.cuda.current_stream(device).cuda_stream)
