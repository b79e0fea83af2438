"""Shared host side of the prefill wrappers: argument checks mirroring the reference, padding, launch."""
from __future__ import annotations

import ctypes
from typing import Optional, Sequence

import torch

from .. import _native as N
from ._common import pad_head_dim, require_gpu


def prefill_workspace(B: int, Hkv: int, kv_len: int, device) -> torch.Tensor:
    """Scratch for the fp16 transposed V tiles the kernel consumes (caller may cache and reuse it)."""
    need = N.lib().sq_prefill_workspace_bytes(B, Hkv, kv_len, 128)
    return torch.empty(need // 2, dtype=torch.float16, device=device)


def run_prefill(q, k, v, *, tensor_layout="HND", output_dtype=torch.float16, return_lse=False, p_quant=N.P_NONE,
                q4=None, k4=None, window: Optional[dict] = None, q_offset: int = 0,
                workspace: Optional[torch.Tensor] = None, out: Optional[torch.Tensor] = None, q_quant: int = 0,
                k_scale: Optional[torch.Tensor] = None):
    """window = None (full causal) or {"block_m": 64|128, "sink": int, "w8": [Hq ints], "w4": [Hq ints]}.
    q_quant = 8: the kernel applies the 8-bit per-token fake quantiser to the rows of q as it loads them.
    k_scale (fp32 [B, Hkv, ceil64(Nk)]): `k` holds the int8 codes of the key and Q.K^T runs as an integer product
    (`sq_prefill_int8qk_fwd`; head_dim 128 only, no 4-bit operands, P not quantised)."""
    if tensor_layout not in N.LAYOUT:
        raise ValueError(f"tensor_layout {tensor_layout} not supported")
    require_gpu(q, k, v, q4, k4)
    head_dim_og = q.size(-1)
    if k_scale is not None:
        if head_dim_og != 128 or q4 is not None or k4 is not None or p_quant != N.P_NONE or q_quant:
            raise ValueError("the integer Q.K^T path takes head_dim 128, no 4-bit operands and no P or q quantisation mode")
        if k.dtype != torch.int8:
            raise ValueError(f"k must hold int8 codes when k_scale is given (got {k.dtype})")
    else:
        q, k, v, q4, k4 = pad_head_dim((q, k, v, q4, k4), head_dim_og)
    assert q.stride(-1) == 1 and k.stride(-1) == 1 and v.stride(-1) == 1, "Last dim of qkv must be contiguous."
    hdim, ndim = (1, 2) if tensor_layout == "HND" else (2, 1)
    B, Hq, Nq = q.size(0), q.size(hdim), q.size(ndim)
    Hkv, Nk = k.size(hdim), k.size(ndim)
    lib = N.lib()
    if workspace is None:
        workspace = prefill_workspace(B, Hkv, Nk, q.device)
    o = out if out is not None else torch.empty(q.shape, dtype=output_dtype, device=q.device)
    lse = torch.empty([B, Hq, Nq], dtype=torch.float32, device=q.device) if return_lse else None
    params = N.PrefillParams()
    params.layout = N.LAYOUT[tensor_layout]
    params.p_quant = p_quant
    params.head_dim_og = head_dim_og
    params.q_offset = q_offset
    params.q_quant = int(q_quant)
    keep = []
    if window is None:
        params.window_mode = N.WINDOW_NONE
        params.block_m = 128
    else:
        w8 = (ctypes.c_int32 * Hq)(*[int(x) for x in window["w8"]])
        w4 = (ctypes.c_int32 * Hq)(*[int(x) for x in window["w4"]])
        keep += [w8, w4]
        params.window_mode = N.WINDOW_SIZES
        params.block_m = int(window["block_m"])
        params.sink = int(window["sink"])
        params.num_heads_w = Hq
        params.w8 = ctypes.cast(w8, ctypes.POINTER(ctypes.c_int32))
        params.w4 = ctypes.cast(w4, ctypes.POINTER(ctypes.c_int32))
    if k_scale is not None:
        b = [N.dl(t) for t in (q, k, k_scale, v, o, lse, workspace)]
        N.check(lib.sq_prefill_int8qk_fwd(*[N.ptr(x) for x in b], ctypes.byref(params), N.current_stream(q.device)))
    else:
        b = [N.dl(t) for t in (q, k, v, q4, k4, o, lse, workspace)]
        N.check(lib.sq_prefill_fwd(*[N.ptr(x) for x in b], ctypes.byref(params), N.current_stream(q.device)))
    o = o[..., :head_dim_og]
    return (o, lse) if return_lse else o


def per_head(values, H: int, what: str) -> list:
    """Scalar, list/tuple or tensor -> list of H numbers (attn_triton_mix_relative.py:341-364)."""
    if isinstance(values, (int, float)):
        return [values] * H
    if isinstance(values, torch.Tensor):
        values = values.detach().cpu().tolist()
    values = list(values)
    if len(values) != H:
        raise ValueError(f"{what}: expected {H} per-head values, got {len(values)}")
    return values


def align_windows(w8, w4, sink: int, block_m: int):
    """Window and sink sizes the kernels take, from arbitrary non-negative integers.

    The reference's kernels walk a range in 64-key blocks (`range(lo, hi, 64)`), so sizes that are multiples of 64 are
    walked as written and pass through unchanged here (192 stays 192 under the 128-row query block of the absolute
    variant too).  For sizes that are not multiples of 64 the reference has no defined behaviour (taken literally, the
    block loop starts at an unaligned key and runs past the end of its range, visiting keys of the next range twice);
    they are rounded up to the next multiple of 64, and so is the sink.  The relative entry point produces multiples of
    128 by itself (attn_triton_mix_relative.py:43-46).

    A 4-bit window wider than an 8-bit window that is smaller than the query block makes the reference's 4-bit range
    run into the query block itself without the causal mask (it reads keys behind the query rows).  Here the 8-bit
    window is raised to the query block in that case: the 4-bit range then ends where the block starts, and the
    block's own keys are visited once, masked, as 8-bit operands."""
    up = lambda x, m: (int(x) + m - 1) // m * m
    w8 = [up(x, 64) for x in w8]
    w4 = [up(x, 64) for x in w4]
    w8 = [max(a, block_m) if b > a and a < block_m else a for a, b in zip(w8, w4)]
    return w8, w4, up(sink, 64)
