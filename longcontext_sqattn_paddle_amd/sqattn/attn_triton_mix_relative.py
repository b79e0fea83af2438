"""`attn_hierarchical_relative_window` of the reference's sqattn/attn_triton_mix_relative.py:309-483.

Sink + hierarchical windows whose sizes are ratios of the KV length, evaluated per 64-row query block.
As in the reference launch (:441-444) the "4-bit" operands are aliased to the 8-bit ones: `q_int4` and
`k_int4` are accepted and ignored.  The reference's copy of all operands to a second GPU when one is
present (:426-437) is not reproduced; everything runs on the tensors' device.
"""
from __future__ import annotations

import numpy as np
import torch

from .. import _native as N
from ._prefill import align_windows, per_head, run_prefill


def window_tokens(ratio: float, kv_len: int) -> int:
    """ceil128(int64(float32(ratio) * kv_len)) exactly as the kernel computes it (:43-46)."""
    raw = int(np.float32(ratio) * np.float32(kv_len))
    return (raw + 127) // 128 * 128


def attn_hierarchical_relative_window(q_int8, k_int8, q_int4, k_int4, v, int8_window_ratios, int4_window_ratios,
                                      sink_size, tensor_layout="HND", output_dtype=torch.float16, return_lse=False,
                                      is_P_fp8_quant=False, *, p_quant=None, workspace=None, out=None, q_quant=0, k_scale=None):
    """`q_quant=8` (extension): `q_int8` is the query before its 8-bit per-token fake quantisation, which the kernel
    then applies while loading the rows (same bits as the separate pass).
    `k_scale` (extension, see `sqattn.fake_quant.fused_int8qk_prepass`): `k_int8` holds the key's int8 codes, `k_scale`
    their per-token scales and `q_int8` the raw query; Q.K^T then is a real integer product."""
    if tensor_layout not in N.LAYOUT:
        raise ValueError(f"tensor_layout {tensor_layout} not supported")
    seq_dim = 1 if tensor_layout == "NHD" else 2
    kv_len = k_int8.shape[seq_dim]
    H = q_int8.shape[1] if tensor_layout == "HND" else q_int8.shape[2]
    r8 = per_head(int8_window_ratios, H, "int8_window_ratios")
    r4 = per_head(int4_window_ratios, H, "int4_window_ratios")
    if not isinstance(sink_size, int) or sink_size < 0:
        raise ValueError(f"sink_size must be a non-negative integer, got {sink_size}")
    # (ratios already give multiples of 128; the sink is rounded up to a 64-key block, and an 8-bit ratio of zero under
    # a wider 4-bit window gets the query block, see align_windows)
    w8, w4, sink_size = align_windows([window_tokens(float(r), kv_len) for r in r8], [window_tokens(float(r), kv_len) for r in r4],
                                      sink_size, 64)
    window = {"block_m": 64, "sink": sink_size, "w8": w8, "w4": w4}
    mode = p_quant if p_quant is not None else (N.P_E4M3_STATIC if is_P_fp8_quant else N.P_NONE)
    return run_prefill(q_int8, k_int8, v, tensor_layout=tensor_layout, output_dtype=output_dtype,
                       return_lse=return_lse, p_quant=mode, window=window, workspace=workspace, out=out, q_quant=q_quant,
                       k_scale=k_scale)
