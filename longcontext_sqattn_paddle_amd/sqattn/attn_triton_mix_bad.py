"""`attn_hierarchical_window` of the reference's sqattn/attn_triton_mix_bad.py:285-426.

Sink + hierarchical windows with absolute sizes (tokens), evaluated per 128-row query block; the 4-bit
window range really uses `q_int4`/`k_int4` (:388-393).  Any non-negative window and sink sizes are accepted; sizes
the reference's kernel has no defined behaviour for (not multiples of its 64-key block) are rounded up as
`_prefill.align_windows` states.
"""
from __future__ import annotations

import torch

from .. import _native as N
from ._prefill import align_windows, per_head, run_prefill


def attn_hierarchical_window(q_int8, k_int8, q_int4, k_int4, v, int8_window_sizes, int4_window_sizes, sink_size,
                             tensor_layout="HND", output_dtype=torch.float16, return_lse=False,
                             is_P_fp8_quant=False, *, p_quant=None, workspace=None, out=None):
    if tensor_layout not in N.LAYOUT:
        raise ValueError(f"tensor_layout {tensor_layout} not supported")
    H = q_int8.size(1) if tensor_layout == "HND" else q_int8.size(2)
    w8 = [int(x) for x in per_head(int8_window_sizes, H, "int8_window_sizes")]
    w4 = [int(x) for x in per_head(int4_window_sizes, H, "int4_window_sizes")]
    if not isinstance(sink_size, int) or sink_size < 0:
        raise ValueError(f"sink_size must be a non-negative integer, got {sink_size}")
    if min(w8 + w4) < 0:
        raise ValueError("window sizes must be non-negative")
    w8, w4, sink_size = align_windows(w8, w4, sink_size, 128)
    window = {"block_m": 128, "sink": sink_size, "w8": w8, "w4": w4}
    same = q_int4 is None or (q_int4.data_ptr() == q_int8.data_ptr() and k_int4.data_ptr() == k_int8.data_ptr())
    mode = p_quant if p_quant is not None else (N.P_E4M3_STATIC if is_P_fp8_quant else N.P_NONE)
    return run_prefill(q_int8, k_int8, v, q4=None if same else q_int4, k4=None if same else k_int4,
                       tensor_layout=tensor_layout, output_dtype=output_dtype, return_lse=return_lse, p_quant=mode,
                       window=window, workspace=workspace, out=out)
