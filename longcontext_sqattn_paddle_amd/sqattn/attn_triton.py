"""`attn_causal` of the reference's sqattn/attn_triton.py:216-315 on the gfx950 prefill kernel.

Same positional signature.  Differences from the reference, all deliberate:
  * the leftover `pdb.set_trace()` after the launch (:311-313) is gone;
  * `return_lse=True` returns `(o, lse)` (the reference computes the LSE and drops it, :275-315);
  * keyword-only extensions: `p_quant` (block-absmax FP8-P), `q_offset` (chunked prefill: query row 0 sits
    at that absolute position and `q_offset + qo_len == kv_len`), `workspace`, `out`.
"""
from __future__ import annotations

import torch

from .. import _native as N
from ._prefill import run_prefill


def attn_causal(q, k, v, tensor_layout="HND", output_dtype=torch.float16, return_lse=False, is_P_fp8_quant=False,
                *, p_quant=None, q_offset=0, workspace=None, out=None):
    mode = p_quant if p_quant is not None else (N.P_E4M3_STATIC if is_P_fp8_quant else N.P_NONE)
    return run_prefill(q, k, v, tensor_layout=tensor_layout, output_dtype=output_dtype, return_lse=return_lse,
                       p_quant=mode, q_offset=q_offset, workspace=workspace, out=out)
