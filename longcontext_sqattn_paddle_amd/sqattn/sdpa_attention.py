"""`sdpa_attention_forward` of the reference's sqattn/sdpa_attention.py:23-71 on torch's SDPA.

Used by layers the plugin leaves untouched and as the dense baseline.  The reference calls Paddle's
`scaled_dot_product_attention` (third-party arithmetic); torch's is the stand-in here.
"""
from __future__ import annotations

from typing import Optional

import torch


def repeat_kv(hidden_states: torch.Tensor, n_rep: int) -> torch.Tensor:
    """[B,N,Hkv,D] -> [B,Hkv*n_rep,N,D] (sdpa_attention.py:9-20)."""
    batch, slen, num_key_value_heads, head_dim = hidden_states.shape
    hidden_states = hidden_states.permute(0, 2, 1, 3)
    if n_rep == 1:
        return hidden_states
    hidden_states = hidden_states[:, :, None, :, :].expand(batch, num_key_value_heads, n_rep, slen, head_dim)
    return hidden_states.reshape(batch, num_key_value_heads * n_rep, slen, head_dim)


def sdpa_attention_forward(module, query, key, value, attention_mask: Optional[torch.Tensor], dropout: float = 0.0,
                           scaling: Optional[float] = None, is_causal: Optional[bool] = None, tensor_layout="NHD", **kwargs):
    """query [B,N,Hq,D], key/value [B,N,Hkv,D] -> [B,N,Hq*D] (the reference returns the bare tensor, :71).
    `scaling` multiplies the query as in the reference (:54); the 1/sqrt(D) lives inside SDPA."""
    if tensor_layout == "NHD":
        if hasattr(module, "num_key_value_groups"):
            key = repeat_kv(key, module.num_key_value_groups)
            value = repeat_kv(value, module.num_key_value_groups)
        else:
            key, value = key.permute(0, 2, 1, 3), value.permute(0, 2, 1, 3)
        query = query.permute(0, 2, 1, 3)
    if attention_mask is not None and attention_mask.ndim == 4:
        attention_mask = attention_mask[:, :, :, : key.shape[-2]]
    if is_causal is None:
        is_causal = query.shape[2] > 1 and attention_mask is None
    if scaling is not None and scaling != 1.0:
        query = query * scaling
    out = torch.nn.functional.scaled_dot_product_attention(query, key, value, attn_mask=attention_mask,
                                                           dropout_p=dropout, is_causal=bool(is_causal))
    out = out.transpose(1, 2).contiguous()
    b, n, h, d = out.shape
    return out.view(b, n, h * d)
