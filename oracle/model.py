"""CPU restatement of the reference's decoder forward pass -- TEST INFRASTRUCTURE ONLY.

Followed reference code: model_hub/LLM.py:40-165 (`layer_prefill`, `layer_decode`, `prefill_forward`,
`decode_forward`) with the helpers of model_hub/qwen.py:292-379 (`word_embedding`, `lm`, `wqkv`, `wo`, `mlp`,
`layernorm`, `position_embedd`).  Built from the pinned pieces of this package: `layer.rmsnorm`, `layer.rope`,
`layer.silu_and_mul`, `attention.exact_attention` (the reference's SDPA / flash attention stand-in), and torch's
16-bit CPU `linear` for the projections (fp32 accumulation, one rounding; the GPU's GEMM accumulates in another
order, which is what the tolerance of the model test covers).  Nothing here is new arithmetic; the wiring (operator
order, head mapping, halves of the rotary embedding and of the gated projection, the growing KV history) is pinned in
tests/test_oracle_model.py: prefill at once equals token-by-token feeding, and both equal an independent float64
transformer written out from the architecture (exactly, for float32 weights, where the rounding points are no-ops).
"""
from __future__ import annotations

import torch

from . import attention as A
from . import layer as L


class CpuDecoder:
    """Holds CPU copies of a model's weights (attribute names of the reference's layers) and a growing KV history."""

    def __init__(self, model):
        self.dtype = model.dtype
        self.num_heads, self.num_kv_heads, self.head_dim = model.num_heads, model.num_key_value_heads, model.head_dim
        self.hidden = model.hidden_size
        self.embed = model.embed_tokens.cpu()
        self.lm_head = model.lm_head.cpu()
        self.norm_w, self.norm_eps = model.norm_weight.cpu(), model.norm_variance_epsilon
        self.table = model.cos_sin_cache.cpu()
        self.layers = []
        for l in model.layers:
            self.layers.append({k: (getattr(l, k).cpu() if torch.is_tensor(getattr(l, k)) else getattr(l, k)) for k in (
                "wqkv", "bqkv", "wo", "gate_up_proj", "down_proj", "input_layernorm_weight", "post_attention_layernorm_weight",
                "input_layernorm_variance_epsilon", "post_attention_layernorm_variance_epsilon")})
        self.k_hist = [None] * len(self.layers)
        self.v_hist = [None] * len(self.layers)
        self.context = 0

    def _layer(self, i, hidden, pos):
        """One decoder layer for one sequence: hidden [1, T, hidden] at positions pos [T] (LLM.py:40-116)."""
        w = self.layers[i]
        lin = torch.nn.functional.linear
        T = hidden.shape[1]
        x = L.rmsnorm(hidden, w["input_layernorm_weight"], w["input_layernorm_variance_epsilon"])
        qkv = lin(x, w["wqkv"], w["bqkv"])
        kv = self.num_kv_heads * self.head_dim
        q, k, v = qkv.split([self.hidden, kv, kv], dim=-1)
        q, k = L.rope(pos, q.reshape(T, -1), k.reshape(T, -1), self.head_dim, self.table)
        k = k.view(1, T, self.num_kv_heads, self.head_dim)
        v = v.reshape(1, T, self.num_kv_heads, self.head_dim)
        self.k_hist[i] = k if self.k_hist[i] is None else torch.cat([self.k_hist[i], k], dim=1)
        self.v_hist[i] = v if self.v_hist[i] is None else torch.cat([self.v_hist[i], v], dim=1)
        qh = q.view(1, T, self.num_heads, self.head_dim).permute(0, 2, 1, 3)
        kh, vh = self.k_hist[i].permute(0, 2, 1, 3), self.v_hist[i].permute(0, 2, 1, 3)
        o, _ = A.exact_attention(qh, kh, vh, causal=True, q_offset=kh.shape[2] - T)
        attn = o.permute(0, 2, 1, 3).reshape(1, T, self.hidden).to(self.dtype)
        hidden = hidden + lin(attn, w["wo"])
        y = L.rmsnorm(hidden, w["post_attention_layernorm_weight"], w["post_attention_layernorm_variance_epsilon"])
        y = lin(L.silu_and_mul(lin(y, w["gate_up_proj"])), w["down_proj"])
        return hidden + y

    def forward(self, ids):
        """ids [1, T] appended to the history; returns the fp32 logits of the last token [1, 1, vocab]."""
        T = ids.shape[1]
        pos = torch.arange(self.context, self.context + T)
        hidden = torch.nn.functional.embedding(ids, self.embed)
        for i in range(len(self.layers)):
            hidden = self._layer(i, hidden, pos)
        self.context += T
        last = L.rmsnorm(hidden[:, -1:, :], self.norm_w, self.norm_eps)
        return torch.nn.functional.linear(last, self.lm_head).float()
