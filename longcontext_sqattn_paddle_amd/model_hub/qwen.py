"""`QwenLayer` / `QwenModel` of the reference's model_hub/qwen.py:15-380 on the gfx950 kernels.

The reference reads the weights of `Qwen/Qwen2.5-7B-Instruct` through PaddleFormers (qwen.py:200-227); there is no
network and no checkpoint here, so `QwenModel` takes a `QwenConfig` and either a Hugging-Face style module to copy
the weights from (`init_model(hf_qwen)`, same attribute names as the reference reads) or nothing, in which case the
weights are drawn at random with the architecture's shapes.  Method names and signatures follow the reference.
"""
from __future__ import annotations

import math
import re
from dataclasses import dataclass

import torch

from ..cache_hub.flash_attn_cache import flash_attn_cache
from ..sqattn.attn_triton import attn_causal
from ..sqattn.attn_triton_decode import attn_decode
from .LLM import LLM
from .utils import apply_rope_with_cos_sin_cache_inplace, linear, linear_rope, linear_silu_and_mul, rmsnorm, yarn_cos_sin_cache


@dataclass
class QwenConfig:
    """The fields of the Hugging-Face config the reference reads (qwen.py:117-128); defaults = Qwen2.5-7B."""
    hidden_size: int = 3584
    intermediate_size: int = 18944
    num_hidden_layers: int = 28
    num_attention_heads: int = 28
    num_key_value_heads: int = 4
    vocab_size: int = 152064
    rope_theta: float = 1000000.0
    max_position_embeddings: int = 32768
    rms_norm_eps: float = 1e-6
    eos_token_id: int = 151645


class QwenLayer:
    """One decoder layer: its weights and the two attention slots (qwen.py:15-112)."""

    def __init__(self, layer_idx, device, attn_type, config, max_length) -> None:
        self.layer_idx = layer_idx
        self.device = device
        self.attention_type = attn_type
        self.config = config
        self.num_layers = config.num_hidden_layers
        self.num_heads = config.num_attention_heads
        self.num_key_value_heads = config.num_key_value_heads
        self.num_key_value_groups = self.num_heads // self.num_key_value_heads
        self.hidden_size = config.hidden_size
        self.head_dim = self.hidden_size // self.num_heads
        self.max_length = max_length
        self.kv_cache = None   # set by QwenModel.init_kv_cache: decode attention needs the per-sequence lengths
        self.p_quant = None    # extension: a P mode of the prefill kernel (e.g. 5 = fp8 P.V); None = exact attention
        self.calibration = None   # a sqattn.window_search.CalibrationCapture while the window search runs on this layer
        self.kv_selection = None  # a cache_hub.kv_selection.KVSelection once the prompt's keys are clustered (extension)

    def prefill_attention(self, query_states, key_states, value_states, layer_idx=None):
        """qwen.py:37-46: exact causal attention over [B, N, H, D] tensors (SDPA / flash attention in the reference;
        `process_model` replaces this slot by the quantised-window closure for the SQAttn layers)."""
        if self.attention_type not in ("SQAttn", "SDPA", "FlashAttn"):
            raise ValueError(f"Unsupported attention type: {self.attention_type}")
        if self.calibration is not None:
            # the reference stores the dense map here, and only for layer_idx 0 / last although its runtime always
            # passes None (qwen.py:38-41, LLM.py:67); the capture reduces Q and K to the histograms directly
            self.calibration.record(query_states, key_states)
        return attn_causal(query_states, key_states, value_states, "NHD", query_states.dtype, p_quant=self.p_quant)

    def decode_attention(self, query_states, key_states, value_states, layer_idx=None):
        """qwen.py:48-54: one query token against the layer's cache buffers [B, max_length, Hkv, D]."""
        if self.attention_type not in ("SQAttn", "SDPA", "FlashAttn"):
            raise ValueError(f"Unsupported attention type: {self.attention_type}")
        if self.kv_selection is not None:
            # extension: attend to the tokens of the best-scoring k-means clusters and to the generated tokens only
            if self.layer_idx == 0:
                self.kv_selection.begin_step(self.kv_cache.attend_length)
            return self.kv_selection.attend(self.layer_idx, query_states, key_states, value_states, self.num_key_value_groups)
        lens = self.kv_cache.attend_length if self.kv_cache is not None else None
        return attn_decode(query_states, key_states, value_states, "NHD", query_states.dtype, seqlens=lens)

    def init_layer(self, hf_qwen_layer):
        """Copy the weights of a Hugging-Face style layer (qwen.py:56-112)."""
        dev = self.device
        a, m = hf_qwen_layer.self_attn, hf_qwen_layer.mlp
        self.wqkv = torch.cat((a.q_proj.weight.detach(), a.k_proj.weight.detach(), a.v_proj.weight.detach()), dim=0).to(dev)
        self.bqkv = torch.cat((a.q_proj.bias.detach(), a.k_proj.bias.detach(), a.v_proj.bias.detach()), dim=0).to(dev)
        self.wo = a.o_proj.weight.detach().to(dev)
        self.gate_up_proj = torch.cat((m.gate_proj.weight.detach(), m.up_proj.weight.detach()), dim=0).to(dev)
        self.down_proj = m.down_proj.weight.detach().to(dev)
        self.input_layernorm_weight = hf_qwen_layer.input_layernorm.weight.detach().to(dev)
        self.input_layernorm_variance_epsilon = getattr(hf_qwen_layer.input_layernorm, "variance_epsilon", self.config.rms_norm_eps)
        self.post_attention_layernorm_weight = hf_qwen_layer.post_attention_layernorm.weight.detach().to(dev)
        self.post_attention_layernorm_variance_epsilon = getattr(hf_qwen_layer.post_attention_layernorm, "variance_epsilon",
                                                                 self.config.rms_norm_eps)

    def init_random(self, generator, dtype):
        """Random weights of the architecture's shapes (projection rows scaled so that activations stay O(1))."""
        dev, c = self.device, self.config
        kv = self.num_key_value_heads * self.head_dim

        def w(rows, cols, scale):
            return (torch.randn(rows, cols, device=dev, generator=generator) * scale).to(dtype)

        h, i = c.hidden_size, c.intermediate_size
        self.wqkv = w(h + 2 * kv, h, h ** -0.5)
        self.bqkv = (torch.randn(h + 2 * kv, device=dev, generator=generator) * 0.02).to(dtype)
        self.wo = w(h, h, h ** -0.5)
        self.gate_up_proj = w(2 * i, h, h ** -0.5)
        self.down_proj = w(h, i, i ** -0.5)
        self.input_layernorm_weight = (1 + 0.05 * torch.randn(h, device=dev, generator=generator)).to(dtype)
        self.post_attention_layernorm_weight = (1 + 0.05 * torch.randn(h, device=dev, generator=generator)).to(dtype)
        self.input_layernorm_variance_epsilon = c.rms_norm_eps
        self.post_attention_layernorm_variance_epsilon = c.rms_norm_eps


class QwenModel(LLM):
    """qwen.py:115-380."""

    def __init__(self, model_name: str, max_length: int, dtype: torch.dtype, device_map: str, attention_type: str,
                 config: QwenConfig = None, hf_model=None, seed: int = 0) -> None:
        super().__init__(model_name, max_length, dtype, device_map)
        if device_map == "auto":
            device_map = "cuda:0"
        if not str(device_map).startswith("cuda"):
            raise RuntimeError("the model lives on the MI355X (device_map 'cuda:0'); there is no CPU path")
        self.device_map = device_map
        self.config = config if config is not None else QwenConfig()
        self.num_layers = self.config.num_hidden_layers
        self.num_heads = self.config.num_attention_heads
        self.num_key_value_heads = self.config.num_key_value_heads
        self.num_key_value_groups = self.num_heads // self.num_key_value_heads
        self.hidden_size = self.config.hidden_size
        self.head_dim = self.hidden_size // self.num_heads
        self.base = self.config.rope_theta
        self.max_position_embeddings = self.config.max_position_embeddings
        self.yarn_factor = 4
        self.vocab_size = self.config.vocab_size
        self.eos_tokens = [self.config.eos_token_id]
        self.attention_type = attention_type
        self.num_gpus = 1
        self.kv_cache = None
        self.init_model(hf_model, seed)

    def init_model(self, hf_qwen=None, seed: int = 0):
        """qwen.py:199-271, single-device branch."""
        dev, c = self.device_map, self.config
        self.layer_mapping = {str(ldx): dev for ldx in range(self.num_layers)}
        g = torch.Generator(device=dev).manual_seed(seed)
        if hf_qwen is not None:
            self.embed_tokens = hf_qwen.model.embed_tokens.weight.detach().to(dev)
            self.lm_head = hf_qwen.lm_head.weight.detach().to(dev)
            self.norm_weight = hf_qwen.model.norm.weight.detach().to(dev)
            self.norm_variance_epsilon = getattr(hf_qwen.model.norm, "variance_epsilon", c.rms_norm_eps)
            inv_freq = hf_qwen.model.rotary_emb.inv_freq.detach()
        else:
            self.embed_tokens = torch.randn(c.vocab_size, c.hidden_size, device=dev, generator=g).to(self.dtype)
            self.lm_head = (torch.randn(c.vocab_size, c.hidden_size, device=dev, generator=g) * c.hidden_size ** -0.5).to(self.dtype)
            self.norm_weight = torch.ones(c.hidden_size, device=dev, dtype=self.dtype)
            self.norm_variance_epsilon = c.rms_norm_eps
            inv_freq = None
        self.position_ids = torch.arange(0, self.max_length, device=dev)
        self.cos_sin_cache = yarn_cos_sin_cache(self.head_dim, self.base, self.max_position_embeddings, self.max_length, dev,
                                                self.yarn_factor, inv_freq)
        self.layers = []
        for idx in range(self.num_layers):
            layer = QwenLayer(idx, device=dev, attn_type=self.attention_type, config=c, max_length=self.max_length)
            if hf_qwen is not None:
                layer.init_layer(hf_qwen.model.layers[idx])
            else:
                layer.init_random(g, self.dtype)
            self.layers.append(layer)

    def init_kv_cache(self, real_input_length, valid_start):
        """qwen.py:273-286."""
        m = re.search("(\\d+)[Bb]", self.model_name)
        self.kv_cache = flash_attn_cache(
            valid_start=valid_start, layer_num=self.num_layers, batch_size=self.batch_size,
            max_length=self.max_new_length + real_input_length, num_key_value_heads=self.num_key_value_heads,
            num_heads=self.num_heads, head_dim=self.head_dim, dtype=self.dtype, layer_mapping=self.layer_mapping,
            num_gpus=self.num_gpus, model_size=int(m.group(1)) if m else 0)
        for layer in self.layers:
            layer.kv_cache = self.kv_cache

    def move(self):
        """qwen.py:288-291."""
        self.kv_cache.move_gpu()

    def word_embedding(self, inputs_id):
        return torch.nn.functional.embedding(inputs_id, self.embed_tokens)

    def lm(self, hidden_states, norm=None):
        """qwen.py:293-300.  `norm` = (weight, epsilon): the final norm in front of the head rides in the same pass."""
        return linear(hidden_states, self.lm_head, norm=norm).float()

    def wqkv(self, hidden_states, layer):
        """qwen.py:302-312: one fused projection, split into views (no copies)."""
        qkv = linear(hidden_states, layer.wqkv, layer.bqkv)
        kv = self.hidden_size // self.num_key_value_groups
        return qkv.split([self.hidden_size, kv, kv], dim=-1)

    def wqkv_position_embedd(self, hidden_states, layer, cache=None, norm=None):
        """`wqkv` followed by `position_embedd` for a decode step (qwen.py:302-312, 369-379) as one pass: returns
        (query_states [bsz, 1, Hq, head_dim], key_states [bsz, 1, Hkv, head_dim], value_states [bsz, 1, kv_dim]),
        q and k rotated, all three views of one projection output.  `cache`: the layer's
        `kv_cache.decode_append_targets(...)`; the pass then also appends k and v to the cache (None is returned if it
        cannot, and nothing has been written).  `norm` = (weight, epsilon): `hidden_states` is the layer's input before
        `input_layernorm`, which then is part of the same pass (same values)."""
        bsz, seq_len, _ = hidden_states.shape
        if getattr(self, "_graph_positions", None) is not None and seq_len == 1:
            position_ids = self._graph_positions   # device-resident position of a captured decode step
        else:
            position_ids = self.position_ids[self.kv_cache.context:self.kv_cache.context + seq_len].unsqueeze(0).repeat(bsz, 1)
        kv = self.hidden_size // self.num_key_value_groups
        qkv = linear_rope(hidden_states, layer.wqkv, layer.bqkv, position_ids, self.head_dim, self.hidden_size + kv, self.cos_sin_cache, cache=cache,
                          norm=norm)
        if qkv is None:
            return None
        q, k, v = qkv.split([self.hidden_size, kv, kv], dim=-1)
        return q.view(bsz, seq_len, self.num_heads, self.head_dim), k.view(bsz, seq_len, self.num_key_value_heads, self.head_dim), v

    def wo(self, hidden_states, layer, bsz, seq_len, dim, residual=None):
        """qwen.py:314-317.  With `residual` the caller's `residual + wo(...)` is part of the same pass (same values)."""
        return linear(hidden_states.reshape(bsz, seq_len, dim), layer.wo, None, residual)

    def mlp(self, hidden_states, layer, residual=None, norm=None):
        """qwen.py:319-326.  `residual` as in `wo`; `norm` = (weight, epsilon): `hidden_states` comes before
        `post_attention_layernorm`, which a decode step's first projection then applies in the same pass."""
        return linear(linear_silu_and_mul(hidden_states, layer.gate_up_proj, norm=norm), layer.down_proj, None, residual)

    def layernorm(self, hidden_states, epsilon, weight):
        """qwen.py:345-350."""
        return rmsnorm(hidden_states, weight, epsilon)

    def apply_rotary_pos_emb(self, query_states, key_states, position_ids):
        """qwen.py:352-367.  The q and k parts of the fused projection are strided row views; the kernel reads them
        in place."""
        bsz, seq_len, hidden_dim = query_states.shape
        kv_dim = key_states.shape[-1]
        q2 = query_states.reshape(bsz * seq_len, hidden_dim) if bsz == 1 or query_states.is_contiguous() else query_states.contiguous().view(-1, hidden_dim)
        k2 = key_states.reshape(bsz * seq_len, kv_dim) if bsz == 1 or key_states.is_contiguous() else key_states.contiguous().view(-1, kv_dim)
        return apply_rope_with_cos_sin_cache_inplace(position_ids, q2, k2, self.head_dim, self.cos_sin_cache)

    def position_embedd(self, query_states, key_states):
        """qwen.py:369-379: every sequence of the batch sits at positions context .. context + seq_len."""
        bsz, seq_len, _ = key_states.shape
        if getattr(self, "_graph_positions", None) is not None and seq_len == 1:
            position_ids = self._graph_positions   # device-resident position of a captured decode step
        else:
            position_ids = self.position_ids[self.kv_cache.context:self.kv_cache.context + seq_len].unsqueeze(0).repeat(bsz, 1)
        return self.apply_rotary_pos_emb(query_states, key_states, position_ids)
