"""The decoder runtime of the reference's model_hub/LLM.py:18-235 around the gfx950 kernels: `layer_prefill`,
`layer_decode`, `prefill_forward`, `decode_forward`, `inference`, `generate` with the reference's names, argument
order and order of operations.  The projections stay plain `torch.nn.functional.linear` calls (hipBLASLt underneath);
everything between them runs on this package's kernels: RMSNorm, rotary embedding, KV-cache rows, prefill and decode
attention, SiLU*mul.

Differences, all deliberate:
  * one GPU (the reference's multi-GPU branches move activations between devices, LLM.py:131-137, 153-157);
  * the normalised activations are written to a fresh tensor instead of being normalised chunk by chunk inside a
    clone (LLM.py:46-53), and the MLP of a chunk is added onto the residual stream in place instead of cloning the
    residual (LLM.py:70-81): the same values with one copy of the hidden states less; the MLP still runs in chunks
    of 8192 // batch tokens, which bounds its 2 x intermediate-size activations;
  * decode attention covers `kv_cache.attend_length` tokens of each sequence, not the whole cache buffer;
  * a left-padded prompt (`valid_start > 0`) runs its attention over the valid tokens only, the padding rows get
    zeros (the reference hands the kernels more queries than keys, which they reject);
  * `generate(..., use_graph=True)` replays the decode step from a HIP graph (no reference counterpart).
"""
from __future__ import annotations

import time

import torch

torch.set_grad_enabled(False)


class LLM:
    """Base class: the model-independent forward loops.  A subclass provides `init_model`, `init_kv_cache`, `move`,
    `word_embedding`, `lm`, `wqkv`, `wo`, `mlp`, `layernorm`, `position_embedd` and `self.layers`."""

    chunk_tokens = 8192   # tokens per MLP chunk at batch 1 (LLM.py:47, 72)

    def __init__(self, model_name: str, max_length: int, dtype: torch.dtype, device_map: str) -> None:
        self.model_name = model_name
        self.max_length = max_length
        self.dtype = dtype
        self.device_map = device_map
        self.capture_layer_inps = None
        self.kv_selection = None   # see enable_kv_selection

    def enable_kv_selection(self, num_centroids: int = 1024, topk: int = 4096, num_iters: int = 10, num_segments: int = 1):
        """Extension (the reference's k-means code has no caller): after every prefill the prompt's keys are clustered
        per layer, sequence and kv head, and the decode steps attend to the `topk` tokens of the best-scoring clusters
        plus the generated tokens instead of the whole cache.  `disable_kv_selection()` returns to dense decoding."""
        from ..cache_hub.kv_selection import KVSelection

        self.kv_selection = KVSelection(num_centroids, topk, num_iters, num_segments)

    def cluster_prompt(self):
        """Cluster the keys the cache holds now (the prefilled prompt) and switch the decode slots to the selection."""
        self.kv_selection.build(self.kv_cache, self.num_key_value_heads, self.num_key_value_groups)
        for layer in self.layers:
            layer.kv_selection = self.kv_selection

    def disable_kv_selection(self):
        self.kv_selection = None
        for layer in getattr(self, "layers", []):
            layer.kv_selection = None

    # ------------------------------------------------------------------ one layer
    def layer_prefill(self, layer_idx, start_bdx, hidden_states):
        """LLM.py:40-86.  hidden_states [bsz, seq_len, hidden] is updated in place and returned."""
        if self.capture_layer_inps is not None:
            self.capture_layer_inps.append(hidden_states.detach().clone())   # the layers below update hidden_states in place
        bsz, seq_len, dim = hidden_states.shape
        layer = self.layers[layer_idx]
        normed = self.layernorm(hidden_states, layer.input_layernorm_variance_epsilon, layer.input_layernorm_weight)
        query_states, key_states, value_states = self.wqkv(normed, layer)
        del normed
        query_states, key_states = self.position_embedd(query_states, key_states)
        query_states = query_states.view(bsz, seq_len, self.num_heads, self.head_dim)
        key_states = key_states.view(bsz, seq_len, self.num_key_value_heads, self.head_dim)
        value_states = value_states.view(bsz, seq_len, self.num_key_value_heads, self.head_dim)
        key_states, value_states = self.kv_cache.prefill_update_kv_cache(query_states, key_states, value_states, layer_idx, start_bdx)
        pad = seq_len - key_states.shape[1]   # left padding the cache dropped (valid_start of this sequence)
        if pad == 0:
            temp_attn_out = layer.prefill_attention(query_states, key_states, value_states, None)
        else:
            # the attention kernels want as many queries as keys (the reference asserts it, attn_triton.py:272):
            # the padding rows attend to nothing and contribute zeros
            temp_attn_out = query_states.new_zeros(bsz, seq_len, dim)
            temp_attn_out[:, pad:] = layer.prefill_attention(query_states[:, pad:], key_states, value_states,
                                                             None).reshape(bsz, seq_len - pad, dim)
        self.kv_cache.sync(layer_idx, start_bdx)
        hidden_states += self.wo(temp_attn_out, layer, bsz, seq_len, dim)
        del query_states, key_states, value_states, temp_attn_out
        step = max(self.chunk_tokens // bsz, 1)
        for start_idx in range(0, seq_len, step):
            end_idx = min(seq_len, start_idx + step)
            chunk = hidden_states[:, start_idx:end_idx, :]
            chunk += self.mlp(self.layernorm(chunk, layer.post_attention_layernorm_variance_epsilon,
                                             layer.post_attention_layernorm_weight), layer)
        return hidden_states

    def layer_decode(self, layer_idx, hidden_states):
        """LLM.py:88-116."""
        residual = hidden_states
        bsz, seq_len, dim = hidden_states.shape
        layer = self.layers[layer_idx]
        fused = None
        if seq_len == 1 and hasattr(self, "wqkv_position_embedd"):
            # input norm, projection, rotary embedding and the cache rows of the new token in one pass (same values)
            norm = (layer.input_layernorm_weight, layer.input_layernorm_variance_epsilon)
            targets = self.kv_cache.decode_append_targets(layer_idx) if hasattr(self.kv_cache, "decode_append_targets") else None
            fused = self.wqkv_position_embedd(hidden_states, layer, cache=targets, norm=norm)
            appended = fused is not None and targets is not None
            if fused is None:
                fused = self.wqkv_position_embedd(hidden_states, layer, norm=norm)
        if fused is not None:
            query_states, key_states, value_states = fused
        else:
            appended = False
            hidden_states = self.layernorm(hidden_states, layer.input_layernorm_variance_epsilon, layer.input_layernorm_weight)
            query_states, key_states, value_states = self.wqkv(hidden_states, layer)
            query_states, key_states = self.position_embedd(query_states, key_states)
            query_states = query_states.view(bsz, -1, self.num_heads, self.head_dim)
            key_states = key_states.view(bsz, -1, self.num_key_value_heads, self.head_dim)
        value_states = value_states.view(bsz, -1, self.num_key_value_heads, self.head_dim)
        if appended:
            key_states, value_states = self.kv_cache.decode_update_kv_cache(key_states, value_states, layer_idx, appended=True)
        else:
            key_states, value_states = self.kv_cache.decode_update_kv_cache(key_states, value_states, layer_idx)
        attn_out = layer.decode_attention(query_states, key_states, value_states, None)
        if isinstance(attn_out, tuple):   # the slot `process_model(..., patch_decode=True)` binds returns a 1-tuple (LLM.py:105)
            attn_out = attn_out[0]
        residual = self.wo(attn_out, layer, bsz, seq_len, dim, residual=residual)   # residual + wo(...)
        if seq_len == 1:   # post-attention norm inside the gated projection (same values)
            return self.mlp(residual, layer, residual=residual,
                            norm=(layer.post_attention_layernorm_weight, layer.post_attention_layernorm_variance_epsilon))
        hidden_states = self.layernorm(residual, layer.post_attention_layernorm_variance_epsilon,
                                       layer.post_attention_layernorm_weight)
        return self.mlp(hidden_states, layer, residual=residual)                     # residual + mlp(...)

    # ------------------------------------------------------------------ whole model
    def prefill_forward(self, inputs_ids):
        """LLM.py:118-149: sequences are prefilled one by one; returns the logits of each sequence's last token."""
        bsz, seq_len = inputs_ids.shape
        last_hidden_states = torch.empty((bsz, 1, self.hidden_size), dtype=self.dtype, device=inputs_ids.device)
        for start_bdx in range(bsz):
            hidden_states = self.word_embedding(inputs_ids[start_bdx:start_bdx + 1])
            for ldx in range(self.num_layers):
                hidden_states = self.layer_prefill(ldx, start_bdx, hidden_states)
            last_hidden_states[start_bdx:start_bdx + 1] = hidden_states[:, -1:, :]
            del hidden_states
        last_hidden_states = self.layernorm(last_hidden_states.contiguous(), self.norm_variance_epsilon, self.norm_weight)
        return self.lm(last_hidden_states)

    def decode_forward(self, inputs_ids):
        """LLM.py:151-165."""
        hidden_states = self.word_embedding(inputs_ids)
        for ldx in range(self.num_layers):
            hidden_states = self.layer_decode(ldx, hidden_states)
        return self.lm(hidden_states[:, -1:, :], norm=(self.norm_weight, self.norm_variance_epsilon))

    # ------------------------------------------------------------------ captured decode step (extension)
    def capture_decode_step(self, first_token):
        """Record one decode step (all layers, final norm, lm head) into a HIP graph and run it once.

        Outside the attention kernel a decode step is a chain of small launches (five GEMMs, two norms, rotary,
        cache append, residual adds per layer) whose launch cost exceeds their run time; replaying them as one graph
        removes it.  Everything the step depends on lives on the device and is advanced by the graph itself: the
        token buffer is written by the caller, the position by an in-graph increment, the cache lengths by the
        append kernel.  The arg-max over the logits stays outside the graph.  Returns the logits of this step."""
        dev = first_token.device
        self._graph_token = first_token.clone()
        self._graph_positions = torch.full((first_token.shape[0], 1), self.kv_cache.context, dtype=torch.int64, device=dev)
        self.kv_cache.check_room()
        torch.cuda.synchronize()
        self._graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(self._graph):
            self._graph_logits = self.decode_forward(self._graph_token)   # host bookkeeping of this step runs here, once
            self._graph_positions += 1
        self._graph.replay()
        return self._graph_logits

    def replay_decode_step(self, token):
        """Run the captured step for `token` [batch, 1]; returns its logits (a buffer reused by every replay)."""
        self.kv_cache.check_room()
        self._graph_token.copy_(token)
        self._graph.replay()
        self.kv_cache.note_decode_step()
        return self._graph_logits

    def release_decode_graph(self):
        self._graph = None
        self._graph_positions = None
        self._graph_token = self._graph_logits = None

    def inference(self, inputs_ids, verbose: bool = True, use_graph: bool = False):
        """LLM.py:167-203: greedy decoding; returns the generated ids as nested lists [batch][max_new_length]."""
        outputs_ids = []
        for layer in self.layers:
            layer.kv_selection = None     # clusters of an earlier prompt
        torch.cuda.synchronize()
        prefill_start = time.time()
        logits = self.prefill_forward(inputs_ids=inputs_ids)
        output_ids = logits.argmax(dim=-1)
        outputs_ids.append(output_ids)
        self.move()
        torch.cuda.synchronize()
        self.prefill_latency = time.time() - prefill_start
        if verbose:
            print(f"Prefilling latency: {round(self.prefill_latency, 4)} s")
        if self.kv_selection is not None and self.max_new_length > 1:
            cluster_start = time.time()
            self.cluster_prompt()
            torch.cuda.synchronize()
            self.cluster_latency = time.time() - cluster_start
            if verbose:
                print(f"Clustering latency: {round(self.cluster_latency, 4)} s")
        if self.max_new_length > 1:
            decode_start, timed_steps = time.time(), self.max_new_length - 1
            for step in range(self.max_new_length - 1):
                if not use_graph or step == 0:
                    logits = self.decode_forward(inputs_ids=output_ids)    # the first step also warms the libraries up
                elif step == 1:
                    logits = self.capture_decode_step(output_ids)
                else:
                    logits = self.replay_decode_step(output_ids)
                output_ids = logits.argmax(dim=-1)
                outputs_ids.append(output_ids)
                if use_graph and step == 1 and self.max_new_length > 3:
                    torch.cuda.synchronize()      # steady state of the replays: leave the warm-up and capture steps out
                    decode_start, timed_steps = time.time(), self.max_new_length - 3
            torch.cuda.synchronize()
            if use_graph:
                self.release_decode_graph()
            self.decode_latency = (time.time() - decode_start) / timed_steps
            if verbose:
                print(f"Decoding latency: {round(self.decode_latency * 1000, 2)} ms/step, "
                      f"Throughput: {round(self.batch_size / self.decode_latency, 2)} tokens/s")
        return torch.cat(outputs_ids, dim=-1).tolist()

    def generate(self, attention_type, inputs_ids, attention_masks, max_new_length, verbose: bool = True,
                 use_graph: bool = False):
        """LLM.py:205-235.  attention_masks [batch, input_length] of 0/1 with the padding on the left, or None."""
        bs, input_length = inputs_ids.shape
        assert input_length + max_new_length <= self.max_length, (
            f"Error: input_length({input_length}) + max_new_length({max_new_length}) exceeds max_length({self.max_length})")
        self.batch_size = bs
        self.input_length = input_length
        self.max_new_length = max_new_length
        self.attention_type = attention_type
        if attention_masks is None:
            valid_start = [0] * bs
        else:
            valid_start = (attention_masks.shape[1] - attention_masks.sum(dim=-1)).tolist()
        self.init_kv_cache(input_length, valid_start)
        return self.inference(inputs_ids, verbose=verbose, use_graph=use_graph)
