"""K-means KV selection for the decode phase (no counterpart in the reference, whose `cache_hub/kmeans.py` has no
caller; defined by the end-to-end benchmark configuration: "... using the SQAttn prefill, the decode kernels and
k-means KV selection").

After the prompt is prefilled, the keys of every layer are clustered per (sequence, kv head) with
`segment_k_means` (cache_hub/kmeans.py:332-375).  A decode step then attends, per kv head, to
  * the tokens of the clusters whose centroids score highest against the step's queries (`topk_select`), and
  * every token appended after the clustering (the generated ones), which belong to no cluster,
through `attn_decode_selected`.  Everything stays on the device: the per-sequence number of valid list entries is
derived from the cache's `attend_length`, so a step needs no host synchronisation.
"""
from __future__ import annotations

from typing import List

import torch

from ..sqattn.attn_triton_decode import attn_decode_selected
from .. import _native as N
from .kmeans import _workspace, segment_k_means, topk_select


class KVSelection:
    def __init__(self, num_centroids: int = 1024, topk: int = 4096, num_iters: int = 10, num_segments: int = 1):
        if num_centroids % 32 != 0:
            raise AssertionError("num_centroids must be a multiple of 32 (cache_hub/kmeans.py:146)")
        self.num_centroids, self.topk, self.num_iters, self.num_segments = num_centroids, topk, num_iters, num_segments
        self.layers: List[dict] = []
        self.ids = None          # int32 [B * Hkv, topk + room]: the step's selection, then the appended tokens
        self.list_len = None     # int32 [B]: valid entries of a sequence's lists in this step
        self.offset = None       # int32 [B]: topk - prompt length of the sequence
        self.room = 0
        self.groups_hint = 0     # q heads per kv head, when known at build time (sizes the decode workspace once)

    def build(self, kv_cache, num_kv_heads: int, num_kv_groups: int = 0) -> None:
        """Cluster the prompt's keys of every layer.  `kv_cache`: the runtime's `flash_attn_cache` after prefill."""
        self.groups_hint = num_kv_groups
        B, Hkv = kv_cache.batch_size, num_kv_heads
        dev = kv_cache.key_cache[0].device
        prompt = [int(n) for n in kv_cache._host_valid]     # tokens cached per sequence (host mirror, no sync)
        self.room = kv_cache.max_length - min(prompt)
        self.layers = []
        for layer in range(len(kv_cache.key_cache)):
            per_seq = []
            for b in range(B):
                n = prompt[b]
                if n < self.num_centroids:
                    raise ValueError(f"sequence {b} has {n} cached tokens, fewer than the {self.num_centroids} clusters asked for")
                key = kv_cache.key_cache[layer][b, :n].permute(1, 0, 2).contiguous()       # [Hkv, n, D]
                value = kv_cache.value_cache[layer][b, :n].permute(1, 0, 2).contiguous()
                centroids, _, clusters, cluster_size = segment_k_means(key, value, self.num_centroids, self.num_iters, self.num_segments)
                per_seq.append((centroids, clusters, cluster_size))
            width = max(c[1].shape[2] for c in per_seq)
            clusters = torch.zeros(B * Hkv, self.num_centroids, width, dtype=torch.int32, device=dev)
            for b, (_, cl, _) in enumerate(per_seq):
                clusters[b * Hkv:(b + 1) * Hkv, :, :cl.shape[2]] = cl
            self.layers.append({"centroids": torch.cat([c[0] for c in per_seq]), "clusters": clusters,
                                "cluster_size": torch.cat([c[2] for c in per_seq])})
        # list layout: [0, topk) the selection of the step, [topk, topk + room) the tokens behind each sequence's prompt
        self.ids = torch.full((B * Hkv, self.topk + self.room), -1, dtype=torch.int32, device=dev)
        start = torch.tensor(prompt, dtype=torch.int32, device=dev).repeat_interleave(Hkv)
        self.ids[:, self.topk:] = start[:, None] + torch.arange(self.room, dtype=torch.int32, device=dev)[None, :]
        self.offset = torch.tensor([self.topk - n for n in prompt], dtype=torch.int32, device=dev)
        self.list_len = torch.zeros(B, dtype=torch.int32, device=dev)
        # buffers of a step, allocated once: the selection, the top-k scratch, the decode partials
        self.picked = self.ids[:, :self.topk]
        self.topk_ws = _workspace(B * Hkv, 1, self.num_centroids, dev)
        lib = N.lib()
        splits = lib.sq_decode_num_splits(B, Hkv, self.topk + self.room)
        self.decode_ws = torch.empty(lib.sq_decode_workspace_bytes(B, Hkv * self.groups_hint, 128, splits) // 4, dtype=torch.float32, device=dev) \
            if self.groups_hint else None

    def begin_step(self, attend_length: torch.Tensor) -> None:
        """Once per decode step, after the first layer's cache append set `attend_length`: a sequence's lists hold the
        topk selected tokens and its attend_length - prompt appended ones."""
        torch.add(attend_length, self.offset, out=self.list_len)

    def attend(self, layer_idx: int, query_states, key_cache, value_cache, num_kv_groups: int):
        """query_states [B, 1, Hq, D]; key_cache / value_cache [B, max_length, Hkv, D] -> [B, 1, Hq, D]."""
        st = self.layers[layer_idx]
        topk_select(query_states[:, 0], st["centroids"], st["clusters"], st["cluster_size"], self.topk, num_kv_groups,
                    out=self.picked, workspace=self.topk_ws)      # straight into the leading columns of the lists
        return attn_decode_selected(query_states, key_cache, value_cache, self.ids, "NHD", query_states.dtype, seqlens=self.list_len,
                                    workspace=self.decode_ws)
