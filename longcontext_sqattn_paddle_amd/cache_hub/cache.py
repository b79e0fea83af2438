"""`KV_Cache` of the reference's cache_hub/cache.py:4-83: sizes and the memory budget of a per-layer KV cache."""
from __future__ import annotations

import torch

_GIB = 1024.0 ** 3


class KV_Cache:
    """Base class: remembers the geometry and works out how much device memory is left for the cache after the
    weights and the prefill activations, with the reference's own formula (cache.py:46-83)."""

    def __init__(self, layer_num: int, batch_size: int, max_length: int, num_key_value_heads: int, num_heads: int,
                 head_dim: int, dtype: torch.dtype, layer_mapping: dict, num_gpus: int, model_size: int) -> None:
        self.layer_num = layer_num
        self.batch_size = batch_size
        self.max_length = max_length
        self.kv_head = num_key_value_heads
        self.num_heads = num_heads
        self.head_dim = head_dim
        self.dtype = dtype
        self.layer_mapping = layer_mapping
        self.context = 0
        self.num_gpus = num_gpus
        self.model_size = model_size
        if not torch.cuda.is_available():
            raise RuntimeError("the KV cache lives on the MI355X; there is no CPU path")
        total_gpu_memory = self.num_gpus * torch.cuda.get_device_properties(0).total_memory / _GIB
        model_weight_consumption = self.model_size * 2          # GiB for a model_size given in 10^9 bf16 weights
        act = self.max_length * self.head_dim * 2 / _GIB        # one [max_length, head_dim] bf16 plane
        # hidden states twice, q/k/v, four more hidden-state sized temporaries (cache.py:53-78)
        prefill_consumption = (2 * self.num_heads + (self.num_heads + 2 * self.kv_head) + 4 * self.num_heads) * act
        self.free_memory = total_gpu_memory - model_weight_consumption - prefill_consumption * self.num_gpus
