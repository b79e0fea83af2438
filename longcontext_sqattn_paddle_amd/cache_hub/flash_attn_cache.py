"""`flash_attn_cache` of the reference's cache_hub/flash_attn_cache.py:22-256 on the gfx950 row-copy kernels.

Same constructor, attributes (`key_cache`, `value_cache`, `valid_start`, `valid_length`, `context`) and methods
(`prefill_update_kv_cache`, `sync`, `decode_update_kv_cache`, `move_gpu`, `pre_allocate_decision`).  Differences,
all deliberate:
  * one GPU and no host offload: when the budget of `pre_allocate_decision` says the cache does not fit, the
    constructor raises instead of keeping the cache in host memory (the reference's `allocated == False` branch,
    :83-108); 288 GB hold the 1M-token, 28-layer cache of Qwen2.5-7B (60 GB);
  * `valid_length` is int32 [batch_size] with one entry per sequence, filled as each sequence is prefilled; the
    reference keeps a single entry derived from the first sequence (:190-203), which is the same whenever its
    decode indexing is right (all sequences equally long);
  * the decode update never leaves the device (no host copy of the lengths), and it also maintains
    `attend_length = valid_length + 1` during a step, the per-sequence length the decode attention kernel takes,
    where the reference attends over the whole buffer;
  * `sync` really waits for the copy (the reference's wait is commented out, :234-238).
"""
from __future__ import annotations

import torch

from .. import _native as N
from .cache import KV_Cache


class flash_attn_cache(KV_Cache):
    """KV cache for full attention: per layer one key and one value buffer [batch, max_length, kv_heads, head_dim]."""

    def __init__(self, valid_start, layer_num: int, batch_size: int, max_length: int, num_key_value_heads: int,
                 num_heads: int, head_dim: int, dtype: torch.dtype, layer_mapping: dict, num_gpus: int,
                 model_size: int) -> None:
        super().__init__(layer_num, batch_size, max_length, num_key_value_heads, num_heads, head_dim, dtype,
                         layer_mapping, num_gpus, model_size)
        if dtype not in (torch.bfloat16, torch.float16):
            raise ValueError(f"KV cache dtype {dtype} not supported (bf16 or fp16)")
        devices = {str(layer_mapping[str(ldx)]) for ldx in range(layer_num)}
        if num_gpus != 1 or len(devices) != 1:
            raise ValueError("this build keeps the whole KV cache on one GPU (num_gpus == 1, one device in layer_mapping)")
        self.device = torch.device(devices.pop().replace("gpu:", "cuda:"))
        if isinstance(valid_start, (tuple, list)):
            self.valid_start = [int(x) for x in valid_start]
        elif torch.is_tensor(valid_start):
            self.valid_start = [int(x) for x in valid_start.reshape(-1).tolist()]
        else:
            self.valid_start = [int(valid_start)] * batch_size
        if len(self.valid_start) != batch_size:
            raise ValueError(f"valid_start has {len(self.valid_start)} entries for {batch_size} sequences")
        self.batch_indices = torch.arange(self.batch_size, dtype=torch.int32, device=self.device)
        self.allocated = self.pre_allocate_decision()
        if not self.allocated:
            raise MemoryError(
                f"KV cache of {self._kv_gib():.1f} GiB (x1.3 headroom) does not fit the {self.free_memory:.1f} GiB left "
                "on the device; host offload is not part of this build")
        shape = (self.batch_size, self.max_length, self.kv_head, self.head_dim)
        self.key_cache = [torch.empty(shape, device=self.device, dtype=self.dtype) for _ in range(self.layer_num)]
        self.value_cache = [torch.empty(shape, device=self.device, dtype=self.dtype) for _ in range(self.layer_num)]
        self.valid_length = torch.zeros(self.batch_size, dtype=torch.int32, device=self.device)
        self.attend_length = torch.zeros(self.batch_size, dtype=torch.int32, device=self.device)
        self._host_valid = [0] * self.batch_size     # host mirror of valid_length: bounds checks without a sync
        self.copystream = torch.cuda.Stream(device=self.device)
        self.copyevents = {str(self.device): torch.cuda.Event()}
        self.KVreadyevents = {str(self.device): torch.cuda.Event()}
        self._lib = N.lib()

    def _kv_gib(self) -> float:
        return 2 * self.layer_num * self.batch_size * self.max_length * self.kv_head * self.head_dim * 2 / 1024.0 ** 3

    def pre_allocate_decision(self) -> bool:
        """flash_attn_cache.py:130-142."""
        return self.free_memory > self._kv_gib() * 1.3

    def move_gpu(self) -> None:
        """The cache is born on the GPU (flash_attn_cache.py:144-151 moves a host cache over)."""

    def prefill_update_kv_cache(self, query_states, key_states, value_states, layer_idx, start_bdx):
        """Store one sequence's keys and values from `valid_start` on (flash_attn_cache.py:153-232).

        key_states/value_states [1, seq_len, kv_heads, head_dim].  Returns the stored slices
        `key_states[:, valid_start:]`, `value_states[:, valid_start:]` like the reference.  The copy runs on the
        cache's copy stream behind the work already queued on the current stream; `sync` joins it.
        """
        bsz, seq_len, _, _ = key_states.shape
        assert bsz == 1, "Multi-batch prefilling only support prefill single batch one by one."
        assert seq_len <= self.max_length, f"Prefilling sequence length {seq_len} exceeds max length {self.max_length}."
        if not 0 <= start_bdx < self.batch_size:
            raise IndexError(f"batch index {start_bdx} outside the cache's {self.batch_size} sequences")
        _valid_start = self.valid_start[start_bdx]
        _valid_length = seq_len - _valid_start
        dev = str(self.device)
        self.KVreadyevents[dev].record()
        with torch.cuda.stream(self.copystream):
            self.copystream.wait_event(self.KVreadyevents[dev])
            b = [N.dl(t) for t in (key_states, value_states, self.key_cache[layer_idx], self.value_cache[layer_idx])]
            N.check(self._lib.sq_kv_cache_store(*[N.ptr(x) for x in b], int(start_bdx), int(_valid_start),
                                                N.current_stream(self.device)))
            key_states.record_stream(self.copystream)
            value_states.record_stream(self.copystream)
            if self._host_valid[start_bdx] != _valid_length:
                self.valid_length[start_bdx:start_bdx + 1].fill_(_valid_length)
                self._host_valid[start_bdx] = _valid_length
            self.copyevents[dev].record()
        if layer_idx == self.layer_num - 1 and start_bdx + bsz == self.batch_size:
            self.context += seq_len
        return key_states[:, _valid_start:, :, :], value_states[:, _valid_start:, :, :]

    def sync(self, layer_idx, start_bdx) -> None:
        """The current stream waits for the last prefill copy (flash_attn_cache.py:234-238)."""
        torch.cuda.current_stream(self.device).wait_event(self.copyevents[str(self.device)])

    def decode_append_targets(self, layer_idx):
        """(key_cache, value_cache, valid_length, attend_length) of a layer, for a projection kernel that writes the
        new token's k and v itself (`model_hub.utils.linear_rope`); `decode_update_kv_cache(..., appended=True)`
        afterwards does the rest of the step's bookkeeping."""
        self.check_room()
        return self.key_cache[layer_idx], self.value_cache[layer_idx], self.valid_length, self.attend_length

    def decode_update_kv_cache(self, key_states, value_states, layer_idx, appended=False):
        """Append one token per sequence at `valid_length` (flash_attn_cache.py:239-256).

        key_states/value_states [batch, 1, kv_heads, head_dim].  Returns the layer's whole cache buffers like the
        reference; `self.attend_length` (int32 [batch], on the device) holds how many of their rows are valid for
        this step's attention.  `valid_length` and `context` advance after the last layer.  `appended`: the caller's
        projection kernel has already written this layer's rows (see `decode_append_targets`).
        """
        self.check_room()
        last = layer_idx == self.layer_num - 1
        if not appended or last:   # appended: the rows and `attend_length` are in place; the last layer still advances the length
            b = [N.dl(t) for t in (key_states, value_states, self.key_cache[layer_idx], self.value_cache[layer_idx],
                                   self.valid_length, self.attend_length)]
            N.check(self._lib.sq_kv_cache_append(*[N.ptr(x) for x in b], 1 if last else 0, N.current_stream(self.device)))
        if last:
            self.note_decode_step()
        return self.key_cache[layer_idx], self.value_cache[layer_idx]

    def check_room(self) -> None:
        if max(self._host_valid) >= self.max_length:
            raise IndexError(f"KV cache is full: a sequence already holds max_length = {self.max_length} tokens")

    def note_decode_step(self) -> None:
        """Host-side bookkeeping of one finished decode step (`context`, the mirror of `valid_length`).  Called by
        `decode_update_kv_cache` after the last layer; a caller that replays a captured decode step, where no Python
        runs between the layers, calls `check_room()` before and this after every replay."""
        self.context += 1
        self._host_valid = [n + 1 for n in self._host_valid]
