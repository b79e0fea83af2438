"""CPU restatement of the two tensor updates of the reference's KV cache -- TEST INFRASTRUCTURE ONLY.

Followed reference code: cache_hub/flash_attn_cache.py:153-232 (`prefill_update_kv_cache`) and :239-256
(`decode_update_kv_cache`).  Pure index arithmetic on torch-CPU tensors, so the GPU result must match bit for bit.
Pinned in tests/test_oracle_kv_cache.py by element-by-element Python loops on tiny inputs and by the invariants
the layout implies (rows outside the written range untouched; prefill followed by appends reproduces the
concatenated token sequence).
"""
from __future__ import annotations

import torch


def prefill_store(key_cache, value_cache, key_states, value_states, batch_index: int, valid_start: int):
    """`cache[b, :n] = states[0, valid_start:valid_start + n]`, n = seq_len - valid_start (:177-178, :207-222).
    Caches [B, L, Hkv, D] are updated in place; returns n."""
    assert key_states.shape[0] == 1, "one sequence per call (:166-169)"
    seq_len = key_states.shape[1]
    assert seq_len <= key_cache.shape[1], "sequence longer than the cache (:170-172)"
    n = seq_len - valid_start
    key_cache[batch_index, :n] = key_states[0, valid_start:valid_start + n].to(key_cache.dtype)
    value_cache[batch_index, :n] = value_states[0, valid_start:valid_start + n].to(value_cache.dtype)
    return n


def decode_append(key_cache, value_cache, key_states, value_states, valid_length, advance: bool):
    """`cache[b, valid_length[b]] = states[b, 0]` for every b (:248-253); `valid_length += 1` when `advance`
    (after the last layer, :253-255).  Returns the per-sequence number of rows the step's attention covers,
    valid_length + 1 (build-defined: the reference attends over the whole buffer)."""
    B = key_cache.shape[0]
    for b in range(B):
        pos = int(valid_length[b])
        key_cache[b, pos] = key_states[b, 0]
        value_cache[b, pos] = value_states[b, 0]
    attend = valid_length + 1
    if advance:
        valid_length += 1
    return attend
