"""The reference's "fake-quant + SDPA" path on CPU, timed by `bench.py` as the CPU baseline.

TEST INFRASTRUCTURE ONLY (see `oracle/__init__.py`).  Restates what `ATTN_TYPE=SQAttn` does around its
kernel (sqattn/attn_replacer.py:334-365: GQA expand, K mean-centring, int8 per-token Q/K and int8
per-channel V fake-quant, plus the two 4-bit passes it also computes) and replaces the Triton launch by
causal scaled-dot-product attention as in sqattn/sdpa_attention.py:23-71 (there Paddle's SDPA, here
torch's CPU SDPA), all in bf16 on the host cores.
"""
from __future__ import annotations

import time

import torch

from . import fake_quant as FQ
from .plugin import repeat_kv


def fake_quant_sdpa_cpu(query, key, value, num_kv_groups: int):
    """query [B,N,Hq,D], key/value [B,N,Hkv,D] bf16 -> [B,N,Hq*D] bf16."""
    B, N, Hq, D = query.shape
    k = repeat_kv(key, num_kv_groups)
    v = repeat_kv(value, num_kv_groups)
    q = query.permute(0, 2, 1, 3)
    k = k - k.mean(dim=2, keepdim=True)
    q8 = FQ.int_fake_quant(q, 8, True, "per_token")
    FQ.int_fake_quant(q, 4, True, "per_token")      # computed by the reference, unused by its launch
    k8 = FQ.int_fake_quant(k, 8, True, "per_token")
    FQ.int_fake_quant(k, 4, True, "per_token")
    v8 = FQ.int_fake_quant(v, 8, True, "per_channel")
    o = torch.nn.functional.scaled_dot_product_attention(q8, k8, v8, is_causal=True)
    return o.transpose(1, 2).contiguous().view(B, N, Hq * D)


def time_cpu_baseline(N=4096, Hq=4, Hkv=1, D=128, budget_s=12.0, seed=1):
    """Repeat the config-1 shape for about `budget_s` seconds; returns (TFLOP/s causal-counted, threads,
    seconds per pass, passes)."""
    g = torch.Generator().manual_seed(seed)
    q = torch.randn(1, N, Hq, D, generator=g).bfloat16()
    k = torch.randn(1, N, Hkv, D, generator=g).bfloat16()
    v = torch.randn(1, N, Hkv, D, generator=g).bfloat16()
    fake_quant_sdpa_cpu(q, k, v, Hq // Hkv)  # warm-up
    t0 = time.perf_counter()
    n = 0
    while True:
        fake_quant_sdpa_cpu(q, k, v, Hq // Hkv)
        n += 1
        if time.perf_counter() - t0 > budget_s:
            break
    dt = (time.perf_counter() - t0) / n
    flops = 4.0 * N * N * D * Hq / 2
    return flops / dt / 1e12, torch.get_num_threads(), dt, n
