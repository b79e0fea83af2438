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


def cpu_model() -> str:
    try:
        with open("/proc/cpuinfo") as f:
            for line in f:
                if line.lower().startswith("model name"):
                    return line.split(":", 1)[1].strip()
    except OSError:
        pass
    return "unknown CPU"


def time_cpu_baseline(N=4096, Hq=4, Hkv=1, D=128, budget_s=12.0, seed=1, threads=None):
    """Repeat the config-1 shape for about `budget_s` seconds; returns (TFLOP/s causal-counted, threads,
    seconds per pass, passes).  `threads` limits torch's intra-op threads for the measurement (restored afterwards)."""
    before = torch.get_num_threads()
    if threads is not None:
        torch.set_num_threads(threads)
    try:
        return _time_c1(N, Hq, Hkv, D, budget_s, seed)
    finally:
        torch.set_num_threads(before)


def _time_c1(N, Hq, Hkv, D, budget_s, seed):
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


def fake_quant_sdpa_cpu_chunked(query, key, value, num_kv_groups: int, q_chunk: int = 2048):
    """The same path for long sequences: the operand passes as above, the attention in chunks of `q_chunk` query rows
    against the keys up to the chunk's last row with an explicit causal mask, so that no N x N tensor exists."""
    B, N, Hq, D = query.shape
    k = repeat_kv(key, num_kv_groups)
    v = repeat_kv(value, num_kv_groups)
    q = query.permute(0, 2, 1, 3)
    k = k - k.mean(dim=2, keepdim=True)
    q8 = FQ.int_fake_quant(q, 8, True, "per_token")
    k8 = FQ.int_fake_quant(k, 8, True, "per_token")
    v8 = FQ.int_fake_quant(v, 8, True, "per_channel")
    out = torch.empty_like(q8)
    for r0 in range(0, N, q_chunk):
        r1 = min(r0 + q_chunk, N)
        mask = torch.arange(r1)[None, :] <= torch.arange(r0, r1)[:, None]
        out[:, :, r0:r1] = torch.nn.functional.scaled_dot_product_attention(q8[:, :, r0:r1], k8[:, :, :r1], v8[:, :, :r1], attn_mask=mask)
    return out.transpose(1, 2).contiguous().view(B, N, Hq * D)


def time_prefill_points(points=(4096, 16384, 32768), Hq=4, Hkv=1, D=128, full_heads=28, target_n=131072, seed=2):
    """Config 2 on the host: `Hq` of its `full_heads` query heads (one kv-head group is 7; 4 are timed) at growing
    lengths, one pass each, and the quadratic extrapolation to `target_n` tokens and all heads from the largest point.
    Returns (list of {N, seconds, TFLOP_per_s}, extrapolated seconds)."""
    g = torch.Generator().manual_seed(seed)
    pts = []
    for N in points:
        q = (torch.randn(1, N, Hq, D, generator=g) * D ** -0.5).bfloat16()
        k = (torch.randn(1, N, Hkv, D, generator=g) * D ** -0.5).bfloat16()
        v = (torch.randn(1, N, Hkv, D, generator=g) * D ** -0.5).bfloat16()
        t0 = time.perf_counter()
        fake_quant_sdpa_cpu_chunked(q, k, v, Hq // Hkv)
        dt = time.perf_counter() - t0
        pts.append({"N": N, "seconds": round(dt, 4), "heads_timed": Hq, "TFLOP_per_s": round(4.0 * N * N * D * Hq / 2 / dt / 1e12, 4)})
    last = pts[-1]
    extrapolated = last["seconds"] * (target_n / last["N"]) ** 2 * (full_heads / Hq)
    return pts, extrapolated


def time_decode_cpu(L=131072, Hq=28, Hkv=4, D=128, reps=5, seed=3):
    """Config 3 at batch 1 on the host: one query token against a full 128K-token bf16 cache (the reference calls its
    framework's flash-attention here, model_hub/qwen.py:52-53; this is softmax(q k^T / sqrt(D)) v with the kv heads
    shared by their 7 query heads and fp32 scores).  Returns (GB/s of K+V streamed, seconds per call)."""
    g = torch.Generator().manual_seed(seed)
    q = torch.randn(1, Hkv, Hq // Hkv, D, generator=g).bfloat16()
    kc = torch.randn(1, Hkv, L, D, generator=g).bfloat16()
    vc = torch.randn(1, Hkv, L, D, generator=g).bfloat16()

    def call():
        s = torch.matmul(q, kc.transpose(-1, -2)).float() * D ** -0.5
        return torch.matmul(torch.softmax(s, dim=-1).to(torch.bfloat16), vc)

    call()
    t0 = time.perf_counter()
    for _ in range(reps):
        call()
    dt = (time.perf_counter() - t0) / reps
    return 2.0 * L * Hkv * D * 2 / dt / 1e9, dt


def time_kmeans_iteration_cpu(N=131072, C=1024, D=128, heads=4, seed=4):
    """Config 4 on the host: one Lloyd iteration of one head as the reference's kernels define it (fp32 inner products,
    first arg-max, fp32 cluster sums, mean, L2 normalisation; cache_hub/kmeans.py:7-124), timed once; the four heads of
    the configuration are independent, so the iteration is `heads` times that.  Returns (seconds per head, TFLOP/s)."""
    g = torch.Generator().manual_seed(seed)
    key = torch.randn(N, D, generator=g).bfloat16()
    cent = key[(torch.arange(C, dtype=torch.float32) * (N / C) + N / C / 2).long()].clone()
    t0 = time.perf_counter()
    kf = key.float()
    idx = torch.argmax(kf @ cent.float().T, dim=1)
    sums = torch.zeros(C, D).index_add_(0, idx, kf)
    cnt = torch.bincount(idx, minlength=C).float()
    x = sums / cnt[:, None]
    x = x / x.norm(dim=1, keepdim=True)
    cent = torch.where((cnt > 0)[:, None], x.bfloat16(), cent)
    dt = time.perf_counter() - t0
    return dt, 2.0 * N * C * D / dt / 1e12
