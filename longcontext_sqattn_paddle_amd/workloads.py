"""Seeded synthetic inputs of the benchmark configurations (CPU generator, fp32 draw, bf16 cast).

The reference's own RNG streams (`paddle.manual_seed`) cannot be reproduced without Paddle, so
"identical seeded inputs" means: this generator feeds both the HIP kernels and whatever they are
checked against.
"""
from __future__ import annotations

import torch


def _gen(seed: int) -> torch.Generator:
    return torch.Generator().manual_seed(seed)


def prefill_inputs(B=1, Hq=28, Hkv=4, N=131072, D=128, *, seed=2, scale=None, outlier_frac=0.02,
                   outlier_mult=8.0, dtype=torch.bfloat16):
    """Config-2 style: N(0,1)*scale (default 1/sqrt(D)); per kv-head round(outlier_frac*D) K channels x8.
    Returns q [B,Hq,N,D], k, v [B,Hkv,N,D]."""
    g = _gen(seed)
    scale = (1.0 / D ** 0.5) if scale is None else scale
    q = torch.randn(B, Hq, N, D, generator=g) * scale
    k = torch.randn(B, Hkv, N, D, generator=g) * scale
    v = torch.randn(B, Hkv, N, D, generator=g) * scale
    n_out = int(round(outlier_frac * D))
    for h in range(Hkv):
        ch = torch.randperm(D, generator=g)[:n_out]
        k[:, h, :, ch] *= outlier_mult
    return q.to(dtype), k.to(dtype), v.to(dtype)


def plugin_inputs(B=1, Hq=4, Hkv=1, N=4096, D=128, *, seed=1, dtype=torch.bfloat16):
    """Config-1 style at the plugin boundary (NHD): query [B,N,Hq,D], key/value [B,N,Hkv,D] ~ N(0,1)."""
    g = _gen(seed)
    q = torch.randn(B, N, Hq, D, generator=g)
    k = torch.randn(B, N, Hkv, D, generator=g)
    v = torch.randn(B, N, Hkv, D, generator=g)
    return q.to(dtype), k.to(dtype), v.to(dtype)


def decode_inputs(B=1, Hq=28, Hkv=4, L=131072, D=128, *, seed=3, min_len=None, dtype=torch.bfloat16):
    """Config-3 style: q [B,1,Hq,D], NHD caches [B,L,Hkv,D] ~ N(0,1), seqlens ~ U{min_len..L}
    (default min_len = 3L/4, i.e. 96K for a 128K cache)."""
    g = _gen(seed)
    q = torch.randn(B, 1, Hq, D, generator=g)
    kc = torch.randn(B, L, Hkv, D, generator=g)
    vc = torch.randn(B, L, Hkv, D, generator=g)
    lo = (3 * L) // 4 if min_len is None else min_len
    lens = torch.randint(lo, L + 1, (B,), generator=g, dtype=torch.int32)
    return q.to(dtype), kc.to(dtype), vc.to(dtype), lens


def kmeans_inputs(G=4, N=131072, D=128, *, n_modes=512, sigma=0.3, seed=4, dtype=torch.bfloat16):
    """Config-4 style: mixture of `n_modes` Gaussian centres per head plus noise. Returns key, value [G,N,D]."""
    g = _gen(seed)
    mu = torch.randn(G, n_modes, D, generator=g)
    which = torch.randint(0, n_modes, (G, N), generator=g)
    key = torch.gather(mu, 1, which[..., None].expand(G, N, D)) + sigma * torch.randn(G, N, D, generator=g)
    value = torch.randn(G, N, D, generator=g)
    return key.to(dtype), value.to(dtype)


def window_flops(N: int, D: int, sink: int, w8, w4, block_m: int = 64) -> float:
    """Algorithmic FLOPs of one sink + window prefill call: 4 * D * sum over heads and query blocks of
    (rows x keys visited), the diagonal block counted as its causal half.  `w8` / `w4` are the per-head window sizes in
    tokens; the key ranges are those of the reference's kernels (sink, 4-bit window, 8-bit window, own block:
    sqattn/attn_triton_mix_relative.py:36-75)."""
    total = 0.0
    for a8, a4 in zip(w8, w4):
        for qs in range(0, N, block_m):
            qe = qs + block_m
            rows = min(qe, N) - qs
            left4, left8 = max(sink, qe - a4), max(sink, qe - a8)
            keys = min(sink, qs) + max(left8 - left4, 0) + max(qs - left8, 0)
            total += rows * keys + rows * (rows + 1) / 2
    return 4.0 * D * total
