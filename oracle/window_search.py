"""CPU restatement of the calibration histograms and window search (test infrastructure only).

Follows `sqattn/window_search.py` of the reference: the dense causal attention map of one head
(`sqattn/attn_replacer.py:253-278`) is reduced to an "energy by distance" histogram, and the smallest window that
keeps a given share of that energy is read off the histogram.  Everything here is numpy in float64 on dense
[N, N] maps, so only small N.  (The reference holds the map in the model's 16-bit dtype and accumulates the bins in
fp32; this restatement keeps the exact probabilities, and bin indices are formed in fp32 as the reference's tensor
expressions form them.)  Pinned in tests/test_oracle_window_search.py by element-by-element loops on tiny
maps, by closed forms (uniform rows, a single off-diagonal) and by conservation sums.
"""
from __future__ import annotations

import math

import numpy as np

KIND_ABSOLUTE = 0        # bins = distance i - j                                   (window_search.py:20-48, 283-321)
KIND_RELATIVE = 1        # bins = floor(num_bins * (i - j) / i)                    (window_search.py:51-87)
KIND_RELATIVE_SINK = 2   # bins = floor(num_bins * (i - j) / (i - sink)), j >= sink (window_search.py:244-280)


def attention_map(q: np.ndarray, k: np.ndarray, groups: int = 1) -> np.ndarray:
    """softmax(q k^T / sqrt(D)) under the causal mask, per head: q [Hq, N, D], k [Hkv, N, D] -> [Hq, N, N] float64
    (attn_replacer.py:253-278 with the GQA expansion of :254-255)."""
    q = np.asarray(q, dtype=np.float64)
    k = np.repeat(np.asarray(k, dtype=np.float64), groups, axis=0)
    n, d = q.shape[-2], q.shape[-1]
    s = q @ k.transpose(0, 2, 1) / math.sqrt(d)
    s = np.where(np.tril(np.ones((n, n), dtype=bool))[None], s, -np.inf)
    s = s - s.max(axis=-1, keepdims=True)
    e = np.exp(s)
    return e / e.sum(axis=-1, keepdims=True)


def histogram_loop(attention_map_: np.ndarray, max_len: int) -> np.ndarray:
    """The reference's host loop (window_search.py:5-17): distance counts from 1 here, and distances >= max_len
    are dropped."""
    a = np.asarray(attention_map_, dtype=np.float64)
    n = a.shape[0]
    i, j = np.meshgrid(np.arange(n), np.arange(n), indexing="ij")
    dist = i - j + 1
    keep = (j <= i) & (dist < max_len)
    return np.bincount(dist[keep], weights=(a * dist)[keep], minlength=max_len).astype(np.float64)


def _rel_f32(dist: np.ndarray, den: np.ndarray, num_bins: int):
    """relative distance and its bin exactly as the fp32 tensor expressions of the reference produce them"""
    rel = dist.astype(np.float32) / den.astype(np.float32)
    scaled = rel * np.float32(num_bins)
    return rel, scaled, np.clip(np.floor(scaled).astype(np.int64), 0, num_bins - 1)


def histogram(attention_map_: np.ndarray, kind: int, bins: int, sink: int = 0) -> np.ndarray:
    """Energy histogram of one head's map [N, N] -> float64 [bins].

    KIND_ABSOLUTE: `hist[i-j] += A[i,j] * (i-j)` over j <= i and j >= sink; distances >= bins are dropped
        (window_search.py:20-48 with sink = 0, :283-321 with a sink).
    KIND_RELATIVE: bin `clamp(floor(bins * (i-j)/max(i,1)), 0, bins-1)`, weight `A * (i-j)` (:51-87).
    KIND_RELATIVE_SINK: only j >= sink; rows i <= sink have relative distance 0, the others
        `(i-j)/max(i-sink, 1)`; weight `A * (bins * rel + 1)` (:244-280).
    """
    a = np.asarray(attention_map_, dtype=np.float64)
    n = a.shape[0]
    i, j = np.meshgrid(np.arange(n), np.arange(n), indexing="ij")
    dist = i - j
    keep = j <= i
    if kind == KIND_ABSOLUTE:
        keep &= j >= sink
        h = np.bincount(dist[keep], weights=(a * dist)[keep], minlength=bins)
        return h[:bins].astype(np.float64)
    if kind == KIND_RELATIVE:
        _, _, b = _rel_f32(dist, np.maximum(i, 1), bins)
        return np.bincount(b[keep], weights=(a * dist)[keep], minlength=bins).astype(np.float64)
    if kind == KIND_RELATIVE_SINK:
        keep &= j >= sink
        rel, scaled, b = _rel_f32(dist, np.maximum(i - sink, 1), bins)
        low = i <= sink
        scaled = np.where(low, np.float32(0), scaled)
        b = np.where(low, 0, b)
        w = a * (scaled + np.float32(1)).astype(np.float64)   # `rel * num_bins + 1` is an fp32 tensor expression (:266)
        return np.bincount(b[keep], weights=w[keep], minlength=bins).astype(np.float64)
    raise ValueError(f"unknown histogram kind {kind}")


def find_optimal_window(hist: np.ndarray, threshold: float) -> int:
    """Smallest multiple of 128 whose distances hold `threshold` of the energy (window_search.py:116-128):
    1 for an empty histogram, len(hist) if the share is never reached."""
    hist = np.asarray(hist, dtype=np.float64)
    total = hist.sum()
    if total == 0:
        return 1
    run = 0.0
    for d in range(0, len(hist), 128):
        run += hist[d:d + 128].sum()
        if run >= threshold * total:
            return d + 128
    return len(hist)


def find_optimal_relative_window(hist: np.ndarray, threshold: float, num_bins: int = 100) -> float:
    """`(first bin at which the running energy reaches threshold * total, plus one) / num_bins`, at most 1;
    0.1 for an empty histogram (window_search.py:90-113)."""
    hist = np.asarray(hist, dtype=np.float64)
    total = hist.sum()
    if total == 0:
        return 0.1
    run, best = 0.0, 0
    for b in range(len(hist)):
        run += hist[b]
        if run >= threshold * total:
            best = b
            break
    return min((best + 1) / num_bins, 1.0)
