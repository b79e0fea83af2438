"""Window search: attention-energy histograms and the window sizes read off them (`sqattn/window_search.py`).

The reference reduces a layer's dense attention map `current_attention` [1, Hq, N, N] to one histogram per head and
picks, per head, the smallest window that keeps `bit8_thres` / `bit4_thres` of the energy.  Same function names and
arguments here; two things differ:

* `attention_histograms(query, key, ...)` computes the histograms of all heads straight from Q and K on the GPU
  (`sq_attention_histogram`), so the [N, N] map is never built.  The calibration drivers use it through the
  layer's `calibration` slot (model_hub/qwen.py `QwenLayer.prefill_attention`).
* In the reference the drivers never see a map: `model.layer_prefill` calls `layer.prefill_attention(q, k, v, None)`
  (model_hub/LLM.py:67) and the slot only stores the map for `layer_idx` 0 or last (model_hub/qwen.py:38-41), so
  every histogram stays zero and every head gets the defaults (1 token / ratio 0.1).  Here the slot records whenever a
  calibration is active.

The map-based functions (`compute_*_histogram_gpu*`) are kept for callers that do hold a map; they are plain tensor
passes over [N, N] like the reference's.
"""
from __future__ import annotations

import math
from typing import Optional

import numpy as np
import torch

from .. import _native as N
from ._common import pad_head_dim, require_gpu

ABSOLUTE, RELATIVE, RELATIVE_SINK = N.HIST_ABSOLUTE, N.HIST_RELATIVE, N.HIST_RELATIVE_SINK


# --------------------------------------------------------------------------------------- fused: from Q and K
def attention_histograms(query: torch.Tensor, key: torch.Tensor, kind: int, bins: int, sink: int = 0,
                         tensor_layout: str = "NHD", out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """Energy histograms of causal softmax attention for every (batch, query head): float64 [B, Hq, bins].

    query [B, N, Hq, D] / key [B, N, Hkv, D] for "NHD" (what the layer's attention slot receives), [B, H, N, D] for
    "HND"; bf16 or fp16; D <= 128.  `kind`: ABSOLUTE (`compute_attention_histogram_gpu`, or
    `compute_absolute_attention_histogram_gpu_with_sink` when sink > 0), RELATIVE
    (`compute_relative_attention_histogram_gpu`), RELATIVE_SINK (`compute_relative_attention_histogram_gpu_with_sink`).
    With `out` the histograms are added to it (the reference sums the histograms of the calibration samples).
    """
    require_gpu(query, key)
    if tensor_layout not in ("NHD", "HND"):
        raise ValueError(f"Unknown tensor layout: {tensor_layout}")
    if query.dim() != 4 or key.dim() != 4:
        raise AssertionError("query and key must be 4-D")
    head_dim = query.shape[-1]
    query, key = pad_head_dim((query, key), head_dim)
    if tensor_layout == "NHD":
        query, key = query.permute(0, 2, 1, 3), key.permute(0, 2, 1, 3)   # views: the kernel takes any strides
    B, Hq = query.shape[0], query.shape[1]
    if out is None:
        out = torch.zeros(B, Hq, bins, dtype=torch.float64, device=query.device)
    params = N.HistogramParams(kind=int(kind), bins=int(bins), sink=int(sink), softmax_scale=1.0 / math.sqrt(head_dim))
    q_, k_, h_ = N.dl(query), N.dl(key), N.dl(out)
    N.check(N.lib().sq_attention_histogram(N.ptr(q_), N.ptr(k_), N.ptr(h_), params, N.current_stream(query.device)))
    return out


class CalibrationCapture:
    """What a layer's attention slot accumulates while a calibration runs: one histogram per query head."""

    def __init__(self, kind: int, bins: int, sink: int, num_heads: int, device):
        self.kind, self.bins, self.sink = kind, bins, sink
        self.hist = torch.zeros(1, num_heads, bins, dtype=torch.float64, device=device)

    def record(self, query_states: torch.Tensor, key_states: torch.Tensor) -> None:
        """query_states [B, N, Hq, D], key_states [B, N, Hkv, D]; sequences of a batch add into the same histograms."""
        for b in range(query_states.shape[0]):
            attention_histograms(query_states[b:b + 1], key_states[b:b + 1], self.kind, self.bins, self.sink, "NHD", out=self.hist)

    def numpy(self) -> np.ndarray:
        return self.hist[0].cpu().numpy()


# --------------------------------------------------------------------------------------- from a dense map
def _map_energy(attention_map: torch.Tensor, kind: int, bins: int, sink: int) -> np.ndarray:
    """One head's map [N, N] -> histogram [bins] (float64 numpy), the three binning rules in one place."""
    a = attention_map.to(torch.float32)
    n = a.shape[0]
    rows = torch.arange(n, device=a.device).view(n, 1)
    cols = torch.arange(n, device=a.device).view(1, n)
    dist = rows - cols
    keep = cols <= rows
    if kind != RELATIVE:
        keep = keep & (cols >= sink)
    if kind == ABSOLUTE:
        idx, weight = dist, a * dist.float()
        keep = keep & (dist < bins)
    else:
        if kind == RELATIVE:
            den = rows.clamp(min=1).float()
            scaled = dist.float() / den * bins
        else:
            den = (rows.float() - sink).clamp(min=1)
            scaled = dist.float() / den * bins
            scaled = torch.where(rows <= sink, torch.zeros_like(scaled), scaled)
        idx = scaled.floor().long().clamp(0, bins - 1)
        weight = a * dist.float() if kind == RELATIVE else a * (scaled + 1)
    hist = torch.zeros(bins, dtype=torch.float64, device=a.device)
    hist.index_add_(0, idx[keep], weight[keep].double())
    return hist.cpu().numpy()


def compute_attention_histogram(attention_map: np.ndarray, max_len: int) -> np.ndarray:
    """Host version (window_search.py:5-17): distance counted from 1, `hist[i-j+1] += A[i,j] * (i-j+1)`."""
    a = np.asarray(attention_map, dtype=np.float64)
    n = a.shape[0]
    hist = np.zeros(max_len)
    for d in range(1, min(n + 1, max_len)):
        hist[d] = np.trace(a, offset=-(d - 1)) * d   # the (d-1)-th sub-diagonal holds the pairs at distance d
    return hist


def compute_attention_histogram_gpu(attention_map: torch.Tensor, max_len: int) -> np.ndarray:
    """window_search.py:20-48."""
    return _map_energy(attention_map, ABSOLUTE, max_len, 0)


def compute_relative_attention_histogram_gpu(attention_map: torch.Tensor, num_bins: int = 100) -> np.ndarray:
    """window_search.py:51-87."""
    return _map_energy(attention_map, RELATIVE, num_bins, 0)


def compute_relative_attention_histogram_gpu_with_sink(attention_map: torch.Tensor, num_bins: int = 200, sink_len: int = 128) -> np.ndarray:
    """window_search.py:244-280."""
    return _map_energy(attention_map, RELATIVE_SINK, num_bins, sink_len)


def compute_absolute_attention_histogram_gpu_with_sink(attention_map: torch.Tensor, max_len: int, sink_len: int = 128) -> np.ndarray:
    """window_search.py:283-321."""
    return _map_energy(attention_map, ABSOLUTE, max_len, sink_len)


# --------------------------------------------------------------------------------------- windows from histograms
def find_optimal_relative_window(histogram: np.ndarray, threshold: float, num_bins: int = 100) -> float:
    """window_search.py:90-113: (first bin at which the running energy reaches the share, + 1) / num_bins, capped at 1;
    0.1 when there is no energy."""
    histogram = np.asarray(histogram, dtype=np.float64)
    total = histogram.sum()
    if total == 0:
        return 0.1
    reached = np.nonzero(np.cumsum(histogram) >= threshold * total)[0]
    first = int(reached[0]) if len(reached) else 0
    return min((first + 1) / num_bins, 1.0)


def find_optimal_window(histogram: np.ndarray, threshold: float) -> int:
    """window_search.py:116-128: smallest multiple of 128 tokens that holds the share; 1 when there is no energy."""
    histogram = np.asarray(histogram, dtype=np.float64)
    total = histogram.sum()
    if total == 0:
        return 1
    pad = (-len(histogram)) % 128
    per_block = np.pad(histogram, (0, pad)).reshape(-1, 128).sum(axis=1)
    reached = np.nonzero(np.cumsum(per_block) >= threshold * total)[0]
    return (int(reached[0]) + 1) * 128 if len(reached) else len(histogram)


# --------------------------------------------------------------------------------------- calibration drivers
def _num_heads(layer, model):
    if model is not None:
        return model.config.num_attention_heads
    return layer.self_attn.config.num_attention_heads


def _run_samples(layer, layer_idx, samples_inps, samples_layer_kwargs, model, capture):
    """Push every calibration sample through the layer with the capture active (window_search.py:142-159)."""
    layer.calibration = capture
    try:
        for i in range(len(samples_inps)):
            inps = samples_inps[i]
            if inps.ndim == 2:
                inps = inps[None, :, :]
            if model is not None:
                model.layer_prefill(layer_idx, 0, inps.clone())   # layer_prefill works in place; the samples stay as they are
            else:
                layer(inps, **samples_layer_kwargs[i])
    finally:
        layer.calibration = None


def calibrate_layer_windows_absolute(layer, layer_idx, samples_inps, samples_layer_kwargs, max_len, args, model=None):
    """window_search.py:131-176: per head, windows in tokens -> (largest 8-bit window, largest 4-bit window, per head)."""
    num_heads = _num_heads(layer, model)
    capture = CalibrationCapture(ABSOLUTE, int(max_len), 0, num_heads, samples_inps[0].device)
    _run_samples(layer, layer_idx, samples_inps, samples_layer_kwargs, model, capture)
    windows = []
    for head_idx, histogram in enumerate(capture.numpy()):
        windows.append({"head_idx": head_idx, "bit8": find_optimal_window(histogram, args.bit8_thres),
                        "bit4": find_optimal_window(histogram, args.bit4_thres)})
    return max(w["bit8"] for w in windows), max(w["bit4"] for w in windows), windows


def calibrate_layer_windows_relative(layer, layer_idx, samples_inps, samples_layer_kwargs, max_len, args, model=None):
    """window_search.py:179-228: per head, windows as a share of the context behind the sink."""
    num_heads = _num_heads(layer, model)
    num_bins = getattr(args, "relative_bins", 200)
    sink_len = getattr(args, "sink_window_size", 256)
    capture = CalibrationCapture(RELATIVE_SINK, num_bins, sink_len, num_heads, samples_inps[0].device)
    _run_samples(layer, layer_idx, samples_inps, samples_layer_kwargs, model, capture)
    windows = []
    for head_idx, histogram in enumerate(capture.numpy()):
        windows.append({"head_idx": head_idx,
                        "bit8_relative": find_optimal_relative_window(histogram, args.bit8_thres, num_bins),
                        "bit4_relative": find_optimal_relative_window(histogram, args.bit4_thres, num_bins),
                        "sink_len": sink_len})
    return max(w["bit8_relative"] for w in windows), max(w["bit4_relative"] for w in windows), windows


def calibrate_layer_windows(layer, layer_idx, samples_inps, samples_layer_kwargs, max_len, args, model=None):
    """window_search.py:231-241."""
    if getattr(args, "use_relative_distance", False):
        return calibrate_layer_windows_relative(layer, layer_idx, samples_inps, samples_layer_kwargs, max_len, args, model)
    return calibrate_layer_windows_absolute(layer, layer_idx, samples_inps, samples_layer_kwargs, max_len, args, model)
