"""Pins oracle/window_search.py (and the host-side map functions of sqattn/window_search.py, which run on CPU
tensors too) by element-by-element loops on tiny maps, closed forms and conservation sums."""
import math

import numpy as np
import pytest
import torch

from longcontext_sqattn_paddle_amd.sqattn import window_search as H
from oracle import window_search as W


def _random_map(n, seed, heads=1):
    rng = np.random.default_rng(seed)
    q = rng.standard_normal((heads, n, 16)) * 1.5
    k = rng.standard_normal((heads, n, 16)) * 1.5
    return W.attention_map(q, k)


def test_attention_map_is_causal_softmax():
    rng = np.random.default_rng(0)
    q, k = rng.standard_normal((4, 33, 8)), rng.standard_normal((2, 33, 8))
    a = W.attention_map(q, k, groups=2)
    assert a.shape == (4, 33, 33)
    assert np.allclose(a.sum(-1), 1.0, atol=1e-12) and np.triu(a, 1).max() == 0.0
    # row i, by hand: heads 2 and 3 read kv head 1
    i = 20
    s = (k[1, : i + 1] @ q[3, i]) / math.sqrt(8)
    assert np.allclose(a[3, i, : i + 1], np.exp(s - s.max()) / np.exp(s - s.max()).sum(), atol=1e-14)
    ref = torch.softmax(torch.from_numpy(q[0] @ k[0].T / math.sqrt(8)).masked_fill(~torch.ones(33, 33).tril().bool(), -math.inf), -1)
    assert np.allclose(a[0], ref.numpy(), atol=1e-14)


@pytest.mark.parametrize("kind,bins,sink", [(W.KIND_ABSOLUTE, 40, 0), (W.KIND_ABSOLUTE, 23, 5), (W.KIND_ABSOLUTE, 64, 3),
                                            (W.KIND_RELATIVE, 10, 0), (W.KIND_RELATIVE, 37, 0),
                                            (W.KIND_RELATIVE_SINK, 20, 4), (W.KIND_RELATIVE_SINK, 7, 0), (W.KIND_RELATIVE_SINK, 16, 11)])
def test_histogram_against_an_element_loop(kind, bins, sink):
    """Every (i, j) visited one at a time with scalar fp32 arithmetic for the bin, as the definitions read."""
    n = 37
    a = _random_map(n, 3 + kind)[0]
    want = np.zeros(bins)
    f = np.float32
    for i in range(n):
        for j in range(i + 1):
            d = i - j
            if kind == W.KIND_ABSOLUTE:
                if j >= sink and d < bins:
                    want[d] += a[i, j] * d
            elif kind == W.KIND_RELATIVE:
                rel = f(d) / f(max(i, 1))
                b = min(max(int(math.floor(rel * f(bins))), 0), bins - 1)
                want[b] += a[i, j] * d
            else:
                if j < sink:
                    continue
                rel = f(0) if i <= sink else f(d) / f(max(i - sink, 1))
                scaled = rel * f(bins)
                b = min(max(int(math.floor(scaled)), 0), bins - 1)
                want[b] += a[i, j] * float(scaled + f(1))
    got = W.histogram(a, kind, bins, sink)
    assert got.shape == (bins,)
    assert np.allclose(got, want, rtol=1e-12, atol=1e-14)
    # the host-side map functions follow the same definitions (fp32 maps there)
    t = torch.from_numpy(a).float()
    host = {W.KIND_ABSOLUTE: lambda: H.compute_absolute_attention_histogram_gpu_with_sink(t, bins, sink) if sink else H.compute_attention_histogram_gpu(t, bins),
            W.KIND_RELATIVE: lambda: H.compute_relative_attention_histogram_gpu(t, bins),
            W.KIND_RELATIVE_SINK: lambda: H.compute_relative_attention_histogram_gpu_with_sink(t, bins, sink)}[kind]()
    assert np.allclose(host, want, rtol=1e-5, atol=1e-6)


def test_closed_forms():
    n = 300
    # uniform rows: A[i, j] = 1/(i+1)  ->  hist[d] = d * sum_{i >= d} 1/(i+1)
    a = np.tril(np.ones((n, n))) / np.arange(1, n + 1)[:, None]
    h = W.histogram(a, W.KIND_ABSOLUTE, n)
    harmonic = np.cumsum(1.0 / np.arange(1, n + 1))
    for d in (0, 1, 7, 150, 299):
        assert math.isclose(h[d], d * (harmonic[-1] - (harmonic[d - 1] if d else 0.0)), rel_tol=1e-12, abs_tol=1e-14)
    # all mass on one sub-diagonal at distance w (rows above it look at themselves)
    w = 130
    a = np.zeros((n, n))
    a[np.arange(w, n), np.arange(0, n - w)] = 1.0
    a[np.arange(w), np.arange(w)] = 1.0
    h = W.histogram(a, W.KIND_ABSOLUTE, n)
    assert h[w] == w * (n - w) and h.sum() == h[w]
    assert W.find_optimal_window(h, 0.95) == 256 and H.find_optimal_window(h, 0.95) == 256
    # a sink row pattern: all mass on key 0 -> relative distance 1 for every row >= 1 -> last bin, weight i
    a = np.zeros((n, n))
    a[:, 0] = 1.0
    h = W.histogram(a, W.KIND_RELATIVE, 50)
    assert h[49] == n * (n - 1) / 2 and h[:49].sum() == 0.0
    assert W.find_optimal_relative_window(h, 0.9, 50) == 1.0 == H.find_optimal_relative_window(h, 0.9, 50)
    # ... and behind a sink of 16 tokens that key is not counted at all
    assert W.histogram(a, W.KIND_RELATIVE_SINK, 50, sink=16).sum() == 0.0
    # identity map: distance 0 everywhere; the sink variant weighs each row at or behind the sink with 1
    h = W.histogram(np.eye(n), W.KIND_RELATIVE_SINK, 50, sink=16)
    assert h[0] == n - 16 and h[1:].sum() == 0.0
    assert W.histogram(np.eye(n), W.KIND_ABSOLUTE, n).sum() == 0.0


def test_conservation_and_the_loop_variant():
    n = 90
    a = _random_map(n, 9)[0]
    expected_distance = (a * (np.arange(n)[:, None] - np.arange(n)[None, :])).sum()
    h_abs = W.histogram(a, W.KIND_ABSOLUTE, n)
    h_rel = W.histogram(a, W.KIND_RELATIVE, 25)
    assert math.isclose(h_abs.sum(), expected_distance, rel_tol=1e-12)
    assert math.isclose(h_rel.sum(), expected_distance, rel_tol=1e-12)   # same weights, other bins
    # truncation drops exactly the far distances
    assert np.array_equal(W.histogram(a, W.KIND_ABSOLUTE, 30), h_abs[:30])
    # a sink removes the columns below it and nothing else
    h_sink = W.histogram(a, W.KIND_ABSOLUTE, n, sink=10)
    left = (a[:, :10] * (np.arange(n)[:, None] - np.arange(10)[None, :])).sum()
    assert math.isclose(h_abs.sum() - h_sink.sum(), left, rel_tol=1e-10)
    # the host loop counts distance from 1: bin d holds the pairs at i - j = d - 1, weighted with d
    loop = W.histogram_loop(a, n + 1)
    diag_mass = np.array([np.trace(a, offset=-d) for d in range(n)])
    assert np.allclose(loop[1:], diag_mass * np.arange(1, n + 1), rtol=1e-12)
    assert loop[0] == 0.0
    assert np.allclose(h_abs[1:], diag_mass[1:] * np.arange(1, n), rtol=1e-12)
    assert np.allclose(H.compute_attention_histogram(a, n + 1), loop, rtol=1e-12)
    assert np.allclose(H.compute_attention_histogram(a, 20), W.histogram_loop(a, 20), rtol=1e-12)


def test_window_from_histogram_edge_cases():
    for mod in (W, H):
        assert mod.find_optimal_window(np.zeros(500), 0.9) == 1
        assert mod.find_optimal_relative_window(np.zeros(100), 0.9) == 0.1
        h = np.zeros(1000)
        h[5], h[300], h[900] = 50.0, 30.0, 20.0
        assert mod.find_optimal_window(h, 0.5) == 128
        assert mod.find_optimal_window(h, 0.51) == 384
        assert mod.find_optimal_window(h, 0.8) == 384
        assert mod.find_optimal_window(h, 0.81) == 1024     # the block [896, 1024) runs past the 1000 bins
        assert mod.find_optimal_window(h, 1.5) == 1000      # never reached: the histogram's length
        r = np.array([1.0, 0.0, 3.0, 6.0])
        assert mod.find_optimal_relative_window(r, 0.1, 4) == 0.25
        assert mod.find_optimal_relative_window(r, 0.4, 4) == 0.75
        assert mod.find_optimal_relative_window(r, 0.41, 4) == 1.0
        assert mod.find_optimal_relative_window(r, 2.0, 4) == 0.25   # never reached: the reference's bin 0
        assert mod.find_optimal_relative_window(r, 0.4, 2) == 1.0    # more bins than num_bins says: capped at 1


def test_host_and_oracle_agree_on_random_histograms():
    rng = np.random.default_rng(5)
    for _ in range(50):
        h = rng.random(rng.integers(1, 700)) * (rng.random() < 0.9)
        t = float(rng.random())
        assert H.find_optimal_window(h, t) == W.find_optimal_window(h, t)
        assert H.find_optimal_relative_window(h, t, 64) == W.find_optimal_relative_window(h, t, 64)
