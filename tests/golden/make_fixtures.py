"""Writes the golden fixtures of this directory: small seeded inputs and the outputs of the CPU oracle for them.

The reference ships no golden vectors for this path and cannot be run here (its modules import PaddlePaddle), so the
vectors are produced by the oracle, whose functions are pinned by closed forms, brute force and invariants in
tests/test_oracle_*.py.  What the fixtures add: a frozen record that later changes of the oracle or of the kernels
are compared with (tests/test_golden_cpu.py: oracle against file; tests/test_gpu_golden.py: kernels against file).

    python tests/golden/make_fixtures.py        # rewrites tests/golden/*.npz

16-bit tensors are stored as their bit patterns (uint16), everything with numpy.savez_compressed, no pickles.
"""
import os
import sys

import numpy as np
import torch

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.join(HERE, "..", ".."))

from oracle import attention as A  # noqa: E402
from oracle import kmeans as K  # noqa: E402
from oracle import plugin as P  # noqa: E402
from oracle import window_search as W  # noqa: E402


def bits(t: torch.Tensor) -> np.ndarray:
    return t.contiguous().view(torch.int16).numpy().view(np.uint16)


def randn(shape, seed, scale=1.0, dtype=torch.bfloat16):
    g = torch.Generator().manual_seed(seed)
    return (torch.randn(*shape, generator=g) * scale).to(dtype)


def prefill():
    q, k, v = randn((1, 4, 192, 128), 101), randn((1, 2, 192, 128), 102), randn((1, 2, 192, 128), 103)
    out = {"q": bits(q), "k": bits(k), "v": bits(v)}
    for name, mode in (("none", A.P_NONE), ("e4m3_static", A.P_STATIC448), ("e4m3_block", A.P_BLOCK_ABSMAX)):
        o, lse = A.prefill_blockwise(q, k, v, p_quant=mode, out_dtype=torch.float32)
        out[f"out_{name}"], out[f"lse_{name}"] = o.numpy(), lse.numpy()
    # the two fp8 P.V modes (e4m3 V with a per-channel power-of-two scale; P on the static grid / with a per-row tile scale)
    for name, mode in (("fp8pv", A.P_STATIC448_GRID), ("mx_fp8pv", A.P_MX_ROW)):
        o, lse = A.prefill_blockwise(q, k, v, p_quant=mode, v_quant="e4m3_channel", out_dtype=torch.float32)
        out[f"out_{name}"], out[f"lse_{name}"] = o.numpy(), lse.numpy()
    # sink 64 + per-head windows (8-bit 64 / 128 / 64 / 128 tokens, 4-bit 128 / 128 / 192 / 192), 64-row query blocks
    o, lse = A.prefill_blockwise(q, k, v, out_dtype=torch.float32, block_m=64, sink=64, w8=[64, 128, 64, 128], w4=[128, 128, 192, 192])
    out["out_window"], out["lse_window"] = o.numpy(), lse.numpy()
    o, lse = A.prefill_blockwise(q, k, v, p_quant=A.P_MX_ROW, v_quant="e4m3_channel", out_dtype=torch.float32, block_m=64, sink=64,
                                 w8=[64, 128, 64, 128], w4=[128, 128, 192, 192])
    out["out_window_mx_fp8pv"], out["lse_window_mx_fp8pv"] = o.numpy(), lse.numpy()
    np.savez_compressed(os.path.join(HERE, "prefill_small.npz"), **out)


def decode():
    q, k, v = randn((2, 8, 1, 128), 111), randn((2, 2, 300, 128), 112), randn((2, 2, 300, 128), 113)
    lens = [300, 171]
    o, lse = A.decode_blockwise(q, k, v, kv_lens=lens)
    np.savez_compressed(os.path.join(HERE, "decode_small.npz"), q=bits(q), k=bits(k), v=bits(v), lens=np.array(lens, dtype=np.int32),
                        out=o.numpy(), lse=lse.numpy())


def prepass():
    q, k, v = randn((1, 96, 4, 128), 121, 2.0), randn((1, 96, 2, 128), 122, 3.0), randn((1, 96, 2, 128), 123)
    k = (k.float() + 1.5).to(torch.bfloat16)   # a key mean worth removing
    q8, q4, k8, k4, v8 = P.int_prepass(q, k, v, want_4bit=True)
    np.savez_compressed(os.path.join(HERE, "prepass_small.npz"), q=bits(q), k=bits(k), v=bits(v), q8=bits(q8), q4=bits(q4), k8=bits(k8),
                        k4=bits(k4), v8=bits(v8))


def kmeans():
    g = torch.Generator().manual_seed(131)
    centres = torch.randn(2, 24, 128, generator=g)
    which = torch.randint(0, 24, (2, 768), generator=g)
    key = (torch.gather(centres, 1, which[..., None].expand(-1, -1, 128)) + 0.3 * torch.randn(2, 768, 128, generator=g)).bfloat16()
    value = randn((2, 768, 128), 132)
    cent, vsum, clusters, size = K.segment_k_means(key, value, 32, num_iters=4, num_segments=1)
    np.savez_compressed(os.path.join(HERE, "kmeans_small.npz"), key=bits(key), value=bits(value), centroids=bits(cent), value_sum=bits(vsum),
                        clusters=clusters.numpy().astype(np.int32), cluster_size=size.numpy().astype(np.int32))


def window_search():
    q, k = randn((1, 200, 4, 128), 141, 2.0), randn((1, 200, 2, 128), 142)
    a = W.attention_map(q[0].permute(1, 0, 2).double().numpy(), k[0].permute(1, 0, 2).double().numpy(), 2)
    out = {"q": bits(q), "k": bits(k)}
    for name, kind, nbins, sink in (("absolute", 0, 200, 0), ("absolute_sink", 0, 128, 32), ("relative", 1, 50, 0), ("relative_sink", 2, 40, 32)):
        out[name] = np.stack([W.histogram(a[h], kind, nbins, sink) for h in range(4)])
    out["window_absolute_0p9"] = np.array([W.find_optimal_window(h, 0.9) for h in out["absolute"]], dtype=np.int32)
    out["window_relative_0p9"] = np.array([W.find_optimal_relative_window(h, 0.9, 40) for h in out["relative_sink"]])
    np.savez_compressed(os.path.join(HERE, "window_search_small.npz"), **out)


if __name__ == "__main__":
    todo = {f.__name__: f for f in (prefill, decode, prepass, kmeans, window_search)}
    for name in (sys.argv[1:] or list(todo)):   # optional arguments: the fixtures to rewrite
        todo[name]()
        print("wrote", name)
