"""Calibration histograms (`sq_attention_histogram`) and the window search built on them, against the oracle's dense
restatement (oracle/window_search.py) at sizes the [N, N] map still fits, and through sums the binning must conserve
at sizes where it does not."""
import math
from types import SimpleNamespace

import numpy as np
import pytest
import torch

from oracle import window_search as W

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def _qk(B, N, Hq, Hkv, D, seed, dtype=torch.bfloat16, gain=2.0):
    g = torch.Generator().manual_seed(seed)
    q = (torch.randn(B, N, Hq, D, generator=g) * gain).to(dtype)
    k = (torch.randn(B, N, Hkv, D, generator=g)).to(dtype)
    return q, k


def _oracle(q, k, kind, bins, sink):
    """q [B, N, Hq, D], k [B, N, Hkv, D] -> float64 [B, Hq, bins]"""
    B, N, Hq, D = q.shape
    out = np.zeros((B, Hq, bins))
    for b in range(B):
        a = W.attention_map(q[b].permute(1, 0, 2).double().numpy(), k[b].permute(1, 0, 2).double().numpy(), Hq // k.shape[2])
        for h in range(Hq):
            out[b, h] = W.histogram(a[h], kind, bins, sink)
    return out


def _close(got, want):
    """fp32 probabilities and fp32 partial sums on the GPU against float64: 1e-4 of a bin, or 1e-6 of the head's
    total energy for bins that hold next to nothing."""
    got = got.cpu().numpy()
    assert got.shape == want.shape
    tol = 1e-4 * np.abs(want) + 1e-6 * np.abs(want).sum(axis=-1, keepdims=True) + 1e-12
    bad = np.abs(got - want) > tol
    assert not bad.any(), (int(bad.sum()), float(np.abs(got - want).max()))


@pytest.mark.parametrize("kind,bins,sink", [(0, 333, 0), (0, 100, 0), (0, 400, 64), (0, 333, 7),
                                            (1, 100, 0), (1, 8192, 0), (2, 200, 256), (2, 50, 5), (2, 16, 0)])
@pytest.mark.parametrize("B,N,Hq,Hkv,D,dtype,layout", [(1, 333, 4, 2, 128, torch.bfloat16, "NHD"),
                                                      (2, 129, 6, 2, 64, torch.float16, "HND"),
                                                      (1, 64, 2, 2, 128, torch.bfloat16, "NHD")])
def test_histograms_match_the_dense_restatement(B, N, Hq, Hkv, D, dtype, layout, kind, bins, sink):
    from longcontext_sqattn_paddle_amd.sqattn.window_search import attention_histograms

    print(f"case histogram kind={kind} bins={bins} sink={sink} B={B} N={N} Hq={Hq} Hkv={Hkv} D={D} {dtype} {layout}", flush=True)
    q, k = _qk(B, N, Hq, Hkv, D, seed=17 * N + kind, dtype=dtype)
    want = _oracle(q, k, kind, bins, sink)
    qd, kd = q.to(DEV), k.to(DEV)
    if layout == "HND":
        qd, kd = qd.permute(0, 2, 1, 3).contiguous(), kd.permute(0, 2, 1, 3).contiguous()
    got = attention_histograms(qd, kd, kind, bins, sink, layout)
    torch.cuda.synchronize()
    assert got.dtype == torch.float64 and tuple(got.shape) == (B, Hq, bins)
    _close(got, want)


def test_histograms_accumulate_and_reject_bad_arguments():
    from longcontext_sqattn_paddle_amd.sqattn.window_search import attention_histograms

    q, k = _qk(1, 200, 4, 1, 128, seed=5)
    qd, kd = q.to(DEV), k.to(DEV)
    once = attention_histograms(qd, kd, 2, 64, 16)
    acc = attention_histograms(qd, kd, 2, 64, 16, out=once.clone())
    torch.cuda.synchronize()
    # (fp32 atomics into the LDS histogram land in a different order every launch)
    assert torch.allclose(acc, 2 * once, rtol=1e-5, atol=0)
    # strided views: every second token of a longer tensor
    q2, k2 = _qk(1, 400, 4, 1, 128, seed=6)
    view = attention_histograms(q2.to(DEV)[:, ::2], k2.to(DEV)[:, ::2], 0, 200)
    dense = attention_histograms(q2[:, ::2].contiguous().to(DEV), k2[:, ::2].contiguous().to(DEV), 0, 200)
    assert torch.allclose(view, dense, rtol=1e-5, atol=1e-9)
    with pytest.raises(ValueError):
        attention_histograms(qd, kd, 1, 64, sink=16)        # the plain relative histogram has no sink
    with pytest.raises(ValueError):
        attention_histograms(qd, kd, 2, 8193, sink=16)      # relative bins live in LDS
    with pytest.raises(ValueError):
        attention_histograms(qd, kd, 3, 64)
    with pytest.raises(ValueError):
        attention_histograms(qd, kd, 0, 0)
    with pytest.raises(AssertionError):
        attention_histograms(qd, kd[:, :100], 0, 64)
    with pytest.raises(RuntimeError):
        attention_histograms(q, k, 0, 64)                   # CPU tensors: there is no host path


def test_long_sequence_conservation():
    """N = 16384, 28/4 heads: the dense map would take 30 GB.  What the binning must conserve: the absolute histogram
    with every distance kept and the relative histogram spread the same weights p (i - j) over different bins, so
    their totals agree per head; and the total is the mean attention distance summed over rows, which a chunked
    exact softmax gives independently."""
    from longcontext_sqattn_paddle_amd.sqattn.window_search import attention_histograms

    N, Hq, Hkv, D = 16384, 28, 4, 128
    q, k = _qk(1, N, Hq, Hkv, D, seed=8, gain=1.5)
    qd, kd = q.to(DEV), k.to(DEV)
    h_abs = attention_histograms(qd, kd, 0, N)
    h_rel = attention_histograms(qd, kd, 1, 100)
    h_cut = attention_histograms(qd, kd, 0, 1000)
    torch.cuda.synchronize()
    assert torch.allclose(h_abs.sum(-1), h_rel.sum(-1), rtol=1e-6)
    assert torch.allclose(h_cut, h_abs[..., :1000], rtol=1e-6, atol=1e-9)
    # independent total for two heads: rows in chunks, float64 softmax on the device
    pos = torch.arange(N, device=DEV, dtype=torch.float64)
    for h in (0, 27):
        total = 0.0
        for r0 in range(0, N, 2048):
            s = (qd[0, r0:r0 + 2048, h].double() @ kd[0, :, h // 7].double().T) / math.sqrt(D)
            rows = pos[r0:r0 + 2048, None]
            s = s.masked_fill(pos[None, :] > rows, -math.inf)
            p = torch.softmax(s, dim=-1)
            total += float((p * (rows - pos[None, :]).clamp(min=0)).sum())
        assert math.isclose(float(h_abs[0, h].sum()), total, rel_tol=1e-5)


def test_compress_model_installs_windows_that_the_dense_path_confirms():
    """Two calibration samples through a 4-layer decoder: layers 1 and 2 get windows.  Layer 1 is re-derived by hand:
    its inputs through layer 0, Q and K by the runtime's own projections, the dense map and its histogram per head
    (oracle), the search on the summed histograms."""
    from longcontext_sqattn_paddle_amd.model_hub.qwen import QwenConfig, QwenModel
    from longcontext_sqattn_paddle_amd.sqattn import compress as C

    cfg = QwenConfig(hidden_size=512, intermediate_size=1024, num_hidden_layers=4, num_attention_heads=4, num_key_value_heads=2,
                     vocab_size=1000, max_position_embeddings=4096)
    g = torch.Generator().manual_seed(3)
    samples = [torch.randint(0, 1000, (1, 700), generator=g).to(DEV), torch.randint(0, 1000, (1, 450), generator=g).to(DEV)]
    for relative in (False, True):
        model = QwenModel("tiny-qwen", max_length=1024, dtype=torch.bfloat16, device_map=DEV, attention_type="SQAttn", config=cfg, seed=11)
        args = SimpleNamespace(attn_type="SQAttn", bit8_thres=0.6, bit4_thres=0.9, use_relative_distance=relative, relative_bins=40,
                               sink_window_size=64, quant=True, qk_qtype="int", v_qtype="int")
        # by hand, before compress_model replaces any attention slot
        want = None
        for s in samples:
            x, _ = C.get_layer_inputs(model, s, args)
            model.batch_size, model.max_new_length = 1, 0
            model.init_kv_cache(s.shape[1], [0])
            x = model.layer_prefill(0, 0, x.clone())
            layer = model.layers[1]
            normed = model.layernorm(x, layer.input_layernorm_variance_epsilon, layer.input_layernorm_weight)
            qs, ks, _ = model.wqkv(normed, layer)
            qs, ks = model.position_embedd(qs, ks)
            qs = qs.view(1, -1, 4, 128).cpu()
            ks = ks.view(1, -1, 2, 128).cpu()
            h = _oracle(qs, ks, 2, 40, 64)[0] if relative else _oracle(qs, ks, 0, 700, 0)[0]
            want = h if want is None else want + h
        alloc = C.compress_model(model, None, DEV, args, raw_samples=samples)
        torch.cuda.synchronize()
        assert sorted(alloc) == [1, 2]
        for li in (1, 2):
            assert alloc[li]["sink"] == 256 and len(alloc[li]["bit8"]) == 4 and len(alloc[li]["bit4"]) == 4
            assert model.layers[li].prefill_attention.__func__.__name__ == "attention_fn"
            assert model.layers[li].calibration is None
        assert model.layers[0].prefill_attention.__func__.__name__ == "prefill_attention"
        for head in range(4):
            if relative:
                assert alloc[1]["bit8"][head] == W.find_optimal_relative_window(want[head], 0.6, 40)
                assert alloc[1]["bit4"][head] == W.find_optimal_relative_window(want[head], 0.9, 40)
                assert 0 < alloc[2]["bit8"][head] <= alloc[2]["bit4"][head] <= 1.0
            else:
                assert alloc[1]["bit8"][head] == W.find_optimal_window(want[head], 0.6)
                assert alloc[1]["bit4"][head] == W.find_optimal_window(want[head], 0.9)
                assert alloc[2]["bit8"][head] % 128 == 0 and alloc[2]["bit8"][head] <= alloc[2]["bit4"][head]
        # the calibrated model still generates
        out = model.generate("SQAttn", samples[0][:, :512], None, 4, verbose=False)
        assert len(out) == 1 and len(out[0]) == 4
