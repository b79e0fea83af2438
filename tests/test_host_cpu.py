"""CPU checks of the host-side mirror of the reference interface (no kernel call)."""
import types

import pytest
import torch

from oracle import fake_quant as FQ


def test_fake_quant_classes_match_oracle_on_cpu():
    from longcontext_sqattn_paddle_amd.sqattn.fake_quant import FloatQuantizer, IntegerQuantizer, float_quantize

    x = torch.randn(1, 2, 33, 64, generator=torch.Generator().manual_seed(4)).bfloat16()
    for bit, sym, gran in ((8, True, "per_token"), (4, True, "per_token"), (8, True, "per_channel"), (8, False, "per_token"),
                           (8, True, "per_tensor")):
        assert torch.equal(IntegerQuantizer(bit, sym, gran).fake_quant_tensor(x), FQ.int_fake_quant(x, bit, sym, gran))
    for fmt in ("e4m3", "e5m2"):
        assert torch.equal(FloatQuantizer(fmt, True, "per_token").fake_quant_tensor(x), FQ.float_fake_quant(x, fmt, "per_token"))
    kat = torch.tensor([448.0, 300.0, 1.96, 2.0 ** -8, 0.0, -3.3])
    assert torch.equal(float_quantize(kat, 4, 3), torch.tensor([224.0, 144.0, 1.875, 2.0 ** -6, 0.0, -3.25]))
    q, s, z = IntegerQuantizer(8, True, "per_token").real_quant_tensor(x)
    assert z is None and float(q.abs().max()) <= 128 and s.shape == (1, 2, 33, 1)
    with pytest.raises(AssertionError):
        FloatQuantizer("e3m4", True, "per_token")


def test_process_model_and_window_normalisation():
    from longcontext_sqattn_paddle_amd.sqattn import attn_replacer as R
    from longcontext_sqattn_paddle_amd.sqattn.attn_triton_mix_relative import window_tokens

    assert R._normalise_windows([1, 2], 3) == ([1, 2], [3, 3])
    assert R._normalise_windows(None, None) == (0, 0)
    assert R._normalise_windows(5, [1, 2, 3]) == ([5, 5, 5], [1, 2, 3])
    assert window_tokens(0.1, 131072) == 13184 and window_tokens(0.1, 4096) == 512 and window_tokens(0.0, 77) == 0
    model = types.SimpleNamespace(layers=[types.SimpleNamespace(), types.SimpleNamespace()])
    args = types.SimpleNamespace(qk_qtype="int", v_qtype="int", use_relative_distance=True)
    R.process_model(model, "SQAttn", {1: {"bit8": 0.1, "bit4": 0.1, "sink": 8}}, args)
    assert hasattr(model.layers[1], "prefill_attention") and not hasattr(model.layers[0], "prefill_attention")
    with pytest.raises(ValueError, match="Unsupported attention type"):
        R.process_model(model, "Sage")
    bad = types.SimpleNamespace(qk_qtype="fp4", v_qtype="int", use_relative_distance=True)
    with pytest.raises(ValueError, match="Invalid quantization type"):
        R._quantizers(bad)
    x = torch.arange(2 * 3 * 2 * 4, dtype=torch.float32).view(2, 3, 2, 4)
    r = R.repeat_kv(x, 3)
    assert r.shape == (2, 6, 3, 4) and torch.equal(r[:, 0], r[:, 2]) and torch.equal(r[:, 3], x[:, :, 1])


def test_sdpa_forward_shapes_on_cpu():
    from longcontext_sqattn_paddle_amd.sqattn.sdpa_attention import sdpa_attention_forward

    mod = types.SimpleNamespace(num_key_value_groups=2)
    q = torch.randn(1, 10, 4, 16)
    k = torch.randn(1, 10, 2, 16)
    out = sdpa_attention_forward(mod, q, k, k, attention_mask=None, scaling=1.0, is_causal=True)
    assert out.shape == (1, 10, 64)
    ref = torch.nn.functional.scaled_dot_product_attention(q.permute(0, 2, 1, 3), k.permute(0, 2, 1, 3).repeat_interleave(2, 1),
                                                           k.permute(0, 2, 1, 3).repeat_interleave(2, 1), is_causal=True)
    assert torch.allclose(out, ref.transpose(1, 2).reshape(1, 10, 64), atol=1e-6)


def test_calibration_host_logic_without_a_gpu():
    """`compress_model` needs token samples (no dataset loading here); the calibration drivers refuse CPU tensors
    loudly instead of falling back; the capture object only exists on a device."""
    import pytest
    import torch

    from longcontext_sqattn_paddle_amd.sqattn import compress, window_search

    with pytest.raises(ValueError):
        compress.compress_model(model=None, tokenizer=None, device="cuda:0", args=None)
    q = torch.zeros(1, 8, 2, 128, dtype=torch.bfloat16)
    with pytest.raises(RuntimeError):
        window_search.attention_histograms(q, q, window_search.ABSOLUTE, 8)
    assert (window_search.ABSOLUTE, window_search.RELATIVE, window_search.RELATIVE_SINK) == (0, 1, 2)
    assert compress.SINK_TOKENS == 256 and compress.MAX_SAMPLE_TOKENS == 5000


def test_align_windows_rule():
    from longcontext_sqattn_paddle_amd.sqattn._prefill import align_windows

    # multiples of 64 stay as given (the reference walks them in 64-key blocks); others go up to the next multiple of 64
    assert align_windows([0, 128, 13184], [0, 256, 13184], 256, 64) == ([0, 128, 13184], [0, 256, 13184], 256)
    assert align_windows([1, 129, 1000], [1, 129, 1000], 100, 128) == ([64, 192, 1024], [64, 192, 1024], 128)
    assert align_windows([192, 64, 320], [320, 64, 192], 192, 128) == ([192, 64, 320], [320, 64, 192], 192)
    # 8-bit window below the query block under a wider 4-bit window: raised to the block
    assert align_windows([0, 0, 64], [384, 0, 0], 0, 64) == ([64, 0, 64], [384, 0, 0], 0)
    assert align_windows([0], [256], 0, 128) == ([128], [256], 0)


def _brute_mix_mask(kv_len, w8, w4, sink):
    """Element loop from the written semantics: row i sees 8-bit key j iff j <= i and (j < sink or j > i - w8); the
    4-bit copy of key j iff j >= sink and i - w8 - w4 < j <= i - w8."""
    m = torch.zeros(kv_len, 2 * kv_len, dtype=torch.bool)
    for i in range(kv_len):
        for j in range(kv_len):
            m[i, j] = j <= i and (j < sink or j > i - w8)
            m[i, kv_len + j] = j >= sink and (i - w8 - w4 < j <= i - w8)
    return m


def test_mix_bit_mask_restatements_against_element_loops():
    from longcontext_sqattn_paddle_amd.sqattn.attn_replacer import construct_mix_bit_mask
    from oracle import plugin

    for kv_len, w8, w4, sink in ((24, 5, 7, 3), (17, 0, 4, 0), (16, 100, 100, 2), (9, 1, 0, 4)):
        want = _brute_mix_mask(kv_len, w8, w4, sink)
        assert torch.equal(plugin.mix_bit_mask(kv_len, w8, w4, sink), want)
        assert torch.equal(construct_mix_bit_mask(kv_len, w8, w4, sink, "cpu"), want)
    # every key is seen at most once per row (8-bit copy or 4-bit copy), and the row's own token always as 8-bit
    m = plugin.mix_bit_mask(40, 6, 9, 4)
    assert not bool((m[:, :40] & m[:, 40:]).any()) and bool(torch.diagonal(m[:, :40]).all())
    # per-head lists
    w8s, w4s = [5, 0, 12], [7, 3, 0]
    want = torch.stack([_brute_mix_mask(20, a, b, 2) for a, b in zip(w8s, w4s)])
    assert torch.equal(plugin.mix_bit_mask(20, w8s, w4s, 2), want)
    assert torch.equal(construct_mix_bit_mask(20, w8s, w4s, 2, "cpu"), want)


def test_delayed_sdpa_wrapper_quantised_branch_matches_the_oracle():
    """The masked-SDPA emulation over [8-bit keys ; 4-bit keys] (attn_replacer.py:123-186), host code on torch: runs on
    the CPU, so it is checked here against the oracle's float64 restatement."""
    import types

    from longcontext_sqattn_paddle_amd.sqattn.attn_replacer import delayed_sdpa_wrapper
    from oracle import plugin

    g = torch.Generator().manual_seed(5)
    q, k, v = (torch.randn(1, 3, 48, 32, generator=g) for _ in range(3))
    k = k + 0.7
    args = types.SimpleNamespace(quant=True, qk_qtype="int", v_qtype="int", vis_attn=False)
    for w8, w4 in ((6, 10), ([4, 9, 48], [8, 0, 5])):
        out = delayed_sdpa_wrapper(0, w8, w4, 4, args)(None, q, k, v, None, scaling=1.0)
        ref = plugin.masked_sdpa_emulation(q, k, v, bit8_window=w8, bit4_window=w4, sink=4)
        assert out.shape == (1, 48, 3 * 32)
        got = out.view(1, 48, 3, 32).permute(0, 2, 1, 3).double()
        assert float((got - ref).abs().max()) < 1e-5
    # the plain branch is SDPA with the caller's mask
    plain = delayed_sdpa_wrapper(0, 0, 0, 0, types.SimpleNamespace(quant=False))(None, q, k, v, None, tensor_layout="HND")
    want = torch.nn.functional.scaled_dot_product_attention(q, k, v, is_causal=True).transpose(1, 2).reshape(1, 48, 96)
    assert torch.allclose(plain, want, atol=1e-6)


def test_decode_shares_by_length_add_up():
    """The rule by which the decode kernels deal the W workgroups of a ragged batch to its sequences (csrc/decode_gfx950.hip,
    share_of): every sequence one workgroup, the other W - B by cumulative rounding down of (W - B) * prefix / total in
    32-bit integers, the lengths counted in units of 32 tokens and prefix and total shifted right until the total is
    below 2^20.  Replayed in Python integers: the product fits 32 bits, the shares are positive, add up to W exactly, stay
    within one (plus 2^-19 of W - B) of a sequence's proportional share, and follow the lengths."""
    import numpy as np

    rng = np.random.default_rng(11)
    for case in range(300):
        B = int(rng.integers(2, 33))
        S = int(rng.integers(2, 129))
        W = B * S
        kind = case % 4
        if kind == 0:
            lens = rng.integers(0, 2 ** 31 - 1, B)
        elif kind == 1:
            lens = rng.integers(98304, 131073, B)
        elif kind == 2:
            lens = np.where(rng.random(B) < 0.5, 0, rng.integers(1, 5000, B))
        else:
            lens = np.full(B, int(rng.integers(1, 2 ** 20)))
        units = (lens.astype(np.uint64) + 31) >> 5
        cum = np.cumsum(units).astype(np.uint32)           # fits 32 bits: 32 sequences of 2^26 units
        total = cum[-1]
        sh = max(0, int(total).bit_length() - 20)
        ts = int(total) >> sh
        assert ts < 2 ** 20 and (W - B) * ts < 2 ** 32       # the kernel's product fits its 32-bit integer
        e1 = np.array([(W - B) * (int(c) >> sh) // ts for c in cum], dtype=np.int64) if ts > 0 else np.zeros(B, np.int64)
        e0 = np.concatenate([[0], e1[:-1]])
        n = 1 + e1 - e0
        base = np.arange(B) + e0
        assert (n >= 1).all()
        if total > 0:
            assert int(n.sum()) == W and int(base[-1] + n[-1]) == W
            want = (W - B) * units.astype(np.float64) / float(total)
            assert (np.abs((n - 1) - want) < 1.0 + (W - B) * 2.0 ** -19 + 1e-9).all()
        else:
            assert (n == 1).all()
        assert (base[1:] == base[:-1] + n[:-1]).all()
