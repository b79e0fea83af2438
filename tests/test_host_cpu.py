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
