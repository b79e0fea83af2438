"""Pins the fake-quantiser restatement with closed forms and hand-derived known answers."""
import torch

from oracle import fake_quant as FQ


def test_round_half_away():
    x = torch.tensor([0.5, 1.5, 2.5, -0.5, -2.5, 0.49, -1.2])
    assert FQ.round_half_away(x).tolist() == [1.0, 2.0, 3.0, -1.0, -3.0, 0.0, -1.0]


def test_int8_per_token_symmetric_closed_form():
    g = torch.Generator().manual_seed(0)
    x = torch.randn(1, 2, 16, 64, generator=g).bfloat16()
    y = FQ.int_fake_quant(x, 8, True, "per_token")
    x32 = x.float()
    s = x32.abs().amax(-1, keepdim=True) / 127
    exp = (torch.clamp(torch.sign(x32 / s) * torch.floor((x32 / s).abs() + 0.5), -128, 127) * s).bfloat16()
    assert torch.equal(y, exp)
    # the absmax element of every token maps to exactly +-127 * scale
    idx = x32.abs().argmax(-1, keepdim=True)
    assert torch.equal(torch.gather(y, -1, idx), (torch.gather(torch.sign(x32), -1, idx) * 127 * s).bfloat16())
    # error bound: half a step (plus bf16 output rounding)
    assert float(((y.float() - x32).abs() / s).max()) <= 0.5 + 1.0
    # 4-bit grid has at most 16 levels per token
    y4 = FQ.int_fake_quant(x, 4, True, "per_token").float()
    s4 = x32.abs().amax(-1, keepdim=True) / 7
    lv = torch.round(y4 / s4)
    assert lv.min() >= -8 and lv.max() <= 7


def test_per_channel_reduces_over_dims_0_and_1():
    # for [B,H,N,D] the range is per (token, channel), shared by batch and heads (fake_quant.py:30-32)
    x = torch.zeros(2, 3, 4, 5)
    x[1, 2, 3, 4] = 10.0
    x[0, 0, 3, 4] = 1.0
    x[0, 0, 0, 0] = 1.0
    y = FQ.int_fake_quant(x, 8, True, "per_channel")
    assert abs(float(y[0, 0, 3, 4]) - round(1.0 / (10 / 127)) * (10 / 127)) < 1e-6   # shares the scale of 10.0
    assert float(y[0, 0, 0, 0]) == 1.0                                              # own scale


def test_asymmetric_closed_form():
    x = torch.tensor([[[[-1.0, 0.0, 0.25, 3.0]]]])
    y = FQ.int_fake_quant(x, 8, False, "per_token")
    s = 4.0 / 255
    z = min(max(0 - FQ.round_half_away(torch.tensor(-1.0 / s)).item(), 0), 255)
    exp = [(min(max(FQ.round_half_away(torch.tensor(v / s)).item() + z, 0), 255) - z) * s for v in (-1.0, 0.0, 0.25, 3.0)]
    assert torch.allclose(y.flatten(), torch.tensor(exp), atol=1e-6)


def test_float_quantize_known_answers():
    # worked by hand from fake_quant.py:165-199 (exponent clamp to [1-bias, 2^(e-1)-1], mantissa clip,
    # no subnormals): e4m3 tops out at 240, folds inputs >= 256 into the 2^7 binade, maps tiny inputs up.
    x = torch.tensor([448.0, 300.0, 240.0, 196.0, 1.96, 1.0, 0.02, 2.0 ** -6, 2.0 ** -8, 1e-4, 0.0, -3.3])
    exp = torch.tensor([224.0, 144.0, 240.0, 192.0, 1.875, 1.0, 0.01953125, 2.0 ** -6, 2.0 ** -6, 0.025390625, 0.0, -3.25])
    assert torch.equal(FQ.float_quantize(x, 4, 3), exp)
    # 200 = 1.5625 * 2^7 is an exact mantissa tie (4.5 steps): `paddle.round` is documented as
    # half-away-from-zero -> 5 steps -> 208 (a half-to-even round would give 192)
    assert float(FQ.float_quantize(torch.tensor([200.0]), 4, 3)) == 208.0
    x5 = torch.tensor([57344.0, 60000.0, 1e-6, 3.3])
    exp5 = torch.tensor([57344.0, 57344.0, 2.0 ** -14, 3.5])
    assert torch.equal(FQ.float_quantize(x5, 5, 2), exp5)


def test_float_fake_quant_scale():
    x = torch.tensor([[[[0.5, -2.0, 1.0, 0.1]]]])
    y = FQ.float_fake_quant(x, "e4m3", "per_token")
    s = 2.0 / 448
    # absmax element scales to 448 -> folded to 224 by the simulation -> comes back at half its value
    assert abs(float(y[0, 0, 0, 1]) + 224 * s) < 1e-6
    assert abs(float(y[0, 0, 0, 0]) - 112 * s) < 1e-6    # 0.5/s = 112 = 1.75*2^6 exactly representable
