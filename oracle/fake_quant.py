"""CPU restatement of the reference's fake quantisers (sqattn/fake_quant.py).

TEST INFRASTRUCTURE ONLY (see `oracle/__init__.py`).
"""
from __future__ import annotations

import torch


def round_half_away(x: torch.Tensor) -> torch.Tensor:
    """`paddle.round` rounds half away from zero (torch.round rounds half to even)."""
    return torch.sign(x) * torch.floor(torch.abs(x) + 0.5)


def _minmax(x32: torch.Tensor, granularity: str):
    """`BaseQuantizer.get_minmax_range` (fake_quant.py:23-38)."""
    if granularity == "per_tensor":
        return x32.min(), x32.max()
    if granularity == "per_channel":
        return x32.amin(dim=(0, 1), keepdim=True), x32.amax(dim=(0, 1), keepdim=True)
    return x32.amin(dim=-1, keepdim=True), x32.amax(dim=-1, keepdim=True)


def int_fake_quant(x: torch.Tensor, bit: int, symmetric: bool, granularity: str) -> torch.Tensor:
    """`IntegerQuantizer(bit, symmetric, granularity).fake_quant_tensor(x)`
    (fake_quant.py:43-58, 80-86, 98-125)."""
    x32 = x.float()
    mn, mx = _minmax(x32, granularity)
    if symmetric:
        qmin, qmax = float(-(2 ** (bit - 1))), float(2 ** (bit - 1) - 1)
        scale = torch.maximum(mx.abs(), mn.abs()).clamp(min=1e-5) / qmax
        zero = torch.tensor(0.0)
    else:
        qmin, qmax = 0.0, float(2 ** bit - 1)
        scale = (mx - mn).clamp(min=1e-5) / (qmax - qmin)
        zero = (qmin - round_half_away(mn / scale)).clamp(qmin, qmax)
    qv = (round_half_away(x32 / scale) + zero).clamp(qmin, qmax)
    return ((qv - zero) * scale).to(x.dtype)


def int_quant_codes(x: torch.Tensor, bit: int = 8):
    """The integer codes and the fp32 scale behind `IntegerQuantizer(bit, True, "per_token").fake_quant_tensor(x)`
    (fake_quant.py:33-35, 47-52, 114-125): `codes = clamp(round(x / scale), qmin, qmax)` (fp32 tensor of whole numbers),
    `scale = max(|x|) .clip(1e-5) / qmax` over the last dimension, so that `int_fake_quant(x, bit, True, "per_token") ==
    (codes * scale).to(x.dtype)`.  This is what a real integer Q.K^T consumes: the codes go through the integer matrix
    instruction and the two scales multiply the sum."""
    x32 = x.float()
    mn, mx = _minmax(x32, "per_token")
    qmin, qmax = float(-(2 ** (bit - 1))), float(2 ** (bit - 1) - 1)
    scale = torch.maximum(mx.abs(), mn.abs()).clamp(min=1e-5) / qmax
    codes = (round_half_away(x32 / scale) + torch.tensor(0.0)).clamp(qmin, qmax)
    return codes, scale


def float_quantize(x: torch.Tensor, e_bits: int, m_bits: int) -> torch.Tensor:
    """The home-made float simulation, nearest rounding (fake_quant.py:151-204)."""
    bias = 2 ** (e_bits - 1) - 1
    eps = 2.0 ** (-m_bits)
    max_exp = 2 ** (e_bits - 1) - 1
    min_exp = 1 - bias
    sign = torch.sign(x)
    a = torch.abs(x)
    zero_mask = a == 0
    exp = torch.floor(torch.log2(a + 1e-30))
    frac = a / (2.0 ** exp) - 1.0
    exp_c = exp.clamp(min_exp, max_exp)
    frac_q = (round_half_away(frac / eps) * eps).clamp(0.0, 1.0 - eps)
    xq = (1.0 + frac_q) * (2.0 ** exp_c) * sign
    max_val = (2 - 2 ** (-m_bits)) * (2.0 ** max_exp)
    xq = xq.clamp(-max_val, max_val)
    return torch.where(zero_mask, torch.zeros_like(xq), xq)


def float_fake_quant(x: torch.Tensor, fmt: str, granularity: str) -> torch.Tensor:
    """`FloatQuantizer(fmt, True, granularity).fake_quant_tensor(x)` (fake_quant.py:207-248)."""
    e_bits, m_bits, fmax = {"e4m3": (4, 3, 448.0), "e5m2": (5, 2, 57344.0)}[fmt]
    x32 = x.float()
    mn, mx = _minmax(x32, granularity)
    scale = torch.maximum(mx.abs(), mn.abs()).clamp(min=1e-5) / fmax
    t = (x32 / scale).clamp(-fmax, fmax)
    return (float_quantize(t, e_bits, m_bits) * scale).to(x.dtype)
