"""Pins oracle/layer.py (restatement of model_hub/utils.py:4-106) without a GPU."""
import math

import pytest
import torch

from oracle import layer as OL


def _ulp_diff_fraction(a, b):
    """fraction of elements that differ, and the largest difference in units of the 16-bit spacing"""
    a32, b32 = a.float(), b.float()
    diff = (a32 - b32).abs()
    spacing = torch.maximum(a32.abs(), b32.abs()).clamp_min(1e-30) * (2.0 ** -7 if a.dtype == torch.bfloat16 else 2.0 ** -10)
    return float((diff > 0).float().mean()), float((diff / spacing).max())


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_rmsnorm_against_torch_16bit_operators_and_closed_form(dtype):
    g = torch.Generator().manual_seed(1)
    x = (torch.randn(64, 512, generator=g) * 1.7).to(dtype)
    w = (1 + 0.1 * torch.randn(512, generator=g)).to(dtype)
    got = OL.rmsnorm(x, w, 1e-6)
    # the reference's expression (utils.py:17-19) evaluated by torch's own 16-bit CPU operators
    variance = torch.mean(torch.square(x), dim=-1, keepdim=True)
    lib = (x * torch.rsqrt(variance + 1e-6)) * w
    frac, ulps = _ulp_diff_fraction(got, lib)
    assert frac < 0.02 and ulps <= 1.01, (frac, ulps)     # rows whose 16-bit variance or rsqrt rounds the other way
    exact = x.double() / torch.sqrt(x.double().pow(2).mean(-1, keepdim=True) + 1e-6) * w.double()
    rel = float(((got.double() - exact).abs() / exact.abs().clamp_min(1e-3)).max())
    assert rel < (4 * 2.0 ** -8 if dtype == torch.bfloat16 else 4 * 2.0 ** -11)   # four roundings at most
    # scaling x by a power of two leaves the result unchanged while epsilon is negligible (all steps scale exactly)
    assert torch.equal(OL.rmsnorm(x * 4, w, 0.0), OL.rmsnorm(x, w, 0.0))


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_silu_and_mul_against_torch_16bit_operators_and_closed_form(dtype):
    g = torch.Generator().manual_seed(2)
    h = (torch.randn(32, 256, generator=g) * 2.5).to(dtype)
    got = OL.silu_and_mul(h)
    x1, x2 = torch.split(h, 128, dim=-1)
    lib = x2 * (x1 * torch.sigmoid(x1))                   # utils.py:12-13 by torch's 16-bit operators
    assert torch.equal(got, lib)
    exact = x2.double() * (x1.double() * torch.sigmoid(x1.double()))
    tol = 3 * 2.0 ** -8 if dtype == torch.bfloat16 else 3 * 2.0 ** -11
    assert float(((got.double() - exact).abs() / exact.abs().clamp_min(1e-2)).max()) < tol
    zeros = torch.zeros(2, 64, dtype=dtype)
    assert float(OL.silu_and_mul(zeros).abs().sum()) == 0.0


def test_rope_is_a_rotation_of_the_two_halves():
    D, Hq, Hkv, T = 64, 3, 1, 50
    g = torch.Generator().manual_seed(3)
    q = torch.randn(T, Hq * D, generator=g).bfloat16()
    k = torch.randn(T, Hkv * D, generator=g).bfloat16()
    inv = 1.0 / (10000.0 ** (torch.arange(0, D, 2, dtype=torch.float32) / D))
    fr = torch.outer(torch.arange(128, dtype=torch.float32), inv)
    table = torch.cat((fr.cos(), fr.sin()), dim=-1)
    pos = torch.randint(0, 128, (T,), generator=g)
    pos[0] = 0
    qo, ko = OL.rope(pos, q, k, D, table)
    assert qo.shape == q.shape and ko.shape == k.shape
    assert torch.equal(qo[0], q[0]) and torch.equal(ko[0], k[0])              # position 0: cos 1, sin 0
    # against complex multiplication in fp64: (x1 + i x2) * exp(i theta)
    for x, o, H in ((q, qo, Hq), (k, ko, Hkv)):
        xd = x.double().view(T, H, D)
        z = torch.complex(xd[..., :D // 2], xd[..., D // 2:]) * torch.polar(torch.ones(T, 1, D // 2, dtype=torch.float64),
                                                                             fr[pos].double()[:, None, :])
        ref = torch.cat([z.real, z.imag], dim=-1).view(T, H * D)
        assert float((o.double() - ref).abs().max()) < 2.0 ** -7 * float(x.abs().max()) * 1.5
        # a rotation keeps the length of every (x1, x2) pair
        od = o.double().view(T, H, D)
        n0 = xd[..., :D // 2] ** 2 + xd[..., D // 2:] ** 2
        n1 = od[..., :D // 2] ** 2 + od[..., D // 2:] ** 2
        assert bool(((n1 - n0).abs() <= 2.0 ** -6 * n0 + 1e-6).all())   # two 16-bit roundings
    # a swapped sign or swapped table halves fails the complex check above; a wrong position fails this one
    qo2, _ = OL.rope(torch.zeros(T, dtype=torch.long), q, k, D, table)
    assert torch.equal(qo2, q)


def test_yarn_table_properties():
    from longcontext_sqattn_paddle_amd.model_hub.utils import yarn_cos_sin_cache

    D, base, trained = 128, 1000000.0, 32768
    plain = yarn_cos_sin_cache(D, base, trained, 4096, "cpu")
    assert plain.shape == (4096, D) and plain.dtype == torch.float32
    inv = 1.0 / (base ** (torch.arange(0, D, 2, dtype=torch.float32) / D))
    assert torch.allclose(plain[:, :64], torch.outer(torch.arange(4096.0), inv).cos(), atol=1e-6)
    assert torch.allclose(plain[:, :64] ** 2 + plain[:, 64:] ** 2, torch.ones(4096, 64), atol=1e-5)
    long = yarn_cos_sin_cache(D, base, trained, 40000, "cpu")
    factor = 0.1 * math.log(4.0) + 1.0
    assert torch.allclose(long[:, :64] ** 2 + long[:, 64:] ** 2, torch.full((40000, 64), factor ** 2), atol=1e-4)
    # the fastest dimension keeps its frequency, the slowest is slowed down four times
    t = torch.arange(40000.0)
    assert torch.allclose(long[:100, 0], torch.cos(t[:100] * inv[0]) * factor, atol=1e-5)
    assert torch.allclose(long[:, 63], torch.cos(t * inv[63] / 4.0) * factor, atol=1e-4)


def test_linear_closed_forms_and_library_matmul():
    g = torch.Generator().manual_seed(12)
    for dt in (torch.bfloat16, torch.float16):
        x = torch.randn(3, 64, generator=g).to(dt)
        w = (torch.randn(40, 64, generator=g) / 8).to(dt)
        b = torch.randn(40, generator=g).to(dt)
        res = torch.randn(3, 40, generator=g).to(dt)
        # identity weight returns x; with a bias, the 16-bit sum of the two
        eye = torch.eye(64).to(dt)
        assert torch.equal(OL.linear(x, eye), x)
        assert torch.equal(OL.linear(x, eye, x[0]), (x.float() + x[0].float()).to(dt))
        # an all-ones row sums the activations: exact in fp64, rounded once
        ones = torch.ones(2, 64).to(dt)
        assert torch.equal(OL.linear(x, ones)[:, 0], x.double().sum(-1).float().to(dt))
        # the library's matmul (fp32 accumulation in some order): equal up to one 16-bit spacing of the result
        lib = torch.nn.functional.linear(x.float(), w.float(), b.float())
        got = OL.linear(x, w, b)
        spacing = lib.abs().clamp_min(2.0 ** -14) * (2.0 ** -7 if dt == torch.bfloat16 else 2.0 ** -10)
        fp32_noise = (x.float().abs() @ w.float().abs().T + b.float().abs()) * 64 * 2.0 ** -24   # where the sum cancels
        assert bool(((got.float() - lib).abs() <= spacing + fp32_noise).all())
        assert float((got == lib.to(dt)).float().mean()) > 0.97
        # a transposed weight or a dropped bias would not survive this: row i of the weight alone
        for i in (0, 17, 39):
            assert torch.equal(OL.linear(x, w, b)[:, i], OL.linear(x, w[i:i + 1], b[i:i + 1])[:, 0])
        # the residual is a second rounding, not part of the first
        two_step = (res.float() + OL.linear(x, w, b).float()).to(dt)
        assert torch.equal(OL.linear(x, w, b, res), two_step)
        one_step = (x.double() @ w.double().T + b.double() + res.double()).float().to(dt)
        assert not torch.equal(two_step, one_step) or dt == torch.float16
