"""Pins `oracle.plugin.int_prepass` / `key_mean_exact` (restatement of sqattn/attn_replacer.py:334-365 for the
integer quantisers) with hand-derived known answers, an exact rational mean and structural properties."""
from fractions import Fraction

import torch

from oracle import fake_quant as FQ
from oracle import plugin


def _bf(x):
    return torch.tensor(x, dtype=torch.float32).bfloat16()


def test_key_mean_is_the_correctly_rounded_mean():
    g = torch.Generator().manual_seed(5)
    k = (torch.randn(1, 2, 37, 4, generator=g) * 3).bfloat16()   # HND
    got = plugin.key_mean_exact(k)
    for h in range(2):
        for d in range(4):
            exact = sum(Fraction(float(v)) for v in k[0, h, :, d]) / 37
            want = torch.tensor(float(exact), dtype=torch.float64).float().bfloat16()   # fp64 -> fp32 -> bf16
            assert got[0, h, 0, d] == want
    # the library mean agrees up to one bf16 step
    lib = k.mean(dim=2, keepdim=True)
    assert float((got.float() - lib.float()).abs().max()) <= float(got.float().abs().max()) * 2 ** -7


def test_known_answers_centring_per_token_and_per_channel():
    D = 128
    # two tokens, one kv head: channel 0 holds 1 and 3 -> mean 2 -> centred -1, +1; other channels 0
    key = torch.zeros(1, 2, 1, D).bfloat16()
    key[0, 0, 0, 0], key[0, 1, 0, 0] = 1.0, 3.0
    # query row: 1, -2, 0.5 -> absmax 2, scale 2/127: 1/scale = 63.5 -> 64 (half away) -> 64*2/127 = 1.00787 -> bf16 1.0078125
    query = torch.zeros(1, 3, 1, D).bfloat16()
    query[0, 0, 0, :3] = _bf([1.0, -2.0, 0.5])
    # second row: absmax 7 -> the 4-bit scale is exactly 1: 2.5 is a tie and rounds away from zero, -1.25 -> -1, 0.4 -> 0
    query[0, 2, 0, :4] = _bf([7.0, 2.5, -1.25, 0.4])
    # value: heads 0/1 of token 0, channel 0 hold 1 and -4: one scale 4/127 for both heads
    value = torch.zeros(1, 3, 2, D).bfloat16()
    value[0, 0, 0, 0], value[0, 0, 1, 0] = 1.0, -4.0
    key2 = torch.zeros(1, 3, 2, D).bfloat16()
    q8, q4, k8, k4, v8 = plugin.int_prepass(query, key2, value)
    assert q8[0, 0, 0, 0] == _bf(1.0078125) and q8[0, 0, 0, 1] == _bf(-2.0)
    # 0.5/scale = 31.75 -> 32 -> 0.503937 -> bf16 0.50390625
    assert q8[0, 0, 0, 2] == _bf(0.50390625)
    # 4 bit, first row: scale fp32(2/7) is a little above 2/7, so 1/scale = 3.4999998 is NOT a tie: 3 -> 0.857 -> bf16
    # 0.85546875; -2 -> -7 -> -2; 0.5/scale = 1.7499999 -> 2 -> 0.5714 -> bf16 0.5703125
    assert q4[0, 0, 0, 0] == _bf(0.85546875) and q4[0, 0, 0, 1] == _bf(-2.0) and q4[0, 0, 0, 2] == _bf(0.5703125)
    assert q4[0, 2, 0, :4].tolist() == [7.0, 3.0, -1.0, 0.0]
    assert v8[0, 0, 0, 0] == _bf(1.0078125) and v8[0, 0, 1, 0] == _bf(-4.0)   # 1/(4/127) = 31.75 -> 32
    assert float(q8[0, 1].abs().max()) == 0.0   # an all-zero row stays zero (scale clamps at 1e-5/127)
    _, _, k8b, k4b, _ = plugin.int_prepass(query[:, :2], key, value[:, :2, :1])
    assert k8b[0, 0, 0, 0] == _bf(-1.0) and k8b[0, 1, 0, 0] == _bf(1.0) and float(k8b[..., 1:].abs().max()) == 0.0
    assert k4b[0, 0, 0, 0] == _bf(-1.0) and k4b[0, 1, 0, 0] == _bf(1.0)


def test_structure():
    g = torch.Generator().manual_seed(6)
    q = torch.randn(2, 33, 4, 128, generator=g).bfloat16()
    k = torch.randn(2, 33, 2, 128, generator=g).bfloat16()
    v = torch.randn(2, 33, 2, 128, generator=g).bfloat16()
    q8, q4, k8, k4, v8 = plugin.int_prepass(q, k, v)
    # rows are independent: quantising a subset of rows gives the same rows
    q8s = plugin.int_prepass(q[:, 5:9], k[:, 5:9], v[:, 5:9])[0]
    assert torch.equal(q8s, q8[:, 5:9])
    # every 8-bit row holds at most 256 distinct values, every 4-bit row at most 16, and the row maximum survives
    row = q8[1, 7, 2].float()
    assert row.unique().numel() <= 256 and q4[1, 7, 2].float().unique().numel() <= 16
    assert float(row.abs().max()) == float(q[1, 7, 2].float().abs().max())
    # adding a constant per channel to every token of the key changes nothing after centring (up to the dtype's rounding)
    k_shift = (k.float() + 8.0).bfloat16()
    exact_shift = (k_shift.float() - 8.0).bfloat16()   # what survived the shift's own rounding
    a = plugin.int_prepass(q, k_shift, v)[2].float()
    b = plugin.int_prepass(q, exact_shift, v)[2].float()
    assert float((a - b).abs().max()) <= 0.08
    # the value scale is shared by batch and heads: scaling one head changes the other heads' grid
    assert torch.equal(v8, FQ.int_fake_quant(v.permute(0, 2, 1, 3), 8, True, "per_channel").permute(0, 2, 1, 3))
    assert plugin.int_prepass(q, k, v, want_4bit=False)[1] is None


def test_integer_codes_are_what_the_fake_quantiser_dequantises():
    """`int_quant_codes`: whole numbers in [-128, 127], the row's largest element at +-127, and codes * scale rounded to
    the tensor dtype is the fake quantiser's output bit for bit; known answer: (1, -2, 0.5) -> scale 2/127, codes
    (64, -127, 32) (63.5 and 31.75 round half away / to nearest)."""
    g = torch.Generator().manual_seed(8)
    x = (torch.randn(2, 3, 50, 128, generator=g) * torch.logspace(-3, 2, 50)[None, None, :, None]).bfloat16()
    x[0, 0, 7] = 0.0
    codes, scale = FQ.int_quant_codes(x, 8)
    assert torch.equal(codes, codes.round()) and float(codes.min()) >= -128 and float(codes.max()) <= 127
    assert torch.equal(codes.abs().amax(dim=-1)[x.float().abs().amax(dim=-1) >= 1e-5], torch.full((2, 3, 50), 127.0)[x.float().abs().amax(dim=-1) >= 1e-5])
    assert torch.equal((codes * scale).to(x.dtype), FQ.int_fake_quant(x, 8, True, "per_token"))
    assert float(scale[0, 0, 7]) == torch.tensor(1e-5).float() / 127 and not bool(codes[0, 0, 7].any())
    row = torch.zeros(1, 1, 1, 128).bfloat16()
    row[0, 0, 0, :3] = _bf([1.0, -2.0, 0.5])
    c, s = FQ.int_quant_codes(row, 8)
    assert c[0, 0, 0, :3].tolist() == [64.0, -127.0, 32.0] and float(s) == float(torch.tensor(2.0) / 127)


def test_integer_product_closure_against_a_scalar_loop_and_the_fake_quant_closure():
    """`plugin_attention(..., int8_qk=True)`: every score is (sum of code products) x scale_q x scale_k x log2e / sqrt(D),
    checked row by row against a float64 loop over exactly the keys `kv_ranges` lists; and it stays within the size of one
    bf16 rounding per operand of the reference's fake-quantised bf16 product (cosine and a 1 % band)."""
    import math

    from oracle import attention as A

    B, N, Hq, Hkv, D = 1, 200, 4, 2, 128
    g = torch.Generator().manual_seed(21)
    q = torch.randn(B, N, Hq, D, generator=g).bfloat16()
    k = (torch.randn(B, N, Hkv, D, generator=g) + 0.5).bfloat16()
    v = torch.randn(B, N, Hkv, D, generator=g).bfloat16()
    kw = dict(num_kv_groups=2, bit8=0.4, bit4=0.2, sink=64, relative=True)
    got = plugin.plugin_attention(q, k, v, int8_qk=True, **kw).view(B, N, Hq, D)
    ref = plugin.plugin_attention(q, k, v, **kw).view(B, N, Hq, D)
    cos = torch.nn.functional.cosine_similarity(got.double().flatten(), ref.double().flatten(), dim=0)
    assert float(cos) > 0.9999 and float((got.double() - ref.double()).abs().max()) < 0.01 * float(ref.double().abs().max()) + 0.01
    # scalar restatement of a few rows
    kh = plugin.repeat_kv(k, 2)
    kh = kh - plugin.key_mean_exact(kh)
    qh = q.permute(0, 2, 1, 3)
    qc, qs = FQ.int_quant_codes(qh, 8)
    kc, ks = FQ.int_quant_codes(kh, 8)
    v8 = FQ.int_fake_quant(plugin.repeat_kv(v, 2), 8, True, "per_channel").to(torch.float16).double()
    w = A.window_size_relative(0.4, N)
    sm = math.log2(math.e) / math.sqrt(D)
    for h in (0, 3):
        for i in (0, 63, 64, 130, 199):
            qb = i // 64 * 64
            keys = torch.cat([torch.arange(lo, min(hi, i + 1) if masked else hi) for lo, hi, _, masked in A.kv_ranges(qb, qb + 64, sink=64, w8=w, w4=w) if hi > lo])
            dots = (kc[0, h, keys].double() @ qc[0, h, i].double())           # exact integers
            s2 = dots * ks[0, h, keys, 0].double() * float(qs[0, h, i, 0]) * sm
            p = torch.exp2(s2 - s2.max())
            want = (p[:, None] * v8[0, h, keys]).sum(0) / p.sum()
            assert float((got[0, i, h].double() - want).abs().max()) <= 2e-2 * float(want.abs().max()) + 2e-3, (h, i)
