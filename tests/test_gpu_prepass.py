"""GPU parity of `sq_fake_quant_prepass` (through the C ABI) with the oracle's restatement of the operand pre-pass
of sqattn/attn_replacer.py:334-365: bit-exact outputs, both layouts and dtypes, ragged sizes, error paths, and
sampled rows at the benchmark shape."""
import pytest
import torch

from oracle import fake_quant as FQ
from oracle import plugin

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def _inputs(B, N, Hq, Hkv, seed, dtype=torch.bfloat16, outliers=True):
    g = torch.Generator().manual_seed(seed)
    q = torch.randn(B, N, Hq, 128, generator=g)
    k = torch.randn(B, N, Hkv, 128, generator=g) + torch.randn(1, 1, Hkv, 128, generator=g)   # a per-channel offset to centre away
    v = torch.randn(B, N, Hkv, 128, generator=g)
    if outliers:
        k[..., 5] *= 8
        q[:, ::7] = 0   # all-zero rows: the scale clamp
    return q.to(dtype), k.to(dtype), v.to(dtype)


@pytest.mark.parametrize("B,N,Hq,Hkv,dtype,want4", [(1, 257, 4, 1, torch.bfloat16, True), (2, 1000, 8, 2, torch.bfloat16, True),
                                                  (1, 4096, 28, 4, torch.bfloat16, False), (2, 333, 6, 3, torch.float16, True),
                                                  (3, 64, 40, 40, torch.bfloat16, True)])
def test_prepass_is_bit_exact(B, N, Hq, Hkv, dtype, want4):
    from longcontext_sqattn_paddle_amd.sqattn.fake_quant import fused_int_prepass

    print(f"case prepass B={B} N={N} Hq={Hq} Hkv={Hkv} {dtype} want4={want4}", flush=True)
    q, k, v = _inputs(B, N, Hq, Hkv, seed=N, dtype=dtype)
    got = fused_int_prepass(q.to(DEV), k.to(DEV), v.to(DEV), want_4bit=want4, tensor_layout="NHD")
    torch.cuda.synchronize()
    ref = plugin.int_prepass(q, k, v, want_4bit=want4)
    for name, a, b in zip(("q8", "q4", "k8", "k4", "v8"), got, ref):
        if b is None:
            assert a is None
            continue
        assert a.dtype == dtype and a.shape == b.shape
        assert torch.equal(a.cpu(), b), (name, float((a.cpu().float() - b.float()).abs().max()))
        # ... and to the bit, which torch.equal does not see for the sign of zero
        assert torch.equal(a.cpu().contiguous().view(torch.int16), b.contiguous().view(torch.int16)), name


@pytest.mark.parametrize("qk,vq,dtype", [("e4m3", "e4m3", torch.bfloat16), ("e5m2", "int", torch.bfloat16), ("int", "e5m2", torch.float16)])
def test_prepass_float_quantiser_types(qk, vq, dtype):
    """The closure's e4m3 / e5m2 quantisers (sqattn/attn_replacer.py:340-358, float simulation of fake_quant.py:151-204)
    in the fused pre-pass.  Every operation of the simulation is exact in fp32 except `floor(log2(|t| + 1e-30))`, which
    the kernel reads from the exponent field: where a library's fp32 log2 rounds a value a few units in the last place
    below a power of two up to the integer, the two differ by one grid step.  Stated tolerance: at most 1e-4 of the
    elements differ, each by at most one step of its grid (2^-3 relative for e4m3, 2^-2 for e5m2); the integer outputs
    of the same call stay bit-exact."""
    from longcontext_sqattn_paddle_amd.sqattn.fake_quant import fused_int_prepass

    print(f"case prepass float quantisers qk={qk} v={vq} {dtype}", flush=True)
    q, k, v = _inputs(2, 700, 8, 2, seed=5, dtype=dtype)
    got = fused_int_prepass(q.to(DEV), k.to(DEV), v.to(DEV), want_4bit=True, tensor_layout="NHD", qk_qtype=qk, v_qtype=vq)
    torch.cuda.synchronize()
    ref = plugin.int_prepass(q, k, v, want_4bit=True, qk_qtype=qk, v_qtype=vq)
    for name, a, b, qt in zip(("q8", "q4", "k8", "k4", "v8"), got, ref, (qk, "int", qk, "int", vq)):
        a = a.cpu()
        if qt == "int":
            assert torch.equal(a.contiguous().view(torch.int16), b.contiguous().view(torch.int16)), name
            continue
        diff = a != b
        assert float(diff.float().mean()) <= 1e-4, (name, float(diff.float().mean()))
        step = 2.0 ** -3 if qt == "e4m3" else 2.0 ** -2
        rel = (a.float() - b.float()).abs() / b.float().abs().clamp(min=1e-30)
        assert float(rel[diff].max()) <= step * 1.01 if bool(diff.any()) else True, name
    with pytest.raises(ValueError):
        fused_int_prepass(q.to(DEV), k.to(DEV), v.to(DEV), qk_qtype="e3m4")


def test_prepass_hnd_views_and_strides():
    from longcontext_sqattn_paddle_amd.sqattn.fake_quant import fused_int_prepass

    q, k, v = _inputs(2, 300, 4, 2, seed=9)
    ref = plugin.int_prepass(q, k, v)
    # HND tensors that are permuted views of NHD storage (non-compact strides) ...
    got = fused_int_prepass(*(t.to(DEV).permute(0, 2, 1, 3) for t in (q, k, v)), tensor_layout="HND")
    for a, b in zip(got, ref):
        assert torch.equal(a.permute(0, 2, 1, 3).cpu(), b)
    # ... and compact HND tensors
    got = fused_int_prepass(*(t.to(DEV).permute(0, 2, 1, 3).contiguous() for t in (q, k, v)), tensor_layout="HND")
    for a, b in zip(got, ref):
        assert a.is_contiguous() and torch.equal(a.permute(0, 2, 1, 3).cpu(), b)


def test_prepass_benchmark_shape_sampled_rows():
    """128K tokens, 28/4 heads: rows sampled across the tensor must equal the oracle run on the same tokens
    (query rows and value columns are independent of other tokens; the key needs the global mean, checked first)."""
    from longcontext_sqattn_paddle_amd.sqattn.fake_quant import fused_int_prepass

    N = 131072
    g = torch.Generator(device=DEV).manual_seed(3)
    q = torch.randn(1, N, 28, 128, generator=g, device=DEV).bfloat16()
    k = (torch.randn(1, N, 4, 128, generator=g, device=DEV) + 0.5).bfloat16()
    v = torch.randn(1, N, 4, 128, generator=g, device=DEV).bfloat16()
    q8, q4, k8, k4, v8 = fused_int_prepass(q, k, v)
    torch.cuda.synchronize()
    kc_mean = plugin.key_mean_exact(k.cpu().permute(0, 2, 1, 3))          # [1,4,1,128]
    tok = torch.randint(0, N, (512,), generator=torch.Generator().manual_seed(1))
    tok = torch.cat([tok, torch.tensor([0, N - 1])])
    qs, ks, vs = q[:, tok].cpu(), k[:, tok].cpu(), v[:, tok].cpu()
    rq8, rq4, _, _, rv8 = plugin.int_prepass(qs, ks, vs)
    assert torch.equal(q8[:, tok].cpu(), rq8) and torch.equal(q4[:, tok].cpu(), rq4) and torch.equal(v8[:, tok].cpu(), rv8)
    from oracle import fake_quant as FQ
    kc = ks.permute(0, 2, 1, 3) - kc_mean
    assert torch.equal(k8[:, tok].cpu(), FQ.int_fake_quant(kc, 8, True, "per_token").permute(0, 2, 1, 3))
    assert torch.equal(k4[:, tok].cpu(), FQ.int_fake_quant(kc, 4, True, "per_token").permute(0, 2, 1, 3))


def test_prepass_errors():
    from longcontext_sqattn_paddle_amd.sqattn.fake_quant import fused_int_prepass

    q, k, v = (t.to(DEV) for t in _inputs(1, 64, 4, 2, seed=1))
    with pytest.raises(ValueError):
        fused_int_prepass(q, k, v, tensor_layout="XYZ")
    with pytest.raises(ValueError):
        fused_int_prepass(q[..., :64], k[..., :64], v[..., :64])
    with pytest.raises(AssertionError):
        fused_int_prepass(q, k[:, :32], v)            # token counts disagree
    with pytest.raises(ValueError):
        fused_int_prepass(q, k.half(), v)             # mixed dtypes
    with pytest.raises(RuntimeError):
        fused_int_prepass(q.cpu(), k, v)


@pytest.mark.parametrize("layout", ["NHD", "HND"])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_int8qk_prepass_codes_and_scales_are_the_quantisers_factors(layout, dtype):
    """sq_fake_quant_prepass_int8qk: the int8 codes and fp32 scales of the centred key equal the oracle's factors exactly
    (codes * scale rounded to the tensor dtype is the fake-quantised key of the other pre-pass), v8 is unchanged, the query
    is not touched."""
    from longcontext_sqattn_paddle_amd.sqattn.fake_quant import fused_int8qk_prepass, fused_int_prepass

    B, N, Hq, Hkv, D = 2, 333, 8, 2, 128
    g = torch.Generator().manual_seed(17)
    q = torch.randn(B, N, Hq, D, generator=g).to(dtype)
    k = (torch.randn(B, N, Hkv, D, generator=g) * torch.logspace(-4, 1, N)[None, :, None, None] + 0.25).to(dtype)
    v = torch.randn(B, N, Hkv, D, generator=g).to(dtype)
    kh = k.permute(0, 2, 1, 3)
    kc = kh - plugin.key_mean_exact(kh)
    codes_ref, scale_ref = FQ.int_quant_codes(kc, 8)                      # HND
    if layout == "HND":
        qd, kd, vd = (t.permute(0, 2, 1, 3).contiguous().to(DEV) for t in (q, k, v))
    else:
        qd, kd, vd = q.to(DEV), k.to(DEV), v.to(DEV)
    q_before = qd.clone()
    k_codes, k_scale, v8 = fused_int8qk_prepass(qd, kd, vd, layout)
    _, _, k8, _, v8_ref = fused_int_prepass(qd, kd, vd, want_4bit=False, tensor_layout=layout)
    torch.cuda.synchronize()
    assert torch.equal(qd, q_before) and torch.equal(v8, v8_ref)
    got_codes = k_codes.cpu() if layout == "HND" else k_codes.cpu().permute(0, 2, 1, 3)
    assert k_codes.dtype == torch.int8 and torch.equal(got_codes.float(), codes_ref)
    assert k_scale.shape == (B, Hkv, 384) and torch.equal(k_scale.cpu()[:, :, :N], scale_ref[..., 0]) and not bool(k_scale[:, :, N:].any())
    deq = (got_codes.float() * k_scale.cpu()[:, :, :N, None]).to(dtype)
    k8h = k8.cpu() if layout == "HND" else k8.cpu().permute(0, 2, 1, 3)
    assert torch.equal(deq.view(torch.int16), k8h.contiguous().view(torch.int16))
