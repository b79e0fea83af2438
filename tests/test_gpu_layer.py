"""Element-wise layer kernels (RMSNorm, SiLU*mul, RoPE) through the C ABI against oracle/layer.py.

RoPE is bit-exact (separate fp32 products and sums, one rounding).  RMSNorm and SiLU*mul agree bit for bit except
where an fp32 intermediate lies on a rounding boundary of a 16-bit operator result (the GPU's exp/accumulation order
differ from the CPU's in the last fp32 bit): at most one 16-bit spacing, on a stated fraction of the elements."""
import pytest
import torch

from oracle import layer as OL

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def _mismatch(a, b):
    a32, b32 = a.float().cpu(), b.float()
    diff = (a32 - b32).abs()
    spacing = torch.maximum(a32.abs(), b32.abs()).clamp_min(1e-30) * (2.0 ** -7 if b.dtype == torch.bfloat16 else 2.0 ** -10)
    return float((diff > 0).float().mean()), float((diff / spacing).max())


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("rows,dim", [(300, 3584), (17, 4096), (5, 8192), (1000, 128), (3, 8)])
def test_rmsnorm_matches_oracle(dtype, rows, dim):
    from longcontext_sqattn_paddle_amd.model_hub.utils import rmsnorm

    print(f"case rmsnorm {dtype} rows={rows} dim={dim}", flush=True)
    g = torch.Generator().manual_seed(rows + dim)
    x = (torch.randn(rows, dim, generator=g) * 1.3).to(dtype)
    w = (1 + 0.2 * torch.randn(dim, generator=g)).to(dtype)
    ref = OL.rmsnorm(x, w, 1e-6)
    out = rmsnorm(x.to(DEV), w.to(DEV), 1e-6)
    torch.cuda.synchronize()
    frac, ulps = _mismatch(out, ref)
    # a row whose fp32 sum of squares rounds to the neighbouring 16-bit variance shifts by one spacing as a whole
    assert ulps <= 1.01 and frac <= 0.02, (frac, ulps)
    if rows >= 100:
        rows_equal = (out.cpu() == ref).all(dim=-1).float().mean()
        assert float(rows_equal) >= 0.97


def test_rmsnorm_3d_input_and_strided_rows():
    from longcontext_sqattn_paddle_amd.model_hub.utils import rmsnorm

    g = torch.Generator().manual_seed(4)
    big = torch.randn(2, 40, 1024, generator=g).bfloat16()
    w = torch.ones(512, dtype=torch.bfloat16)
    x = big[..., :512]                                   # rows 1024 apart
    ref = OL.rmsnorm(x, w)
    out = rmsnorm(big.to(DEV)[..., :512], w.to(DEV))
    torch.cuda.synchronize()
    assert out.shape == x.shape
    frac, ulps = _mismatch(out, ref)
    assert ulps <= 1.01 and frac <= 0.02


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("rows,inter", [(64, 18944), (3, 8), (1000, 512)])
def test_silu_and_mul_matches_oracle(dtype, rows, inter):
    from longcontext_sqattn_paddle_amd.model_hub.utils import silu_and_mul

    print(f"case silu_and_mul {dtype} rows={rows} I={inter}", flush=True)
    g = torch.Generator().manual_seed(rows + inter)
    h = (torch.randn(rows, 2 * inter, generator=g) * 3.0).to(dtype)
    ref = OL.silu_and_mul(h)
    out = silu_and_mul(h.to(DEV))
    torch.cuda.synchronize()
    assert out.shape == (rows, inter)
    frac, ulps = _mismatch(out, ref)
    assert ulps <= 1.01 and frac <= 2e-3, (frac, ulps)   # sigmoid within an fp32 ulp or two of a 16-bit boundary


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("B,S,Hq,Hkv,D,maxpos", [(1, 700, 28, 4, 128, 4096), (2, 33, 8, 8, 64, 50000), (1, 1, 4, 2, 128, 16)])
def test_rope_is_bit_exact(dtype, B, S, Hq, Hkv, D, maxpos):
    from longcontext_sqattn_paddle_amd.model_hub.utils import apply_rope_with_cos_sin_cache_inplace, yarn_cos_sin_cache

    print(f"case rope {dtype} B={B} S={S} Hq={Hq} Hkv={Hkv} D={D} maxpos={maxpos}", flush=True)
    g = torch.Generator().manual_seed(S + D)
    q = torch.randn(B * S, Hq * D, generator=g).to(dtype)
    k = torch.randn(B * S, Hkv * D, generator=g).to(dtype)
    table = yarn_cos_sin_cache(D, 1000000.0, 32768, maxpos, "cpu")
    pos = torch.randint(0, maxpos, (B, S), generator=g)
    rq, rk = OL.rope(pos, q, k, D, table)
    qd, kd = q.to(DEV), k.to(DEV)
    oq, ok = apply_rope_with_cos_sin_cache_inplace(pos.to(DEV), qd, kd, D, table.to(DEV))
    torch.cuda.synchronize()
    assert oq.shape == (B, S, Hq, D) and ok.shape == (B, S, Hkv, D)
    assert torch.equal(oq.cpu().view(B * S, -1), rq) and torch.equal(ok.cpu().view(B * S, -1), rk)
    # to the bit (torch.equal takes -0.0 for +0.0)
    assert torch.equal(oq.cpu().view(B * S, -1).contiguous().view(torch.int16), rq.contiguous().view(torch.int16))
    assert torch.equal(ok.cpu().view(B * S, -1).contiguous().view(torch.int16), rk.contiguous().view(torch.int16))
    assert torch.equal(qd.cpu(), q) and torch.equal(kd.cpu(), k)              # inputs untouched
    oq32, _ = apply_rope_with_cos_sin_cache_inplace(pos.to(DEV).to(torch.int32), qd, kd, D, table.to(DEV))
    assert torch.equal(oq32, oq)


def test_rope_feeds_the_kv_cache_layout():
    """rope output [B, S, Hkv, D] is what `prefill_update_kv_cache` takes (model_hub/LLM.py:56-66)."""
    from longcontext_sqattn_paddle_amd.cache_hub.flash_attn_cache import flash_attn_cache
    from longcontext_sqattn_paddle_amd.model_hub.utils import apply_rope_with_cos_sin_cache_inplace, yarn_cos_sin_cache

    S, Hq, Hkv, D = 96, 8, 2, 128
    g = torch.Generator().manual_seed(8)
    q = torch.randn(S, Hq * D, generator=g).bfloat16().to(DEV)
    k = torch.randn(S, Hkv * D, generator=g).bfloat16().to(DEV)
    v = torch.randn(1, S, Hkv, D, generator=g).bfloat16().to(DEV)
    table = yarn_cos_sin_cache(D, 1000000.0, 32768, 256, DEV)
    pos = torch.arange(S, device=DEV)[None]
    _, ko = apply_rope_with_cos_sin_cache_inplace(pos, q, k, D, table)
    cache = flash_attn_cache(0, 1, 1, 128, Hkv, Hq, D, torch.bfloat16, {"0": DEV}, 1, 7)
    cache.prefill_update_kv_cache(None, ko, v, 0, 0)
    cache.sync(0, 0)
    torch.cuda.synchronize()
    assert torch.equal(cache.key_cache[0][0, :S], ko[0])


def test_layer_kernel_argument_errors():
    from longcontext_sqattn_paddle_amd.model_hub.utils import rmsnorm, silu_and_mul

    x = torch.zeros(4, 8200, dtype=torch.bfloat16, device=DEV)
    with pytest.raises(ValueError, match="at most"):
        rmsnorm(x, torch.ones(8200, dtype=torch.bfloat16, device=DEV))
    with pytest.raises((ValueError, AssertionError)):
        rmsnorm(x[:, :512], torch.ones(512, dtype=torch.float16, device=DEV))
    with pytest.raises(ValueError, match="multiple of 16"):
        silu_and_mul(torch.zeros(4, 24, dtype=torch.bfloat16, device=DEV))
    with pytest.raises(RuntimeError, match="no CPU path"):
        silu_and_mul(torch.zeros(4, 32, dtype=torch.bfloat16))


# ------------------------------------------------------------------------------------------ decode-step projections
def _linear_case(M, N, K, dtype, seed, bias, residual):
    g = torch.Generator().manual_seed(seed)
    x = torch.randn(M, K, generator=g).to(dtype)
    w = (torch.randn(N, K, generator=g) * K ** -0.5).to(dtype)
    b = torch.randn(N, generator=g).to(dtype) if bias else None
    r = torch.randn(M, N, generator=g).to(dtype) if residual else None
    return x, w, b, r


def _check_linear(out, x, w, b, r):
    """fp32 accumulation over K terms in the kernel's order against the oracle's exact sum: the two round to the
    same 16-bit value except where the exact sum lies within the accumulation error of a rounding boundary, and then
    they are neighbours.  Bound on the fp32 error: K * 2^-24 * sum|x_k w_k| (far above what is observed)."""
    ref = OL.linear(x, w, b, r)
    o, f = out.float().cpu(), ref.float()
    eps = 2.0 ** -8 if x.dtype == torch.bfloat16 else 2.0 ** -11       # half a spacing, relative
    mag = (x.double().abs() @ w.double().abs().T).float() + (b.float().abs() if b is not None else 0)
    spacing = torch.maximum(o.abs(), f.abs()).clamp_min(2.0 ** -14) * 2 * eps
    tol = spacing * 1.01 + mag * x.shape[1] * 2.0 ** -24
    if r is not None:   # a neighbouring 16-bit product moves the sum by the product's spacing, whatever the sum's size
        tol = tol + OL.linear(x, w, b).float().abs().clamp_min(2.0 ** -14) * 2 * eps * 1.01
    assert bool(((o - f).abs() <= tol).all()), float(((o - f).abs() / spacing).max())
    assert float((o == f).float().mean()) >= 0.98


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("M,N,K,bias,residual", [(1, 4608, 3584, True, False), (1, 3584, 3584, False, True),
                                                 (1, 37888, 3584, False, False), (1, 3584, 18944, False, True),
                                                 (2, 1000, 512, True, True), (3, 33, 8, True, False), (4, 777, 4104, False, True),
                                                 (5, 2050, 1024, True, True), (8, 4608, 3584, True, False), (8, 515, 18944, False, True),
                                                 (7, 1, 8, False, False), (1, 40000, 128, True, True)])
def test_linear_rows_matches_oracle(dtype, M, N, K, bias, residual):
    from longcontext_sqattn_paddle_amd.model_hub.utils import linear

    print(f"case linear {dtype} M={M} N={N} K={K} bias={bias} residual={residual}", flush=True)
    x, w, b, r = _linear_case(M, N, K, dtype, 7 * M + N + K, bias, residual)
    out = linear(x.to(DEV), w.to(DEV), b.to(DEV) if bias else None, r.to(DEV) if residual else None, max_rows=8)
    torch.cuda.synchronize()
    assert out.shape == (M, N) and out.dtype == dtype
    _check_linear(out, x, w, b, r)


def test_linear_rows_views_batch_shapes_and_the_gemm_hand_over():
    from longcontext_sqattn_paddle_amd import _native as NV
    from longcontext_sqattn_paddle_amd.model_hub.utils import linear

    g = torch.Generator().manual_seed(2)
    # [batch, 1, hidden] activations as the decode step passes them; the residual keeps that shape
    x = torch.randn(4, 1, 512, generator=g).bfloat16()
    w = (torch.randn(768, 512, generator=g) / 22).bfloat16()
    r = torch.randn(4, 1, 768, generator=g).bfloat16()
    out = linear(x.to(DEV), w.to(DEV), None, r.to(DEV))
    assert out.shape == (4, 1, 768)
    _check_linear(out.view(4, 768), x.view(4, 512), w, None, r.view(4, 768))
    # strided rows of x (columns of a wider tensor) and of the weight (a slice of a fused projection)
    wide = torch.randn(3, 1024, generator=g).bfloat16()
    wfused = (torch.randn(900, 1024, generator=g) / 22).bfloat16()
    out = linear(wide.to(DEV)[:, 256:768], wfused.to(DEV)[100:612, 512:])
    _check_linear(out, wide[:, 256:768], wfused[100:612, 512:], None, None)
    # in place on the residual
    rd = r.to(DEV).clone()
    b = [NV.dl(x.to(DEV).view(4, 512)), NV.dl(w.to(DEV)), NV.dl(rd.view(4, 768))]
    NV.check(NV.lib().sq_linear_rows(NV.ptr(b[0]), NV.ptr(b[1]), None, NV.ptr(b[2]), NV.ptr(b[2]), NV.current_stream(rd.device)))
    torch.cuda.synchronize()
    _check_linear(rd.view(4, 768), x.view(4, 512), w, None, r.view(4, 768))
    # nine rows and more are a GEMM: the wrapper hands them to the BLAS library, the entry point refuses them
    x9 = torch.randn(9, 512, generator=g).bfloat16()
    out9 = linear(x9.to(DEV), w.to(DEV))
    assert float((out9.float().cpu() - OL.linear(x9, w).float()).abs().max()) <= 2.0 ** -6
    o9 = torch.empty(9, 768, dtype=torch.bfloat16, device=DEV)
    b = [NV.dl(x9.to(DEV)), NV.dl(w.to(DEV)), NV.dl(o9)]
    with pytest.raises(ValueError):
        NV.check(NV.lib().sq_linear_rows(NV.ptr(b[0]), NV.ptr(b[1]), None, None, NV.ptr(b[2]), NV.current_stream(o9.device)))
    # mismatched shapes and dtypes
    o4 = torch.empty(4, 768, dtype=torch.bfloat16, device=DEV)
    xd, wd = x.to(DEV).view(4, 512), w.to(DEV)
    for args in [(xd, wd[:, :256].contiguous(), None, None, o4),             # inner dimensions differ
                 (xd, wd, torch.zeros(700, dtype=torch.bfloat16, device=DEV), None, o4),   # bias length
                 (xd, wd, None, o4[:3], o4),                                    # residual rows
                 (xd, wd, None, None, torch.empty(4, 700, dtype=torch.bfloat16, device=DEV))]:
        bb = [NV.dl(t) for t in args]
        with pytest.raises(AssertionError):
            NV.check(NV.lib().sq_linear_rows(*[NV.ptr(t) for t in bb], NV.current_stream(o4.device)))
    bb = [NV.dl(xd), NV.dl(wd.half()), NV.dl(o4)]
    with pytest.raises(ValueError):
        NV.check(NV.lib().sq_linear_rows(NV.ptr(bb[0]), NV.ptr(bb[1]), None, None, NV.ptr(bb[2]), NV.current_stream(o4.device)))
    with pytest.raises(RuntimeError):
        linear(x, w)                                                            # CPU tensors: there is no host path


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("M,I,K,bias", [(1, 18944, 3584, False), (1, 2000, 512, True), (2, 9000, 1024, True), (3, 333, 4104, False),
                                        (4, 8192, 256, True), (8, 515, 2048, False), (5, 1, 8, True), (1, 7, 24, False)])
def test_gated_projection_equals_projection_then_silu_and_mul(dtype, M, I, K, bias):
    """One kernel for gate_up_proj and the activation: the bits of the two separate passes, each of which is checked
    against the oracle above."""
    from longcontext_sqattn_paddle_amd import _native as NV
    from longcontext_sqattn_paddle_amd.model_hub.utils import linear, linear_silu_and_mul, silu_and_mul

    print(f"case gated linear {dtype} M={M} I={I} K={K} bias={bias}", flush=True)
    g = torch.Generator().manual_seed(M + I + K)
    x = torch.randn(M, K, generator=g).to(dtype).to(DEV)
    w = (torch.randn(2 * I, K, generator=g) * 2 * K ** -0.5).to(dtype).to(DEV)
    b = torch.randn(2 * I, generator=g).to(dtype).to(DEV) if bias else None
    fused = linear_silu_and_mul(x, w, b, max_rows=8)
    torch.cuda.synchronize()
    assert fused.shape == (M, I) and fused.dtype == dtype
    if I % 8 == 0:   # (the stand-alone activation pass takes whole 16-byte steps)
        two = silu_and_mul(linear(x, w, b, max_rows=8))
        assert torch.equal(fused.view(torch.int16), two.view(torch.int16))
    ref = OL.silu_and_mul(OL.linear(x.cpu(), w.cpu(), b.cpu() if bias else None))
    assert float((fused.float().cpu() - ref.float()).abs().max()) <= 2.0 ** -6 * max(1.0, float(ref.float().abs().max()))
    # an odd number of weight rows has no two halves; an output of the full width is the plain projection's
    o = torch.empty(M, 2 * I, dtype=dtype, device=DEV)
    bb = [NV.dl(x), NV.dl(w), NV.dl(o)]
    with pytest.raises(AssertionError):
        NV.check(NV.lib().sq_linear_rows_silu_and_mul(NV.ptr(bb[0]), NV.ptr(bb[1]), None, NV.ptr(bb[2]), NV.current_stream(o.device)))
    if I > 1:
        bb = [NV.dl(x), NV.dl(w[:2 * I - 1]), NV.dl(torch.empty(M, I, dtype=dtype, device=DEV))]
        with pytest.raises(AssertionError):
            NV.check(NV.lib().sq_linear_rows_silu_and_mul(NV.ptr(bb[0]), NV.ptr(bb[1]), None, NV.ptr(bb[2]), NV.current_stream(o.device)))
    # more rows than the kernel takes: the wrapper runs the two passes
    if I % 8 == 0:
        x9 = torch.randn(9, K, generator=g).to(dtype).to(DEV)
        assert torch.equal(linear_silu_and_mul(x9, w, b), silu_and_mul(torch.nn.functional.linear(x9, w, b)))


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("M,Hq,Hkv,D,K,bias", [(1, 28, 4, 128, 3584, True), (2, 4, 2, 64, 512, True), (3, 2, 1, 128, 264, False),
                                               (4, 8, 8, 32, 1024, True), (8, 3, 1, 16, 4104, False), (1, 1, 1, 16, 8, True)])
def test_rotary_projection_equals_projection_then_rope(dtype, M, Hq, Hkv, D, K, bias):
    """One kernel for the fused q/k/v projection and the rotary embedding of q and k: the bits of sq_linear_rows
    followed by sq_rope (each checked against the oracle above); v is the plain projection."""
    from longcontext_sqattn_paddle_amd import _native as NV
    from longcontext_sqattn_paddle_amd.model_hub.utils import apply_rope_with_cos_sin_cache_inplace, linear, linear_rope, yarn_cos_sin_cache

    print(f"case rotary linear {dtype} M={M} Hq={Hq} Hkv={Hkv} D={D} K={K} bias={bias}", flush=True)
    g = torch.Generator().manual_seed(M + Hq + D + K)
    n = (Hq + 2 * Hkv) * D
    x = torch.randn(M, 1, K, generator=g).to(dtype).to(DEV)
    w = (torch.randn(n, K, generator=g) * 2 * K ** -0.5).to(dtype).to(DEV)
    b = torch.randn(n, generator=g).to(dtype).to(DEV) if bias else None
    table = yarn_cos_sin_cache(D, 1000000.0, 32768, 5000, DEV)
    pos = torch.randint(0, 5000, (M, 1), generator=g).to(DEV)
    fused = linear_rope(x, w, b, pos, D, (Hq + Hkv) * D, table, max_rows=8)
    plain = linear(x, w, b, max_rows=8).view(M, n)
    q_ref, k_ref = apply_rope_with_cos_sin_cache_inplace(pos, plain[:, :Hq * D], plain[:, Hq * D:(Hq + Hkv) * D], D, table)
    torch.cuda.synchronize()
    assert fused.shape == (M, 1, n) and fused.dtype == dtype
    f = fused.view(M, n)
    assert torch.equal(f[:, :Hq * D].contiguous().view(torch.int16), q_ref.reshape(M, -1).view(torch.int16))
    assert torch.equal(f[:, Hq * D:(Hq + Hkv) * D].contiguous().view(torch.int16), k_ref.reshape(M, -1).view(torch.int16))
    assert torch.equal(f[:, (Hq + Hkv) * D:].contiguous().view(torch.int16), plain[:, (Hq + Hkv) * D:].contiguous().view(torch.int16))
    # int32 positions; nothing rotated = the plain projection
    f32 = linear_rope(x, w, b, pos.to(torch.int32), D, (Hq + Hkv) * D, table, max_rows=8)
    assert torch.equal(f32, fused)
    assert torch.equal(linear_rope(x, w, b, pos, D, 0, table, max_rows=8).view(M, n), plain)
    # more rows than the kernel takes: the two passes
    x9 = torch.randn(9, 1, K, generator=g).to(dtype).to(DEV)
    p9 = torch.randint(0, 5000, (9, 1), generator=g).to(DEV)
    got = linear_rope(x9, w, b, p9, D, (Hq + Hkv) * D, table).view(9, n)
    base = torch.nn.functional.linear(x9, w, b).view(9, n)
    q9, k9 = apply_rope_with_cos_sin_cache_inplace(p9, base[:, :Hq * D], base[:, Hq * D:(Hq + Hkv) * D], D, table)
    assert torch.equal(got[:, :Hq * D], q9.reshape(9, -1)) and torch.equal(got[:, Hq * D:(Hq + Hkv) * D], k9.reshape(9, -1))
    assert torch.equal(got[:, (Hq + Hkv) * D:], base[:, (Hq + Hkv) * D:])
    # argument errors: rotated width not whole heads, wrong number of positions, table of another head_dim
    o = torch.empty(M, n, dtype=dtype, device=DEV)
    x2 = x.view(M, K)
    for args, hd, rf in [((x2, w, b, pos.view(-1), table, o), D, D // 2), ((x2, w, b, pos.view(-1)[:M - 1].contiguous() if M > 1 else torch.zeros(2, dtype=torch.int64, device=DEV), table, o), D, D),
                         ((x2, w, b, pos.view(-1), table[:, :D // 2].contiguous(), o), D, D)]:
        bb = [NV.dl(t) for t in args]
        with pytest.raises(AssertionError):
            NV.check(NV.lib().sq_linear_rows_rope(NV.ptr(bb[0]), NV.ptr(bb[1]), NV.ptr(bb[2]), NV.ptr(bb[3]), NV.ptr(bb[4]), hd, rf, NV.ptr(bb[5]),
                                                  None, None, None, None, NV.current_stream(o.device)))


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("B,Hq,Hkv,D,K,L", [(1, 28, 4, 128, 3584, 300), (3, 4, 2, 64, 512, 40), (4, 2, 1, 16, 264, 9)])
def test_rotary_projection_appends_to_the_kv_cache_like_the_append_pass(dtype, B, Hq, Hkv, D, K, L):
    """With the layer's cache behind it the projection writes the new token's rotated k and its v to row
    valid_length[b] and sets attend_length: the same cache bits as the projection followed by sq_kv_cache_append
    (advance = 0); a full sequence is left alone; valid_length is not touched."""
    from longcontext_sqattn_paddle_amd import _native as NV
    from longcontext_sqattn_paddle_amd.model_hub.utils import linear_rope, yarn_cos_sin_cache

    print(f"case rotary linear + cache {dtype} B={B} Hq={Hq} Hkv={Hkv} D={D} K={K} L={L}", flush=True)
    g = torch.Generator().manual_seed(B + Hq + D + K)
    n = (Hq + 2 * Hkv) * D
    x = torch.randn(B, 1, K, generator=g).to(dtype).to(DEV)
    w = (torch.randn(n, K, generator=g) * 2 * K ** -0.5).to(dtype).to(DEV)
    b = torch.randn(n, generator=g).to(dtype).to(DEV)
    table = yarn_cos_sin_cache(D, 1000000.0, 32768, 5000, DEV)
    pos = torch.randint(0, 5000, (B, 1), generator=g).to(DEV)
    lens = torch.randint(0, L, (B,), generator=g).to(torch.int32)
    if B > 1:
        lens[-1] = L                                     # a full sequence
    base_k = torch.randn(B, L, Hkv, D, generator=g).to(dtype)
    base_v = torch.randn(B, L, Hkv, D, generator=g).to(dtype)

    kc1, vc1, vl1 = base_k.to(DEV), base_v.to(DEV), lens.to(DEV)
    al1 = torch.full((B,), -7, dtype=torch.int32, device=DEV)
    out = linear_rope(x, w, b, pos, D, (Hq + Hkv) * D, table, max_rows=8, cache=(kc1, vc1, vl1, al1))
    assert out is not None
    # the two passes
    kc2, vc2, vl2 = base_k.to(DEV), base_v.to(DEV), lens.to(DEV)
    al2 = torch.full((B,), -7, dtype=torch.int32, device=DEV)
    plain = linear_rope(x, w, b, pos, D, (Hq + Hkv) * D, table, max_rows=8)
    k_new = plain[..., Hq * D:(Hq + Hkv) * D].view(B, 1, Hkv, D)
    v_new = plain[..., (Hq + Hkv) * D:].view(B, 1, Hkv, D)
    bb = [NV.dl(t) for t in (k_new, v_new, kc2, vc2, vl2, al2)]
    NV.check(NV.lib().sq_kv_cache_append(*[NV.ptr(t) for t in bb], 0, NV.current_stream(kc2.device)))
    torch.cuda.synchronize()
    assert torch.equal(out, plain)
    assert torch.equal(kc1.view(torch.int16), kc2.view(torch.int16)) and torch.equal(vc1.view(torch.int16), vc2.view(torch.int16))
    assert torch.equal(al1, al2) and torch.equal(vl1.cpu(), lens) and torch.equal(vl2.cpu(), lens)
    assert not torch.equal(kc1.cpu(), base_k)            # something was written
    if B > 1:
        assert torch.equal(kc1[-1].cpu(), base_k[-1]) and int(al1[-1]) == L
    # caches of another shape, a missing length tensor
    with pytest.raises(AssertionError):
        linear_rope(x, w, b, pos, D, (Hq + Hkv) * D, table, max_rows=8, cache=(kc1[:, :, :, :D // 2].contiguous(), vc1, vl1, al1))
    with pytest.raises(AssertionError):
        linear_rope(x, w, b, pos, D, (Hq + Hkv) * D, table, max_rows=8, cache=(kc1, vc1, vl1[:B - 1] if B > 1 else torch.zeros(2, dtype=torch.int32, device=DEV), al1))
    with pytest.raises(ValueError):
        linear_rope(x, w, b, pos, D, (Hq + Hkv) * D, table, max_rows=8, cache=(kc1, vc1, None, al1))


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("M,N,K", [(1, 4608, 3584), (1, 152064, 3584), (2, 1000, 1024), (3, 520, 4104), (4, 37888, 3584), (1, 24, 8),
                                   (1, 512, 8192), (2, 264, 8192), (4, 64, 5120)])
def test_projections_with_the_norm_in_front_equal_norm_then_projection(dtype, M, N, K):
    """sq_rmsnorm_linear_rows*: the RMS norm of the activation rows inside the projection's pass gives the bits of
    sq_rmsnorm followed by the plain form (each checked against the oracle above), for the plain, the gated and the
    rotary projection, with and without the cache rows."""
    from longcontext_sqattn_paddle_amd.model_hub.utils import linear, linear_rope, linear_silu_and_mul, rmsnorm, yarn_cos_sin_cache

    print(f"case norm + linear {dtype} M={M} N={N} K={K}", flush=True)
    g = torch.Generator().manual_seed(M + N + K)
    x = (torch.randn(M, 1, K, generator=g) * 3.0).to(dtype).to(DEV)
    gamma = (1.0 + 0.2 * torch.randn(K, generator=g)).to(dtype).to(DEV)
    w = (torch.randn(N, K, generator=g) * 2 * K ** -0.5).to(dtype).to(DEV)
    b = torch.randn(N, generator=g).to(dtype).to(DEV)
    res = torch.randn(M, 1, N, generator=g).to(dtype).to(DEV)
    eps = 1e-6
    xn = rmsnorm(x, gamma, eps)
    for bias, residual in ((b, None), (None, res), (b, res)):
        got = linear(x, w, bias, residual, max_rows=4, norm=(gamma, eps), fuse_norm_rows=4)
        want = linear(xn, w, bias, residual, max_rows=4)
        assert torch.equal(got.view(torch.int16), want.view(torch.int16))
    if N % 2 == 0:
        got = linear_silu_and_mul(x, w, b, norm=(gamma, eps), fuse_norm_rows=4)
        want = linear_silu_and_mul(xn, w, b)
        assert got.shape == (M, 1, N // 2) and torch.equal(got.view(torch.int16), want.view(torch.int16))
    D = 8 if N < 512 else 128
    if N % (4 * D) == 0:     # [q (2 heads' worth) | k | v] of equal thirds would not be GQA: q = N/2, k = v = N/4
        Hkv = N // (4 * D)
        rope = N // 2 + Hkv * D
        table = yarn_cos_sin_cache(D, 1000000.0, 32768, 5000, DEV)
        pos = torch.randint(0, 5000, (M, 1), generator=g).to(DEV)
        got = linear_rope(x, w, b, pos, D, rope, table, norm=(gamma, eps), fuse_norm_rows=4)
        want = linear_rope(xn, w, b, pos, D, rope, table)
        assert torch.equal(got.view(torch.int16), want.view(torch.int16))
        L = 12
        lens = torch.randint(0, L, (M,), generator=g).to(torch.int32)
        base_k = torch.randn(M, L, Hkv, D, generator=g).to(dtype)
        base_v = torch.randn(M, L, Hkv, D, generator=g).to(dtype)
        c1 = (base_k.to(DEV), base_v.to(DEV), lens.to(DEV), torch.zeros(M, dtype=torch.int32, device=DEV))
        c2 = (base_k.to(DEV), base_v.to(DEV), lens.to(DEV), torch.zeros(M, dtype=torch.int32, device=DEV))
        got = linear_rope(x, w, b, pos, D, rope, table, cache=c1, norm=(gamma, eps), fuse_norm_rows=4)
        want = linear_rope(xn, w, b, pos, D, rope, table, cache=c2)
        torch.cuda.synchronize()
        assert torch.equal(got, want)
        for t1, t2 in zip(c1, c2):
            assert torch.equal(t1, t2)


def test_norm_in_front_hand_over_and_errors():
    """Rows or row lengths the fused pass does not take go through the two passes with the same result; the C entry
    point itself refuses a row that does not fit its staging buffer, a norm weight of another length or dtype."""
    from longcontext_sqattn_paddle_amd import _native as NV
    from longcontext_sqattn_paddle_amd.model_hub.utils import linear, linear_silu_and_mul, rmsnorm, silu_and_mul

    g = torch.Generator().manual_seed(8)
    dtype = torch.bfloat16
    for M, K in ((4, 8192), (3, 5128), (6, 512), (9, 512)):
        x = torch.randn(M, K, generator=g).to(dtype).to(DEV)
        gamma = (1.0 + 0.2 * torch.randn(K, generator=g)).to(dtype).to(DEV)
        w = (torch.randn(256, K, generator=g) * K ** -0.5).to(dtype).to(DEV)
        xn = rmsnorm(x, gamma, 1e-5)
        assert torch.equal(linear(x, w, max_rows=8, norm=(gamma, 1e-5)), linear(xn, w, max_rows=8))
        assert torch.equal(linear_silu_and_mul(x, w, max_rows=8, norm=(gamma, 1e-5)), linear_silu_and_mul(xn, w, max_rows=8))
    x = torch.randn(4, 8192, generator=g).to(dtype).to(DEV)
    w = torch.randn(64, 8192, generator=g).to(dtype).to(DEV)
    o = torch.empty(4, 64, dtype=dtype, device=DEV)
    good = torch.ones(8192, dtype=dtype, device=DEV)
    for xx, gm in ((x, good),                                    # four rows of 8192 elements do not fit
                   (x[:1], torch.ones(4096, dtype=dtype, device=DEV)),      # wrong length
                   (x[:1], torch.ones(8192, dtype=torch.float16, device=DEV))):   # wrong dtype
        bb = [NV.dl(xx), NV.dl(gm), NV.dl(w), NV.dl(o[:xx.shape[0]])]
        with pytest.raises((AssertionError, NotImplementedError, TypeError, ValueError)):
            NV.check(NV.lib().sq_rmsnorm_linear_rows(NV.ptr(bb[0]), NV.ptr(bb[1]), 1e-6, NV.ptr(bb[2]), None, None, NV.ptr(bb[3]),
                                                     NV.current_stream(o.device)))
    bb = [NV.dl(x[:1]), NV.dl(good), NV.dl(w), NV.dl(o[:1])]
    NV.check(NV.lib().sq_rmsnorm_linear_rows(NV.ptr(bb[0]), NV.ptr(bb[1]), 1e-6, NV.ptr(bb[2]), None, None, NV.ptr(bb[3]), NV.current_stream(o.device)))
    torch.cuda.synchronize()
    assert torch.equal(o[:1], linear(rmsnorm(x[:1], good, 1e-6), w))


def test_mfma_probe_runs_and_checks_its_arguments():
    """sq_probe_mfma_rate (measurement aid, in its own library libsqattn_probe.so): a launch on constant operands returns sums that are exact multiples of the
    products it accumulates, and the argument checks hold."""
    from longcontext_sqattn_paddle_amd import _native as NV

    lib = NV.probe_lib()
    nbytes = int(lib.sq_probe_mfma_operand_bytes())
    assert nbytes == 256 * 512 * 4 * 64 and int(lib.sq_probe_mfma_flops(0, 10)) == 256 * 8 * 10 * 16 * 32768
    assert int(lib.sq_probe_mfma_flops(1, 10)) == 4 * int(lib.sq_probe_mfma_flops(0, 10))
    ones = torch.ones(nbytes // 2, dtype=torch.bfloat16, device=DEV)
    sink = torch.zeros(131072, dtype=torch.float32, device=DEV)
    b = [NV.dl(ones), NV.dl(sink)]
    NV.check(lib.sq_probe_mfma_rate(0, NV.ptr(b[0]), NV.ptr(b[1]), 3, NV.current_stream(sink.device)), lib)
    torch.cuda.synchronize()
    # every MFMA adds 16 products of 1 x 1 to each of a lane's 16 accumulator entries: 3 x 16 MFMAs on 4 accumulators
    assert bool((sink == 3 * 16 * 16 * 16).all())
    e4 = torch.full((nbytes,), 0x38, dtype=torch.uint8, device=DEV)   # e4m3 1.0
    b = [NV.dl(e4), NV.dl(sink)]
    NV.check(lib.sq_probe_mfma_rate(1, NV.ptr(b[0]), NV.ptr(b[1]), 2, NV.current_stream(sink.device)), lib)
    torch.cuda.synchronize()
    assert bool((sink == 2 * 16 * 64 * 16).all())
    for kind, ops, snk, iters in ((2, e4, sink, 1), (0, e4[:1024], sink, 1), (0, e4, sink[:100], 1), (0, e4, sink, 0), (0, e4, sink, (1 << 18) + 1)):
        bb = [NV.dl(ops), NV.dl(snk)]
        with pytest.raises((AssertionError, ValueError)):
            NV.check(lib.sq_probe_mfma_rate(kind, NV.ptr(bb[0]), NV.ptr(bb[1]), iters, NV.current_stream(sink.device)), lib)
