"""GPU parity: prefill kernel (through the C ABI) against the CPU oracle.

Stated tolerances.  Kernel vs the same-algorithm oracle (identical quantisation points; only v_exp_f32 and
fp32 summation order differ): without P quantisation max|d| <= 2e-3 * rms(out) + 2^-11 * max|out| -- the second term
because the kernel rounds p to fp16 relative to a reference point that may trail the row's running maximum by up to
2^8 (the same probability with the same relative rounding error 2^-11 as the reference's, but a dominant key no longer
has p = 1 exactly); with e4m3 P a few
probabilities sit within an ulp of a rounding boundary and flip to the neighbouring e4m3 value, so the
check is cosine >= 0.99999, 99.9 % of elements within 2e-3 * rms and every element within 0.25 * rms.
Kernel vs exact attention: cosine >= 0.999 (the bar of the benchmark configuration).
"""
import math

import pytest
import torch

from oracle import attention as A
from oracle import inputs

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def _cos(a, b):
    a, b = a.double().flatten(), b.double().flatten()
    return float(a @ b / (a.norm() * b.norm()))


def _check(out, ref, quantised, q_tol=2e-3):
    out, ref = out.double().cpu(), ref.double()
    rms = float(ref.pow(2).mean().sqrt())
    d = (out - ref).abs()
    if not quantised:
        assert float(d.max()) <= 2e-3 * rms + 2.0 ** -11 * float(ref.abs().max()), (float(d.max()), rms)
    else:
        assert _cos(out, ref) >= 0.99999
        assert float(torch.quantile(d.flatten()[:: max(1, d.numel() // 1000000)], 0.999)) <= q_tol * rms
        assert float(d.max()) <= 0.25 * rms, (float(d.max()), rms)


def _rand(B, Hq, Hkv, N, D, seed, dtype=torch.bfloat16, scale=1.0):
    g = torch.Generator().manual_seed(seed)
    q = (torch.randn(B, Hq, N, D, generator=g) * scale).to(dtype)
    k = (torch.randn(B, Hkv, N, D, generator=g) * scale).to(dtype)
    v = (torch.randn(B, Hkv, N, D, generator=g) * scale).to(dtype)
    return q, k, v


@pytest.mark.parametrize("B,Hq,Hkv,N", [(1, 4, 2, 512), (2, 14, 2, 700), (1, 2, 1, 64), (1, 3, 3, 1000)])
@pytest.mark.parametrize("mode", [A.P_NONE, A.P_STATIC448, A.P_BLOCK_ABSMAX, 3])
def test_causal_matches_oracle(B, Hq, Hkv, N, mode):
    from longcontext_sqattn_paddle_amd.sqattn.attn_triton import attn_causal

    print(f"case prefill causal B={B} Hq={Hq} Hkv={Hkv} N={N} p_quant={mode}", flush=True)
    q, k, v = _rand(B, Hq, Hkv, N, 128, 100 + N)
    # kernel mode 3 is the static-448 grid with the scale folded into the exponent: same oracle, same tolerance
    ref, lse_ref = A.prefill_blockwise(q, k, v, p_quant=A.P_STATIC448 if mode == 3 else mode, out_dtype=torch.float32)
    out, lse = attn_causal(q.to(DEV), k.to(DEV), v.to(DEV), "HND", torch.float32, return_lse=True, p_quant=mode)
    torch.cuda.synchronize()
    _check(out, ref, mode != A.P_NONE)
    assert torch.allclose(lse.cpu(), lse_ref, atol=2e-4)
    exact, _ = A.exact_attention(q, k, v)
    assert _cos(out.cpu(), exact) >= 0.999


@pytest.mark.parametrize("mode", [4, 5])
@pytest.mark.parametrize("B,Hq,Hkv,N,layout", [(1, 4, 2, 512, "HND"), (2, 14, 2, 700, "NHD"), (1, 7, 1, 2048, "HND")])
def test_fp8_pv_mode_matches_oracle(B, Hq, Hkv, N, layout, mode):
    """Modes 4 and 5 (no reference counterpart): e4m3 P *and* e4m3 V (per batch/kv-head/channel scale) on the fp8
    MFMA; mode 5 adds one power-of-two scale per query row and 64-key tile to P."""
    from longcontext_sqattn_paddle_amd.sqattn.attn_triton import attn_causal

    print(f"case prefill fp8-pv mode={mode} B={B} Hq={Hq} Hkv={Hkv} N={N} {layout}", flush=True)
    q, k, v = inputs.prefill_inputs(B, Hq, Hkv, N, 128, seed=200 + N) if N == 2048 else _rand(B, Hq, Hkv, N, 128, 200 + N)
    ref, lse_ref = A.prefill_blockwise(q, k, v, p_quant=A.P_STATIC448_GRID if mode == 4 else A.P_MX_ROW, v_quant="e4m3_channel",
                                       out_dtype=torch.float32)
    args = [t.to(DEV) for t in (q, k, v)]
    if layout == "NHD":
        args = [t.permute(0, 2, 1, 3).contiguous() for t in args]
    out, lse = attn_causal(*args, layout, torch.float32, return_lse=True, p_quant=mode)
    torch.cuda.synchronize()
    if layout == "NHD":
        out = out.permute(0, 2, 1, 3)
    # 99.9 % of elements within 5e-3 * rms here (2e-3 for the fp16 P.V modes): the fp8 matrix instruction sums its 64
    # products with its own internal alignment, which shows on near-uniform rows of thousands of keys
    _check(out, ref, True, q_tol=5e-3)
    assert torch.allclose(lse.cpu(), lse_ref, atol=2e-4)
    exact, _ = A.exact_attention(q, k, v)
    assert _cos(out.cpu(), exact) >= 0.999   # thin margin by construction: e4m3 on both operands (about 0.9995)


def test_block_scaled_p_keeps_small_probabilities_the_static_scale_flushes():
    """Attention sink: key 0 outscores every other key by about 2^17, so all later tiles hold probabilities near
    2^-17 whose 448-fold lies in the subnormal range of e4m3 (steps of 2^-9) and partly rounds to zero under the
    static scale (modes 3 and 4), although the 8192 of them together carry a few percent of the row.  The per-row
    block scale of mode 5 moves each tile's row sum to [128, 256), i.e. its probabilities back to three mantissa bits."""
    from longcontext_sqattn_paddle_amd.sqattn.attn_triton import attn_causal

    N, D = 8192, 128
    g = torch.Generator().manual_seed(77)
    q = torch.randn(1, 4, N, D, generator=g) * 0.3
    k = torch.randn(1, 2, N, D, generator=g) * 0.3
    v = torch.randn(1, 2, N, D, generator=g)
    q[..., 0] = 4.0
    k[..., 0] *= 0.1
    k[:, :, 0, :] = 0.0
    k[:, :, 0, 0] = 17.0 / (4.0 * 1.44269504 / D ** 0.5)   # score of key 0 in log2 units: 17 above the rest
    v[:, :, 0, :] = 0.0   # the sink carries no value, so the output is made of the small probabilities alone
    q, k, v = q.to(torch.bfloat16), k.to(torch.bfloat16), v.to(torch.bfloat16)
    exact, _ = A.exact_attention(q, k, v)
    errs = {}
    for mode in (3, 4, 5):
        print(f"case prefill sink mode={mode}", flush=True)
        out = attn_causal(q.to(DEV), k.to(DEV), v.to(DEV), "HND", torch.float32, p_quant=mode)
        torch.cuda.synchronize()
        errs[mode] = float((out.cpu().double()[:, :, N // 2:] - exact[:, :, N // 2:]).pow(2).mean().sqrt())
    print("rms error vs exact attention, rows N/2..N:", errs, flush=True)
    assert errs[5] <= 0.5 * errs[4]


@pytest.mark.parametrize("step_up,jump", [(6.0, 40.0), (0.0, 140.0), (3.0, 17.0)])
def test_block_scaled_p_reference_moves_and_overflows(step_up, jump):
    """Mode 5 forms a tile's probabilities against the standing reference point without looking at the scores first.
    Scores that climb by `step_up` (log2) per 64-key tile push the row sums past 2^16 every few tiles (the reference then
    moves up by whole binades, which rescales the tile packed just before as well); one key that leads everything before
    it by `jump` does the same in one step, and by 140 it overflows 2^(s - reference): the tile is formed again from the
    key rows in memory.  Against the oracle's restatement of the same rule, and against exact attention."""
    from longcontext_sqattn_paddle_amd.sqattn.attn_triton import attn_causal

    N, D = 1536, 128
    print(f"case prefill mode 5 reference moves step_up={step_up} jump={jump}", flush=True)
    g = torch.Generator().manual_seed(91)
    q = torch.randn(1, 4, N, D, generator=g) * 0.5
    k = torch.randn(1, 2, N, D, generator=g) * 0.5
    v = torch.randn(1, 2, N, D, generator=g)
    ramp = torch.arange(N, dtype=torch.float32) / 64.0 * step_up
    ramp[700:] += jump          # key 700 sits in the middle of a tile, 1000 on a tile that is a diagonal tile for some rows
    ramp[1000:] += jump / 2
    q[..., 0] = 1.0
    k[:, :, :, 0] = (ramp * (D ** 0.5 / 1.44269504))[None, None]
    q, k, v = q.bfloat16(), k.bfloat16(), v.bfloat16()
    ref, lse_ref = A.prefill_blockwise(q, k, v, p_quant=A.P_MX_ROW, v_quant="e4m3_channel", out_dtype=torch.float32)
    out, lse = attn_causal(q.to(DEV), k.to(DEV), v.to(DEV), "HND", torch.float32, return_lse=True, p_quant=5)
    torch.cuda.synchronize()
    assert bool(torch.isfinite(out).all()) and bool(torch.isfinite(lse).all())
    # The scores here reach 200 and more (log2), so their fp32 rounding (1e-4, and the MFMA adds the products in another
    # order than the oracle) moves a probability by 1e-4 relative -- enough to send one in a thousand across an e4m3
    # rounding boundary, a step of 6 %.  Rows like these hang on a dozen leading keys each, so such a flip shows in the
    # row (up to 0.1 rms) where on random data it disappears: a few percent of the rows differ visibly, none grossly.
    err = (out.cpu().double() - ref.double()).abs()
    rms = float(ref.double().pow(2).mean().sqrt())
    assert float(torch.quantile(err.flatten()[:: 7], 0.90)) <= 5e-3 * rms
    assert float(err.max()) <= 0.25 * rms
    assert _cos(out.cpu(), ref) >= 0.9995
    assert torch.allclose(lse.cpu(), lse_ref, atol=2e-4, rtol=1e-6)       # the log-sum-exp has no quantised quantity in it
    exact, lse_exact = A.exact_attention(q, k, v)
    assert _cos(out.cpu(), exact) >= 0.999
    assert torch.allclose(lse.cpu(), lse_exact.float(), atol=2e-2, rtol=5e-3)


@pytest.mark.parametrize("pattern", ["spikes", "late_giant", "alternating", "edge_spikes", "ramp_down"])
@pytest.mark.parametrize("N,window", [(777, None), (1536, (64, 128, 256)), (2304, (0, 64, 64))])
def test_block_scaled_p_score_patterns_with_and_without_windows(pattern, N, window):
    """Mode 5 on score patterns chosen against its rare paths, full causal and with sink + windows (where a wave leaves
    and re-enters its key range with a tile pending): lone keys 20 to 170 (log2) above the rest, a block of keys 150 above
    everything before it, tiles that alternate between two levels 85 apart, spikes on the last key of a tile and the
    first of the next, scores that fall by 7 per tile.  Same criteria as the test above."""
    from longcontext_sqattn_paddle_amd.sqattn._prefill import run_prefill

    print(f"case prefill mode 5 pattern={pattern} N={N} window={window}", flush=True)
    D = 128
    g = torch.Generator().manual_seed(1001)
    q = torch.randn(1, 4, N, D, generator=g) * 0.5
    k = torch.randn(1, 2, N, D, generator=g) * 0.5
    v = torch.randn(1, 2, N, D, generator=g)
    pos = torch.arange(N, dtype=torch.float32)
    r = torch.zeros(N)
    if pattern == "spikes":
        r[torch.randint(0, N, (6,), generator=g)] = torch.tensor([20.0, 45.0, 90.0, 135.0, 170.0, 60.0])
    elif pattern == "late_giant":
        r[N * 3 // 4:] = 150.0
        r[N // 3: N // 3 + 5] = 30.0
    elif pattern == "alternating":
        r = ((pos // 64) % 2) * 85.0
    elif pattern == "edge_spikes":
        r[63::64] = 90.0
        r[64::128] = 100.0
    else:
        r = -pos / 64.0 * 7.0
    q[..., 0] = 1.0
    k[:, :, :, 0] = (r * (D ** 0.5 / 1.44269504))[None, None]
    q, k, v = q.bfloat16(), k.bfloat16(), v.bfloat16()
    kw = {} if window is None else dict(block_m=64, sink=window[0], w8=[window[1]] * 4, w4=[window[2]] * 4)
    ref, lse_ref = A.prefill_blockwise(q, k, v, p_quant=A.P_MX_ROW, v_quant="e4m3_channel", out_dtype=torch.float32, **kw)
    out, lse = run_prefill(q.to(DEV), k.to(DEV), v.to(DEV), tensor_layout="HND", output_dtype=torch.float32, return_lse=True,
                           p_quant=5, window=kw or None)
    torch.cuda.synchronize()
    assert bool(torch.isfinite(out).all()) and bool(torch.isfinite(lse).all())
    # (a leading probability that lands on the other side of an e4m3 rounding boundary than in the oracle moves a row
    # that hangs on two or three keys by up to 0.06 |v|, which is most of the output's rms here: no bound on single
    # elements, a tight one on their bulk and on the whole)
    err = (out.cpu().double() - ref.double()).abs()
    rms = float(ref.double().pow(2).mean().sqrt())
    assert float(torch.quantile(err.flatten()[:: 3], 0.90)) <= 5e-3 * rms
    assert float(err.max()) <= 1.0 * rms
    assert _cos(out.cpu(), ref) >= 0.9999
    assert torch.allclose(lse.cpu(), lse_ref, atol=3e-4, rtol=2e-6)


def test_nhd_layout_bf16_out_and_gqa_7():
    from longcontext_sqattn_paddle_amd.sqattn.attn_triton import attn_causal

    q, k, v = _rand(1, 28, 4, 384, 128, 7)
    ref, _ = A.prefill_blockwise(q, k, v, p_quant=A.P_STATIC448, out_dtype=torch.float32)
    qn, kn, vn = (t.permute(0, 2, 1, 3).contiguous().to(DEV) for t in (q, k, v))
    out = attn_causal(qn, kn, vn, "NHD", torch.bfloat16, is_P_fp8_quant=True)
    torch.cuda.synchronize()
    assert out.shape == (1, 384, 28, 128) and out.dtype == torch.bfloat16
    o = out.permute(0, 2, 1, 3).float().cpu()
    assert _cos(o, ref) >= 0.9999
    assert float((o - ref).abs().max()) <= 2 ** -7 * float(ref.abs().max()) + 0.25 * float(ref.pow(2).mean().sqrt())


def test_fp16_inputs_and_head_dim_64():
    from longcontext_sqattn_paddle_amd.sqattn.attn_triton import attn_causal

    q, k, v = _rand(1, 4, 2, 320, 64, 9, dtype=torch.float16)
    ref, lse_ref = A.prefill_blockwise(q, k, v, out_dtype=torch.float32)
    out, lse = attn_causal(q.to(DEV), k.to(DEV), v.to(DEV), "HND", torch.float32, return_lse=True)
    torch.cuda.synchronize()
    assert out.shape == (1, 4, 320, 64)
    _check(out, ref, False)
    assert torch.allclose(lse.cpu(), lse_ref, atol=2e-4)


def test_config2_style_inputs_with_k_outliers():
    from longcontext_sqattn_paddle_amd.sqattn.attn_triton import attn_causal

    q, k, v = inputs.prefill_inputs(1, 7, 1, 2048, 128, seed=2)
    ref, _ = A.prefill_blockwise(q, k, v, p_quant=A.P_STATIC448, out_dtype=torch.float32)
    out = attn_causal(q.to(DEV), k.to(DEV), v.to(DEV), "HND", torch.float32, is_P_fp8_quant=True)
    torch.cuda.synchronize()
    _check(out, ref, True)
    exact, _ = A.exact_attention(q, k, v)
    assert _cos(out.cpu(), exact) >= 0.999


def test_chunked_prefill_offset():
    from longcontext_sqattn_paddle_amd.sqattn.attn_triton import attn_causal

    q, k, v = _rand(1, 4, 2, 768, 128, 11)
    ref, lse_ref = A.prefill_blockwise(q, k, v, out_dtype=torch.float32)
    out, lse = attn_causal(q[:, :, 512:].contiguous().to(DEV), k.to(DEV), v.to(DEV), "HND", torch.float32,
                           return_lse=True, q_offset=512)
    torch.cuda.synchronize()
    _check(out, ref[:, :, 512:], False)
    assert torch.allclose(lse.cpu(), lse_ref[:, :, 512:], atol=2e-4)


@pytest.mark.parametrize("sink,r8,r4", [(128, 0.25, 0.25), (256, [0.125, 0.5], [0.5, 0.5]), (0, 0.0, 0.0), (64, 2.0, 2.0)])
def test_relative_window_matches_oracle(sink, r8, r4):
    from longcontext_sqattn_paddle_amd.sqattn.attn_triton_mix_relative import attn_hierarchical_relative_window

    N = 1024
    q, k, v = _rand(1, 2, 1, N, 128, 13)
    l8 = r8 if isinstance(r8, list) else [r8, r8]
    l4 = r4 if isinstance(r4, list) else [r4, r4]
    w8 = [A.window_size_relative(x, N) for x in l8]
    w4 = [A.window_size_relative(x, N) for x in l4]
    ref, lse_ref = A.prefill_blockwise(q, k, v, block_m=64, sink=sink, w8=w8, w4=w4, out_dtype=torch.float32)
    qd, kd, vd = q.to(DEV), k.to(DEV), v.to(DEV)
    out, lse = attn_hierarchical_relative_window(qd, kd, qd, kd, vd, r8, r4, sink, "HND", torch.float32, return_lse=True)
    torch.cuda.synchronize()
    _check(out, ref, False)
    assert torch.allclose(lse.cpu(), lse_ref, atol=2e-4)


@pytest.mark.parametrize("sink,w8,w4,distinct", [(128, 256, 512, True), (64, 128, 128, True), (256, [128, 384], [640, 384], True),
                                                 (128, 256, 512, False), (0, 0, 0, False),
                                                 (64, 192, 320, True), (192, [192, 64], [320, 64], True)])   # multiples of 64 but not of 128: walked as written
def test_absolute_window_matches_oracle(sink, w8, w4, distinct):
    from longcontext_sqattn_paddle_amd.sqattn.attn_triton_mix_bad import attn_hierarchical_window
    from oracle import fake_quant as FQ

    N = 1152
    q, k, v = _rand(1, 2, 1, N, 128, 17)
    q4 = FQ.int_fake_quant(q, 4, True, "per_token") if distinct else q
    k4 = FQ.int_fake_quant(k, 4, True, "per_token") if distinct else k
    l8 = w8 if isinstance(w8, list) else [w8, w8]
    l4 = w4 if isinstance(w4, list) else [w4, w4]
    ref, lse_ref = A.prefill_blockwise(q, k, v, block_m=128, sink=sink, w8=l8, w4=l4, q4=q4, k4=k4, out_dtype=torch.float32)
    qd, kd, vd = q.to(DEV), k.to(DEV), v.to(DEV)
    q4d, k4d = (q4.to(DEV), k4.to(DEV)) if distinct else (qd, kd)
    arg8 = torch.tensor(l8, dtype=torch.int32) if isinstance(w8, list) else w8
    arg4 = torch.tensor(l4, dtype=torch.int32) if isinstance(w4, list) else w4
    out, lse = attn_hierarchical_window(qd, kd, q4d, k4d, vd, arg8, arg4, sink, "HND", torch.float32, return_lse=True)
    torch.cuda.synchronize()
    _check(out, ref, False)
    assert torch.allclose(lse.cpu(), lse_ref, atol=2e-4)


def test_unaligned_window_and_sink_sizes_follow_the_documented_rounding():
    """Sizes the reference's kernel has no defined behaviour for (its block loops promise multiples of the query block):
    windows and the sink are rounded up to the next multiple of 64, and an 8-bit window below
    the query block under a wider 4-bit window is raised to the block (the reference's 4-bit range would read keys behind
    the query rows).  Expected values: the oracle on the sizes written out by hand."""
    from longcontext_sqattn_paddle_amd.sqattn.attn_triton_mix_bad import attn_hierarchical_window
    from longcontext_sqattn_paddle_amd.sqattn.attn_triton_mix_relative import attn_hierarchical_relative_window
    from oracle import fake_quant as FQ

    N = 1152
    q, k, v = _rand(1, 2, 1, N, 128, 19)
    q4, k4 = FQ.int_fake_quant(q, 4, True, "per_token"), FQ.int_fake_quant(k, 4, True, "per_token")
    dev = [t.to(DEV) for t in (q, k, q4, k4, v)]
    # absolute: sink 100 -> 128; windows (1, 1000) -> (64, 1024) -> 8-bit window raised to the 128-row block; (300, 200) -> (320, 256)
    out, lse = attn_hierarchical_window(*dev, torch.tensor([1, 300], dtype=torch.int32), torch.tensor([1000, 200], dtype=torch.int32), 100,
                                        "HND", torch.float32, return_lse=True)
    torch.cuda.synchronize()
    ref, lse_ref = A.prefill_blockwise(q, k, v, block_m=128, sink=128, w8=[128, 320], w4=[1024, 256], q4=q4, k4=k4, out_dtype=torch.float32)
    _check(out, ref, False)
    assert torch.allclose(lse.cpu(), lse_ref, atol=2e-4)
    # relative: ratios (0, 0.3) -> 8-bit window 0 raised to the 64-row query block, 4-bit window ceil128(345) = 384; sink 1 -> 64
    out, lse = attn_hierarchical_relative_window(dev[0], dev[1], dev[0], dev[1], dev[4], 0.0, 0.3, 1, "HND", torch.float32, return_lse=True)
    torch.cuda.synchronize()
    ref, lse_ref = A.prefill_blockwise(q, k, v, block_m=64, sink=64, w8=[64, 64], w4=[384, 384], out_dtype=torch.float32)
    _check(out, ref, False)
    assert torch.allclose(lse.cpu(), lse_ref, atol=2e-4)
    with pytest.raises(ValueError):
        attn_hierarchical_window(*dev, -5, 128, 0)


@pytest.mark.parametrize("mode", [3, 4, 5])
@pytest.mark.parametrize("sink,r8,r4,N", [(128, 0.25, 0.25, 1024), (256, [0.125, 0.5], [0.5, 0.5], 1600), (64, 2.0, 2.0, 777)])
def test_relative_window_quantised_modes(mode, sink, r8, r4, N):
    """The folded-scale e4m3 mode and the two fp8 P.V modes walk the same sink/window/diagonal schedule."""
    from longcontext_sqattn_paddle_amd.sqattn.attn_triton_mix_relative import attn_hierarchical_relative_window

    print(f"case prefill relative window mode={mode} sink={sink} N={N}", flush=True)
    q, k, v = _rand(1, 2, 1, N, 128, 23 + N)
    l8 = r8 if isinstance(r8, list) else [r8, r8]
    l4 = r4 if isinstance(r4, list) else [r4, r4]
    w8 = [A.window_size_relative(x, N) for x in l8]
    w4 = [A.window_size_relative(x, N) for x in l4]
    ref, lse_ref = A.prefill_blockwise(q, k, v, p_quant=A.P_MX_ROW if mode == 5 else A.P_STATIC448_GRID, block_m=64, sink=sink,
                                       w8=w8, w4=w4, out_dtype=torch.float32, v_quant="e4m3_channel" if mode >= 4 else None)
    qd, kd, vd = q.to(DEV), k.to(DEV), v.to(DEV)
    out, lse = attn_hierarchical_relative_window(qd, kd, qd, kd, vd, r8, r4, sink, "HND", torch.float32, return_lse=True,
                                                 p_quant=mode)
    torch.cuda.synchronize()
    _check(out, ref, True, q_tol=5e-3 if mode >= 4 else 2e-3)
    assert torch.allclose(lse.cpu(), lse_ref, atol=2e-4)


@pytest.mark.parametrize("mode", [0, 1, 3, 4, 5])
def test_chunked_prefill_offset_all_modes(mode):
    """8 waves x 32 rows against 2.5K keys with a query offset: every wave runs interior (unmasked) pairs, its own
    diagonal tiles and idle steps."""
    from longcontext_sqattn_paddle_amd.sqattn.attn_triton import attn_causal

    print(f"case prefill chunked mode={mode}", flush=True)
    N, off = 2560, 2048
    q, k, v = _rand(1, 4, 2, N, 128, 31)
    omode = {0: A.P_NONE, 1: A.P_STATIC448, 3: A.P_STATIC448_GRID, 4: A.P_STATIC448_GRID, 5: A.P_MX_ROW}[mode]
    ref, lse_ref = A.prefill_blockwise(q, k, v, p_quant=omode, out_dtype=torch.float32, v_quant="e4m3_channel" if mode >= 4 else None)
    out, lse = attn_causal(q[:, :, off:].contiguous().to(DEV), k.to(DEV), v.to(DEV), "HND", torch.float32,
                           return_lse=True, q_offset=off, p_quant=mode)
    torch.cuda.synchronize()
    # mode 3/4: exp2(x + log2 448) and 448 * exp2(x) differ in the last bits, which moves a probability across an e4m3
    # rounding boundary now and then; with 2K+ keys per row most output elements contain such a flip (each worth
    # about p * 2^-4 * |v|), so the 99.9 % band is a little wider than for short rows
    _check(out, ref[:, :, off:], mode != 0, q_tol={0: 2e-3, 1: 2e-3, 3: 3e-3, 4: 5e-3, 5: 5e-3}[mode])
    assert torch.allclose(lse.cpu(), lse_ref[:, :, off:], atol=2e-4)


def test_prefill_argument_errors():
    from longcontext_sqattn_paddle_amd.sqattn.attn_triton import attn_causal
    from longcontext_sqattn_paddle_amd.sqattn.attn_triton_mix_relative import attn_hierarchical_relative_window

    q = torch.zeros(1, 2, 128, 128, dtype=torch.bfloat16, device=DEV)
    k = torch.zeros(1, 1, 128, 128, dtype=torch.bfloat16, device=DEV)
    with pytest.raises(ValueError):
        attn_causal(q, k, k, "DNH")
    with pytest.raises(ValueError):
        attn_causal(torch.zeros(1, 2, 128, 256, dtype=torch.bfloat16, device=DEV), k, k)
    with pytest.raises(AssertionError):   # qo_len != kv_len (attn_triton.py:272)
        attn_causal(q, k[:, :, :64].contiguous(), k[:, :, :64].contiguous())
    with pytest.raises(AssertionError):   # last dim not contiguous (attn_triton.py:245-247)
        attn_causal(q.transpose(2, 3).contiguous().transpose(2, 3), k, k)
    with pytest.raises(ValueError):       # sink must be a non-negative int (attn_triton_mix_relative.py:367-368)
        attn_hierarchical_relative_window(q, k, q, k, k, 0.1, 0.1, -1)
    with pytest.raises(ValueError):
        attn_hierarchical_relative_window(q, k, q, k, k, 0.1, 0.1, 2.5)
    with pytest.raises(RuntimeError):     # no CPU path
        attn_causal(q.cpu(), k.cpu(), k.cpu())


@pytest.mark.parametrize("mode,peaked", [(0, False), (5, False), (0, True)])
def test_full_size_128k_sampled_rows(mode, peaked):
    """The benchmark shape (1 x 28/4 heads x 131072 x 128): rows sampled over the whole sequence (first row, tile and
    block edges, middle, last) against exact attention of that row on the CPU, plus the base-2 LSE.  Modes 0 (the
    reference's own numerics) and 5 (the benchmark's default) on the benchmark configuration's own inputs, mode 0 also on
    a more peaked distribution."""
    from longcontext_sqattn_paddle_amd.sqattn.attn_triton import attn_causal

    print(f"case prefill 128K sampled rows mode={mode} peaked={peaked}", flush=True)
    N, Hq, Hkv, D = 131072, 28, 4, 128
    if not peaked:  # the benchmark configuration's own generator: N(0,1)/sqrt(128), three key channels per kv head x 8
        q, k, v = (t.to(DEV) for t in inputs.prefill_inputs(1, Hq, Hkv, N, D, seed=2))
    else:           # scores with a spread of a few units instead of a few tenths
        g = torch.Generator(device=DEV).manual_seed(5)
        q = (torch.randn(1, Hq, N, D, device=DEV, generator=g) * 0.7).bfloat16()
        k = (torch.randn(1, Hkv, N, D, device=DEV, generator=g) * 0.7).bfloat16()
        v = torch.randn(1, Hkv, N, D, device=DEV, generator=g).bfloat16()
    out, lse = attn_causal(q, k, v, "HND", torch.float32, return_lse=True, p_quant=mode)
    torch.cuda.synchronize()
    assert bool(torch.isfinite(out).all())
    kc, vc = k.cpu().double(), v.cpu().double()
    rows = [0, 1, 63, 64, 255, 256, 4095, 65535, 65536, 100000, 131071]
    worst = 0.0
    for h in (0, 6, 7, 27):
        kvh = h // (Hq // Hkv)
        for i in rows:
            qi = A.fold_scale(q[:, h:h + 1, i:i + 1].cpu(), D).double()[0, 0, 0]       # carries log2e / sqrt(D)
            s = kc[0, kvh, :i + 1] @ qi
            m = s.max()
            p = torch.exp2(s - m)
            ref = (p[:, None] * vc[0, kvh, :i + 1]).sum(0) / p.sum()
            ref_lse = float(m + torch.log2(p.sum()))
            got = out[0, h, i].cpu().double()
            err = float((got - ref).abs().max())
            # a row that averages thousands of keys of similar weight has an output far below a single value's size:
            # its e4m3 rounding errors are a random sum measured against rms(V) / sqrt(keys), not against the output
            scale = max(float(ref.abs().max()), 3.0 * float(vc[0, kvh].pow(2).mean().sqrt()) / math.sqrt(i + 1)) + (1e-3 if mode == 0 else 0.0)
            worst = max(worst, err / scale)
            # exact mode: fp16 P and V.  Mode 5: e4m3 P (block-scaled) and e4m3 V, whose elements sit within half a
            # spacing (2^-4 relative) of the true value: a row with one key reproduces a quantised V row
            assert err <= (4e-3 if mode == 0 else 8e-2) * scale, (h, i, err, scale)
            assert abs(float(lse[0, h, i]) - ref_lse) <= 2e-3, (h, i, float(lse[0, h, i]), ref_lse)
    print(f"  worst relative row error {worst:.2e}", flush=True)


def test_window_configurations_drawn_at_random():
    """A seeded sweep over what the window entry points take: sequence lengths that are not multiples of the tile, sink
    sizes from none to longer than the sequence, per-head windows from nothing to everything (8-bit wider or narrower than
    4-bit), 1 to 7 q heads per kv head, both layouts, relative and absolute sizes -- each case against the oracle's
    block-wise restatement over `kv_ranges` (2e-3 rms) and its LSE."""
    from longcontext_sqattn_paddle_amd.sqattn.attn_triton_mix_bad import attn_hierarchical_window
    from longcontext_sqattn_paddle_amd.sqattn.attn_triton_mix_relative import attn_hierarchical_relative_window

    rng = torch.Generator().manual_seed(2024)

    def pick(options):
        return options[int(torch.randint(0, len(options), (1,), generator=rng))]

    for case in range(24):
        N = int(torch.randint(65, 2100, (1,), generator=rng))
        group = pick([1, 2, 4, 7])
        Hkv = pick([1, 2])
        Hq = Hkv * group
        sink = pick([0, 64, 128, 256, 512, 4096])
        layout = pick(["HND", "NHD"])
        relative = case % 2 == 0
        q, k, v = _rand(1, Hq, Hkv, N, 128, 1000 + case)
        if relative:
            r8 = [pick([0.0, 0.05, 0.1, 0.25, 0.5, 1.0, 2.0]) for _ in range(Hq)]
            r4 = [pick([0.0, 0.1, 0.3, 0.5, 1.0]) for _ in range(Hq)]
            w8 = [A.window_size_relative(x, N) for x in r8]
            w4 = [A.window_size_relative(x, N) for x in r4]
            # the documented rule for a 4-bit window wider than an 8-bit window below the query block: the 8-bit window is
            # raised to the block (the reference's ranges would read future keys unmasked there)
            w8 = [max(a8, 64) if a4 > a8 else a8 for a8, a4 in zip(w8, w4)]
            block_m = 64
        else:
            w8 = [pick([0, 128, 256, 384, 1024, 4096]) for _ in range(Hq)]
            w4 = [pick([0, 128, 512, 640, 2048]) for _ in range(Hq)]
            w8 = [max(a8, 128) if a4 > a8 else a8 for a8, a4 in zip(w8, w4)]   # (a 4-bit window wider than an 8-bit window below the query block is refused)
            block_m = 128
        print(f"case windows #{case}: N={N} Hq={Hq} Hkv={Hkv} sink={sink} {layout} {'relative' if relative else 'absolute'} w8={w8} w4={w4}", flush=True)
        ref, lse_ref = A.prefill_blockwise(q, k, v, block_m=block_m, sink=sink, w8=w8, w4=w4, out_dtype=torch.float32)
        if layout == "NHD":
            qd, kd, vd = (t.permute(0, 2, 1, 3).contiguous().to(DEV) for t in (q, k, v))
        else:
            qd, kd, vd = q.to(DEV), k.to(DEV), v.to(DEV)
        if relative:
            out, lse = attn_hierarchical_relative_window(qd, kd, qd, kd, vd, r8, r4, sink, layout, torch.float32, return_lse=True)
        else:
            out, lse = attn_hierarchical_window(qd, kd, qd, kd, vd, torch.tensor(w8, dtype=torch.int32), torch.tensor(w4, dtype=torch.int32),
                                                sink, layout, torch.float32, return_lse=True)
        torch.cuda.synchronize()
        if layout == "NHD":
            out = out.permute(0, 2, 1, 3)
        _check(out, ref, False)
        assert torch.allclose(lse.cpu(), lse_ref, atol=2e-4), case


def test_causal_configurations_drawn_at_random():
    """A seeded sweep over the full-causal entry point: P modes 0, 1, 3, 4, 5, lengths that are not multiples of the tile,
    1 to 7 q heads per kv head, batch 1 to 3, both layouts, bf16 and fp16 inputs, head_dim 64 / 96 / 128 (padded by the
    host as the reference pads), chunked calls with a query offset -- each against the oracle's block-wise restatement
    with the tolerances stated at the top (fp8 P.V modes: 99.9 % within 5e-3 rms)."""
    from longcontext_sqattn_paddle_amd.sqattn.attn_triton import attn_causal

    rng = torch.Generator().manual_seed(4242)

    def pick(options):
        return options[int(torch.randint(0, len(options), (1,), generator=rng))]

    for case in range(16):
        mode = [0, 1, 3, 4, 5][case % 5]
        B = pick([1, 1, 2, 3])
        Hkv = pick([1, 2])
        Hq = Hkv * pick([1, 2, 4, 7])
        N = int(torch.randint(33, 1800, (1,), generator=rng))
        D = pick([128, 128, 64, 96])
        dtype = pick([torch.bfloat16, torch.bfloat16, torch.float16])
        layout = pick(["HND", "NHD"])
        off = pick([0, 0, 64 * int(torch.randint(0, max(1, N // 64), (1,), generator=rng))])
        print(f"case causal #{case}: mode={mode} B={B} Hq={Hq} Hkv={Hkv} N={N} D={D} {dtype} {layout} q_offset={off}", flush=True)
        q, k, v = _rand(B, Hq, Hkv, N, D, 3000 + case, dtype=dtype)
        omode = {0: A.P_NONE, 1: A.P_STATIC448, 3: A.P_STATIC448_GRID, 4: A.P_STATIC448_GRID, 5: A.P_MX_ROW}[mode]
        ref, lse_ref = A.prefill_blockwise(q, k, v, p_quant=omode, out_dtype=torch.float32, v_quant="e4m3_channel" if mode >= 4 else None)
        qc = q[:, :, off:].contiguous()
        args = [t.to(DEV) for t in (qc, k, v)]
        if layout == "NHD":
            args = [t.permute(0, 2, 1, 3).contiguous() for t in args]
        out, lse = attn_causal(*args, layout, torch.float32, return_lse=True, p_quant=mode, q_offset=off)
        torch.cuda.synchronize()
        if layout == "NHD":
            out = out.permute(0, 2, 1, 3)
        assert out.shape == (B, Hq, N - off, D)
        _check(out, ref[:, :, off:], mode != 0, q_tol={0: 2e-3, 1: 2e-3, 3: 3e-3, 4: 5e-3, 5: 5e-3}[mode])
        assert torch.allclose(lse.cpu(), lse_ref[:, :, off:], atol=2e-4), case
