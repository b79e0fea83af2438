"""Pins the CPU oracle's attention functions without the reference being runnable:
closed forms, a library cross-check, invariants and an independent scalar brute force."""
import math

import numpy as np
import pytest
import torch

from oracle import attention as A


def _rand(B, Hq, Hkv, Nq, Nk, D, seed, scale=1.0, dtype=torch.bfloat16):
    g = torch.Generator().manual_seed(seed)
    q = (torch.randn(B, Hq, Nq, D, generator=g) * scale).to(dtype)
    k = (torch.randn(B, Hkv, Nk, D, generator=g) * scale).to(dtype)
    v = (torch.randn(B, Hkv, Nk, D, generator=g) * scale).to(dtype)
    return q, k, v


def _cos(a, b):
    a, b = a.double().flatten(), b.double().flatten()
    return float(a @ b / (a.norm() * b.norm()))


def test_exact_attention_matches_torch_sdpa():
    q, k, v = _rand(2, 4, 2, 96, 96, 32, 0)
    out, lse2 = A.exact_attention(q, k, v)
    ref = torch.nn.functional.scaled_dot_product_attention(
        q.double(), k.double().repeat_interleave(2, 1), v.double().repeat_interleave(2, 1), is_causal=True)
    assert torch.allclose(out, ref, rtol=1e-10, atol=1e-12)
    # a transposed GQA mapping (tiled instead of blocked heads) must fail this check
    bad = torch.nn.functional.scaled_dot_product_attention(
        q.double(), k.double().repeat(1, 2, 1, 1), v.double().repeat(1, 2, 1, 1), is_causal=True)
    assert not torch.allclose(out, bad, rtol=1e-3, atol=1e-3)
    # lse2 is base 2 of the natural-scaled scores
    s = (q.double() @ k.double().repeat_interleave(2, 1).transpose(-1, -2)) / math.sqrt(32)
    s = s.masked_fill(torch.triu(torch.ones(96, 96, dtype=torch.bool), 1), float("-inf"))
    assert torch.allclose(lse2, torch.logsumexp(s, -1) / math.log(2), rtol=1e-12)


def test_fold_scale_is_bf16_rounding_of_fp32_product():
    q = torch.tensor([[1.0, 0.3333, -2.5, 7.0]], dtype=torch.bfloat16)
    sm = np.float32(1.0 / 128 ** 0.5 * 1.44269504)
    exp = torch.tensor((q.float().numpy() * sm).astype(np.float32)).to(torch.bfloat16)
    assert torch.equal(A.fold_scale(q, 128), exp)


@pytest.mark.parametrize("scale", [1.0, 1.0 / 128 ** 0.5])
def test_blockwise_no_quant_equals_closed_form(scale):
    q, k, v = _rand(1, 4, 2, 200, 200, 128, 1, scale)
    out, lse = A.prefill_blockwise(q, k, v, out_dtype=torch.float32)
    # closed form on the query that already carries the folded factor: isolates the blockwise algorithm
    ref, lse_ref = A.exact_attention(A.fold_scale(q, 128), k, v, score_scale=math.log(2.0))
    rms = ref.pow(2).mean().sqrt()
    assert float((out.double() - ref).abs().max() / rms) < 4e-3   # fp16 P/V rounding + fp32 sums
    assert torch.allclose(lse.double(), lse_ref, atol=1e-4, rtol=1e-5)
    # against the unfolded closed form the bf16 fold dominates (documented ~4e-2 of rms for N(0,1))
    ref2, _ = A.exact_attention(q, k, v)
    assert _cos(out, ref2) > 0.9999


def test_blockwise_independent_of_row_tile():
    q, k, v = _rand(1, 2, 1, 256, 256, 64, 2)
    for mode in (A.P_NONE, A.P_STATIC448, A.P_BLOCK_ABSMAX):
        o128, l128 = A.prefill_blockwise(q, k, v, p_quant=mode, block_m=128, out_dtype=torch.float32)
        o64, l64 = A.prefill_blockwise(q, k, v, p_quant=mode, block_m=64, out_dtype=torch.float32)
        assert torch.equal(o128, o64) and torch.equal(l128, l64)


def _scalar_fp8_prefill(q, k, v, D):
    """Independent scalar restatement of attn_triton.py:64-86 + :208-213 for ONE head, row by row."""
    f32 = np.float32
    qf = A.fold_scale(q, D).float().numpy()
    kf = k.float().numpy()
    vf = v.to(torch.float16).float().numpy()
    N = qf.shape[0]
    out = np.zeros((N, D), dtype=f32)
    lse = np.zeros(N, dtype=f32)
    grid = torch.arange(256, dtype=torch.uint8).view(torch.float8_e4m3fn).float().numpy()
    grid = np.sort(grid[np.isfinite(grid) & (grid >= 0)])
    for i in range(N):
        m, l, acc = f32(-np.inf), f32(1.0), np.zeros(D, dtype=f32)
        tile0 = (i // 128) * 128
        for j0 in range(0, tile0 + 128, 64):
            if j0 >= N:
                break
            s = np.zeros(64, dtype=f32)
            for c in range(64):
                if j0 + c < N:
                    s[c] = np.dot(qf[i].astype(np.float64), kf[j0 + c].astype(np.float64))
                if j0 >= tile0 and j0 + c > i:
                    s[c] += f32(-1000000.0)
            m_new = max(m, s.max())
            p = np.exp2((s - m_new).astype(np.float64)).astype(f32)
            alpha = f32(np.exp2(np.float64(m - m_new)))
            l = f32(l * alpha + p.sum(dtype=f32))
            acc = acc * alpha
            # e4m3 round-to-nearest-even by search on the value grid, then fp16(x/448)
            x = (p * f32(448.0)).astype(np.float64)
            idx = np.searchsorted(grid, x)
            lo = grid[np.clip(idx - 1, 0, len(grid) - 1)]
            hi = grid[np.clip(idx, 0, len(grid) - 1)]
            pick_hi = (hi - x < x - lo) | ((hi - x == x - lo) & ((np.clip(idx, 0, len(grid) - 1) % 2) == 0))
            p8 = np.where(pick_hi, hi, lo)
            pq = (p8 / 448.0).astype(np.float16).astype(f32)
            for c in range(64):
                if j0 + c < N:
                    acc = acc + pq[c] * vf[j0 + c]
            m = m_new
        out[i] = acc / l
        lse[i] = np.log2(l) + m
    return out, lse


def test_fp8_static_matches_scalar_bruteforce():
    D = 32
    q, k, v = _rand(1, 1, 1, 160, 160, D, 3)
    out, lse = A.prefill_blockwise(q, k, v, p_quant=A.P_STATIC448, out_dtype=torch.float32)
    ref, lse_ref = _scalar_fp8_prefill(q[0, 0], k[0, 0], v[0, 0], D)
    d = np.abs(out[0, 0].numpy() - ref)
    rms = np.sqrt((ref ** 2).mean())
    # fp32 summation order differs (matmul vs sequential); an e4m3 flip would show as ~6e-2*|v|
    assert np.quantile(d, 0.999) < 2e-5 * max(rms, 1.0)
    assert d.max() < 0.05
    assert np.allclose(lse[0, 0].numpy(), lse_ref, atol=2e-5)


def test_fp8_error_levels_against_exact():
    q, k, v = _rand(1, 4, 1, 1024, 1024, 128, 4)
    ref, lse_ref = A.exact_attention(q, k, v)
    rms = float(ref.pow(2).mean().sqrt())
    for mode in (A.P_STATIC448, A.P_BLOCK_ABSMAX):
        out, lse = A.prefill_blockwise(q, k, v, p_quant=mode, out_dtype=torch.float32)
        assert _cos(out, ref) > 0.9995
        mean_rel = float((out.double() - ref).abs().mean()) / rms
        assert 5e-3 < mean_rel < 3e-2  # e4m3 has a 3-bit mantissa: about 1.35e-2 expected
        # the denominator uses the unquantised p, so lse2 is unaffected by the P quantisation
        assert torch.allclose(lse.double(), lse_ref, atol=5e-2)


def test_block_scaled_p_quantiser_properties():
    """`P_MX_ROW` (build-defined, no reference counterpart) pinned by what the definition fixes: the scale 2^k comes from
    the row's sum rs = sum(448 p) = f 2^E (f in [1/2, 1)), k = 8 - E.  Rows whose sum lies in [2/7, 4/7) (rs in [128, 256))
    get scale 1 and equal the static-scale grid; multiplying a row by 2^-j multiplies its result by exactly 2^-j (the scale
    absorbs it) until the clamp at 2^60; every scaled probability stays below 256; every element that is at least 2^-13
    of the row's sum keeps three mantissa bits (relative error <= 2^-4); a zero row stays zero."""
    g = torch.Generator().manual_seed(11)
    p = torch.rand(16, 64, generator=g) + 1e-3
    p = p / p.sum(dim=1, keepdim=True) * torch.linspace(0.29, 0.57, 16)[:, None]      # row sums in [2/7, 4/7)
    assert bool(((p * 448).sum(dim=1) >= 128).all()) and bool(((p * 448).sum(dim=1) < 256).all())
    base = A._quant_p(p, A.P_MX_ROW)
    assert torch.equal(base, A._quant_p(p, A.P_STATIC448_GRID))
    for j in (1, 7, 16, 40, 52):
        assert torch.equal(A._quant_p(p * 2.0 ** -j, A.P_MX_ROW), base * 2.0 ** -j), j
        assert torch.equal(A._quant_p(p * 2.0 ** j, A.P_MX_ROW), base * 2.0 ** j), j       # sums far above 1 as well
    # the exponent itself, at both ends of a binade and at the clamps
    rs = torch.tensor([128.0, 255.99, 256.0, 0.875, 2.0 ** 100, 2.0 ** -70, 0.0])
    assert A.mx_row_exponent(rs).tolist() == [0.0, 0.0, -1.0, 8.0, -93.0, 60.0, 8.0]
    # a lone probability of 2^-9: rs = 0.875, k = 8, scaled value 224 is on the grid and is kept exactly
    one = torch.zeros(1, 64)
    one[0, 0] = 2.0 ** -9
    assert float(A._quant_p(one, A.P_MX_ROW)[0, 0]) == 2.0 ** -9
    # a single dominant probability is scaled to [128, 256): never saturates (e4m3 reaches 448)
    for top in (1.0, 0.57, 3.99, 2.0 ** 15.9):
        row = torch.full((1, 64), 1e-9)
        row[0, 3] = top
        qrow = A._quant_p(row, A.P_MX_ROW)
        assert abs(float(qrow[0, 3]) / top - 1.0) <= 2.0 ** -4
    # beyond the clamp the scale stays 2^60 and small values fall off the grid as under any fixed scale
    tiny = torch.full((1, 64), 2.0 ** -80)
    assert float(A._quant_p(tiny, A.P_MX_ROW).abs().max()) == 0.0
    # precision: elements down to 2^-13 of the row's sum are e4m3 normals
    p2 = torch.rand(32, 64, generator=g) * 2.0 ** -14
    p2[:, 0] = 2.0 ** -14
    q2 = A._quant_p(p2, A.P_MX_ROW)
    big = p2 >= p2.sum(dim=1, keepdim=True) * 2.0 ** -13
    assert float(big.float().mean()) > 0.9
    assert float(((q2 - p2).abs() / p2)[big].max()) <= 2.0 ** -4
    assert float(((A._quant_p(p2, A.P_STATIC448_GRID) - p2).abs() / p2)[big].max()) > 0.2   # what the static scale loses
    assert torch.equal(A._quant_p(torch.zeros(2, 64), A.P_MX_ROW), torch.zeros(2, 64))


def test_block_scaled_p_reference_point_is_lazy_but_the_softmax_is_not():
    """`P_MX_ROW` keeps a row's reference point until the row's sum of a block's probabilities exceeds 2^`MX_LAZY`.  What
    that must not change: the log-sum-exp (no quantised quantity enters it) and the output up to e4m3 noise, also when the
    maxima rise block after block by more than the limit in total and, for some rows, in one step."""
    N, D = 512, 64
    g = torch.Generator().manual_seed(21)
    q = torch.randn(1, 2, N, D, generator=g)
    k = torch.randn(1, 1, N, D, generator=g)
    v = torch.randn(1, 1, N, D, generator=g)
    # scores grow with the key index: about +6 (log2) per 64-key block, and +40 at key 320 for every later row
    ramp = torch.arange(N, dtype=torch.float32) / 64.0 * 6.0
    ramp[320:] += 40.0
    q[..., 0] = 1.0
    k[0, 0, :, 0] = ramp * (D ** 0.5 / 1.44269504)
    q, k, v = q.bfloat16(), k.bfloat16(), v.bfloat16()
    exact, lse_exact = A.exact_attention(q, k, v)
    out, lse = A.prefill_blockwise(q, k, v, p_quant=A.P_MX_ROW, out_dtype=torch.float32)
    eager, lse_eager = A.prefill_blockwise(q, k, v, p_quant=A.P_STATIC448_GRID, out_dtype=torch.float32)
    # (the blockwise path rounds the pre-scaled q to 16 bits like the reference, hence the loose bound against exact)
    assert torch.allclose(lse, lse_exact.float(), atol=1e-2, rtol=5e-3)
    assert torch.allclose(lse, lse_eager, atol=2e-4, rtol=1e-6)
    cos = lambda a, b: float((a.double() * b.double()).sum() / (a.double().norm() * b.double().norm()))
    assert cos(out, exact) >= 0.9995
    # (the static scale with its eager reference represents a row's dominant probability, exactly 1, without error -- 448 is
    # on the grid -- which rows like these, with one leading key each, profit from; the block scale rounds it like any value)
    assert cos(out, exact) >= cos(eager, exact) - 3e-4


def test_window_invariants_and_explicit_mask():
    N, D = 512, 64
    q, k, v = _rand(1, 2, 1, N, N, D, 5)
    full, _ = A.prefill_blockwise(q, k, v, out_dtype=torch.float32, block_m=64)
    big = [N + 256, N + 256]
    w, _ = A.prefill_blockwise(q, k, v, out_dtype=torch.float32, block_m=64, sink=128, w8=big, w4=big)
    assert torch.equal(w, full)  # window >= N  =>  full causal
    # N <= block_m => full causal whatever the windows are
    qs, ks, vs = q[:, :, :64], k[:, :, :64], v[:, :, :64]
    a, _ = A.prefill_blockwise(qs, ks, vs, out_dtype=torch.float32, block_m=128, sink=0, w8=[0, 0], w4=[0, 0])
    b, _ = A.prefill_blockwise(qs, ks, vs, out_dtype=torch.float32, block_m=128)
    assert torch.equal(a, b)
    # general case against the closed form under an explicit mask built from the four ranges
    for bm, sink, w8, w4 in ((64, 128, 128, 256), (128, 64, 128, 128), (64, 0, 0, 0), (128, 256, 256, 384)):
        out, lse = A.prefill_blockwise(q, k, v, out_dtype=torch.float32, block_m=bm, sink=sink,
                                       w8=[w8, w8 + 128], w4=[w4, w4 + 128])
        for h, extra in ((0, 0), (1, 128)):
            mask = A.window_mask(N, N, q_offset=0, block_m=bm, sink=sink, w8=w8 + extra, w4=w4 + extra)
            ref, lse_ref = A.exact_attention(A.fold_scale(q[:, h:h + 1], D), k, v, mask=mask[None, None],
                                             score_scale=math.log(2.0))
            rms = ref.pow(2).mean().sqrt()
            assert float((out[:, h:h + 1].double() - ref).abs().max() / rms) < 5e-3
            assert torch.allclose(lse[:, h:h + 1].double(), lse_ref, atol=1e-4)
    # window 0 => sink + diagonal block only: row 300 (block_m 64) sees [0,128) and [256,300]
    m = A.window_mask(N, N, q_offset=0, block_m=64, sink=128, w8=0, w4=0)
    assert m[300].nonzero().flatten().tolist() == list(range(0, 128)) + list(range(256, 301))


def test_relative_window_size():
    assert A.window_size_relative(0.1, 131072) == 13184      # ceil128(13107)
    assert A.window_size_relative(0.1, 4096) == 512          # ceil128(409)
    assert A.window_size_relative(0.0, 4096) == 0
    assert A.window_size_relative(1.0, 4096) == 4096


def test_chunked_prefill_offset_matches_full():
    N, D = 384, 64
    q, k, v = _rand(1, 2, 2, N, N, D, 6)
    full, lf = A.prefill_blockwise(q, k, v, out_dtype=torch.float32)
    part, lp = A.prefill_blockwise(q[:, :, 256:], k, v, q_offset=256, out_dtype=torch.float32)
    assert torch.equal(part, full[:, :, 256:]) and torch.equal(lp, lf[:, :, 256:])


def test_decode_closed_form_and_split_combine():
    B, Hq, Hkv, L, D = 2, 8, 2, 1000, 64
    g = torch.Generator().manual_seed(7)
    q = torch.randn(B, Hq, 1, D, generator=g).bfloat16()
    k = torch.randn(B, Hkv, L, D, generator=g).bfloat16()
    v = torch.randn(B, Hkv, L, D, generator=g).bfloat16()
    lens = [777, 1000]
    out, lse = A.decode_blockwise(q, k, v, lens)
    ref, lse_ref = A.exact_attention(A.fold_scale(q, D), k, v, causal=False, kv_lens=lens, score_scale=math.log(2.0))
    assert torch.allclose(out.double(), ref[:, :, 0], atol=2e-5, rtol=1e-4)
    assert torch.allclose(lse.double(), lse_ref[:, :, 0], atol=1e-4)
    # split-KV combine identity, with ragged and one empty split for batch 0
    cuts = [(0, 256), (256, 640), (640, 832), (832, 1000)]
    outs, lses = zip(*[A.decode_blockwise(q, k, v, lens, token_range=c) for c in cuts])
    assert torch.isinf(lses[3][0]).all()
    o2, l2 = A.combine_splits(torch.stack(outs), torch.stack(lses))
    assert torch.allclose(o2, out, atol=1e-5, rtol=1e-5) and torch.allclose(l2, lse, atol=1e-5)
    # K mean-centring (attn_triton_decode.py:268-269) leaves the result unchanged
    kc = (k.float() - k.float().mean(dim=2, keepdim=True))
    oc, _ = A.exact_attention(q, kc, v, causal=False, kv_lens=lens)
    o0, _ = A.exact_attention(q, k.float(), v, causal=False, kv_lens=lens)
    assert torch.allclose(oc, o0, atol=1e-9)


# ------------------------------------------------------------------ build-defined fp8 operands (no reference counterpart)
def _e4m3_grid():
    g = torch.arange(256, dtype=torch.uint8).view(torch.float8_e4m3fn).float().numpy().astype(np.float64)
    return np.unique(g[np.isfinite(g) & (g >= 0)])   # -0 and +0 collapse: positions follow the positive encodings


def _e4m3_scalar(x):
    """Round-to-nearest-even onto the e4m3 value grid by search, element by element (no torch cast): an independent
    restatement of the cast the oracle uses.  Even = even position in the sorted grid (positions follow the encodings)."""
    grid = _e4m3_grid()
    x = np.asarray(x, dtype=np.float64)
    out = np.empty_like(x)
    for i, t in np.ndenumerate(x):
        a = min(abs(t), 448.0)
        j = int(np.searchsorted(grid, a))
        if j < len(grid) and grid[j] == a:
            r = a
        else:
            lo, hi = grid[j - 1], grid[min(j, len(grid) - 1)]
            if a - lo < hi - a:
                r = lo
            elif a - lo > hi - a:
                r = hi
            else:
                r = lo if (j - 1) % 2 == 0 else hi
        out[i] = np.copysign(r, t)
    return out


def test_static448_grid_known_answers():
    """`P_STATIC448_GRID` = e4m3(448 p) / 448 in fp32.  Hand-derived on the e4m3 grid (3 mantissa bits: spacing 16 in
    [128, 256), 32 in [256, 448]; subnormal spacing 2^-9 below 2^-6):
      p = 1        -> 448            -> 448
      p = 1/2      -> 224            -> 224
      p = 0.3125   -> 140            -> 144   (128 | 144, nearer 144)
      p = 0.296875 -> 133            -> 128
      p = 0.375    -> 168 = tie of 160 | 176 -> 160 (mantissa 010 is even)
      p = 0.40625  -> 182            -> 176
      p = 0.9      -> 403.2          -> 416   (384 | 416)
      p = 2^-6/448 -> 2^-6 (smallest normal), p = 2^-9/448 -> 2^-9 (smallest subnormal)
      p = 2^-16    -> 7 * 2^-10 = tie of 3 | 4 * 2^-9 -> 4 * 2^-9 (even)
      p = 2^-10/448 -> tie of 0 | 2^-9 -> 0;  p = 1.5 * 2^-10/448 -> 2^-9;  p = 0 -> 0."""
    f = np.float32
    cases = [(1.0, 448.0), (0.5, 224.0), (0.3125, 144.0), (0.296875, 128.0), (0.375, 160.0), (0.40625, 176.0), (0.9, 416.0),
             (2.0 ** -6 / 448, 2.0 ** -6), (2.0 ** -9 / 448, 2.0 ** -9), (2.0 ** -16, 2.0 ** -7), (2.0 ** -10 / 448, 0.0),
             (1.5 * 2.0 ** -10 / 448, 2.0 ** -9), (0.0, 0.0)]
    p = torch.tensor([[c[0] for c in cases] + [0.0] * (64 - len(cases))], dtype=torch.float32)
    # the subnormal cases need p * 448 exact in fp32: p = 2^-k / 448 is not a dyadic number, so check the products first
    prod = (p * 448.0)[0, :len(cases)].double().numpy()
    got = A._quant_p(p, A.P_STATIC448_GRID)[0, :len(cases)].numpy()
    grid_pt = []
    for (pv, want), x, y in zip(cases, prod, got):
        if want in (2.0 ** -6, 2.0 ** -9) or pv in (2.0 ** -10 / 448,):
            # p = 2^-k / 448 is not a dyadic number: the fp32 product may sit an ulp off the intended grid point / tie, and
            # the answer must be the neighbour the product is nearest to, which the scalar search decides
            want = float(_e4m3_scalar(x))
        grid_pt.append(want)
        assert y == f(want) / f(448.0), (pv, x, y, want)
    # and the static mode of the reference is this grid followed by fp16(x / 448) in fp16 arithmetic (attn_triton.py:82)
    ref1 = A._quant_p(p, A.P_STATIC448)[0, :len(cases)]
    want1 = (torch.tensor(grid_pt, dtype=torch.float32).to(torch.float16) / 448).float()
    assert torch.equal(ref1, want1)


def test_static448_grid_matches_scalar_search_on_random_probabilities():
    g = torch.Generator().manual_seed(31)
    p = torch.cat([torch.rand(8, 64, generator=g), torch.rand(8, 64, generator=g) * 2.0 ** -8, torch.rand(8, 64, generator=g) * 2.0 ** -17])
    want = _e4m3_scalar((p * 448.0).double().numpy()) / 448.0
    got = A._quant_p(p, A.P_STATIC448_GRID).double().numpy()
    assert np.array_equal(got, want.astype(np.float32).astype(np.float64))


def test_v_e4m3_channel_scale_rule_and_values():
    """`v_quant="e4m3_channel"` against what its definition fixes: the scale is the power of two with
    224 < amax * s <= 448 per (batch, kv head, channel); the values equal an independent scalar rounding loop;
    |v| >= 2^-6 amax keeps three mantissa bits; a zero channel stays zero without NaN."""
    g = torch.Generator().manual_seed(41)
    v = torch.randn(2, 3, 200, 16, generator=g)
    v[..., 0] *= 1e-3
    v[..., 1] *= 300.0
    v[..., 2] = 0.0
    v[0, 0, :, 3] = 0.0
    v[0, 0, 7, 3] = -448.0            # amax * s == 448 exactly (upper end of the interval)
    v[0, 1, :, 3] = 0.0
    v[0, 1, 9, 3] = 224.0             # amax * s must go to 448, not stay at 224 (lower end is open)
    v[1, 0, :, 4] = torch.linspace(-1, 1, 200) * 2.0 ** -20
    v = v.bfloat16()
    vq, s = A.quant_v_e4m3_channel(v)
    assert vq.shape == v.shape and s.shape == (2, 3, 1, 16)
    amax = v.float().abs().amax(dim=2, keepdim=True)
    nz = amax > 0
    assert torch.equal(torch.exp2(torch.round(torch.log2(s))), s)                          # a power of two
    prod = (amax * s)[nz]
    assert bool(((prod > 224.0) & (prod <= 448.0)).all())
    assert float(s[0, 0, 0, 3]) == 1.0 and float(s[0, 1, 0, 3]) == 2.0
    assert torch.equal(s[~nz], torch.ones_like(s[~nz])) and torch.equal(vq[..., 2], torch.zeros_like(vq[..., 2]))
    assert bool(torch.isfinite(vq).all())
    # values: independent scalar loop over every element
    want = _e4m3_scalar((v.double() * s.double()).numpy()) / s.double().numpy()
    assert np.array_equal(vq.double().numpy(), want)
    # precision where the definition promises it
    big = (v.float().abs() >= 2.0 ** -6 * amax) & nz
    rel = ((vq - v.float()).abs() / v.float().abs())[big]
    assert float(rel.max()) <= 2.0 ** -4
    # scale equivariance: v * 2^j gives exactly vq * 2^j
    for j in (-9, -1, 3, 11):
        vj = (v.float() * 2.0 ** j).bfloat16()
        assert torch.equal(vj.float(), v.float() * 2.0 ** j)   # exact in bf16
        vqj, sj = A.quant_v_e4m3_channel(vj)
        assert torch.equal(vqj, vq * 2.0 ** j) and torch.equal(sj[nz], s[nz] * 2.0 ** -j), j


@pytest.mark.parametrize("mode", [A.P_STATIC448_GRID, A.P_MX_ROW, A.P_NONE])
def test_prefill_with_v_quant_equals_prefill_on_prequantised_v(mode):
    """The V quantisation is a pure pre-processing of V: running the blockwise algorithm with `v_quant` equals running
    it without on a V that an independent scalar loop quantised beforehand (the quantised values have four significant
    bits, so the bf16 tensor and the fp16 operand cast hold them exactly)."""
    q, k, v = _rand(1, 4, 2, 200, 200, 32, 43)
    v = (v.float() * torch.tensor([0.01, 1.0, 50.0, 3.0] * 8)).bfloat16()
    a, la = A.prefill_blockwise(q, k, v, p_quant=mode, v_quant="e4m3_channel", out_dtype=torch.float32)
    amax = v.double().abs().amax(dim=2, keepdim=True).numpy()
    s = 2.0 ** np.floor(np.log2(448.0 / amax))
    vq = torch.tensor(_e4m3_scalar(v.double().numpy() * s) / s).bfloat16()
    b, lb = A.prefill_blockwise(q, k, vq, p_quant=mode, out_dtype=torch.float32)
    assert torch.equal(a, b) and torch.equal(la, lb)


def _scalar_block_absmax_prefill(q, k, v, D):
    """Independent scalar restatement of the block-absmax FP8-P mode for ONE head: per (64 query rows x 64 keys) tile
    the largest probability a of the tile (after each row's running-maximum update) sets the scale 448 / a,
    P8 = e4m3(p * (448 / a)), and the product uses fp16(P8 * (a / 448)) with fp16 V; the denominator sums the
    unquantised p.  Rows are processed in groups of 64, keys in ascending blocks of 64 up to the group's 128-row
    tile end, with the additive -1e6 mask inside the diagonal tile (attn_triton.py:57-77 for the schedule)."""
    f32 = np.float32
    qf = A.fold_scale(q, D).float().numpy()
    kf = k.float().numpy()
    vf = v.to(torch.float16).float().numpy()
    N = qf.shape[0]
    out = np.zeros((N, D), dtype=f32)
    lse = np.zeros(N, dtype=f32)
    for g0 in range(0, N, 64):
        rows = list(range(g0, min(g0 + 64, N)))
        m = {i: f32(-np.inf) for i in rows}
        l = {i: f32(1.0) for i in rows}
        acc = {i: np.zeros(D, dtype=np.float64) for i in rows}
        tile0 = (g0 // 128) * 128
        for j0 in range(0, tile0 + 128, 64):
            if j0 >= N:
                break
            p = {}
            for i in rows:
                s = np.zeros(64, dtype=f32)
                for c in range(64):
                    if j0 + c < N:
                        s[c] = np.dot(qf[i].astype(np.float64), kf[j0 + c].astype(np.float64))
                    if j0 >= tile0 and j0 + c > i:
                        s[c] += f32(-1000000.0)
                m_new = max(m[i], s.max())
                p[i] = np.exp2((s - m_new).astype(np.float64)).astype(f32)
                alpha = f32(np.exp2(np.float64(m[i] - m_new)))
                l[i] = f32(l[i] * alpha + p[i].sum(dtype=f32))
                acc[i] = acc[i] * np.float64(alpha)
                m[i] = m_new
            a = max(float(p[i].max()) for i in rows)
            if a <= 0.0:
                continue
            sc, inv = f32(f32(448.0) / f32(a)), f32(f32(a) / f32(448.0))
            for i in rows:
                p8 = _e4m3_scalar(np.minimum((p[i] * sc).astype(f32), f32(448.0)).astype(np.float64))
                pq = (p8.astype(f32) * inv).astype(np.float16).astype(np.float64)
                for c in range(64):
                    if j0 + c < N:
                        acc[i] = acc[i] + pq[c] * vf[j0 + c]
        for i in rows:
            out[i] = (acc[i] / np.float64(l[i])).astype(f32)
            lse[i] = np.log2(l[i]) + m[i]
    return out, lse


def test_block_absmax_matches_scalar_bruteforce():
    """A wrong group size (per row, per 128 rows), a scale taken before the running-maximum update, or a missing
    fp16 rounding of the dequantised P each move the result by e4m3 steps (~1e-2 of rms) and fail the 2e-5 band."""
    D = 32
    q, k, v = _rand(1, 1, 1, 200, 200, D, 47)
    # make the scale matter: one dominant early key so that later tiles have a << 1 for most row groups
    q[..., 0] = 3.0
    k[0, 0, :, 0] *= 0.1
    k[0, 0, 3, 0] = 9.0       # key 3 leads every row by about 2^7: the tiles behind the first hold a of 2^-7 .. 2^-3
    out, lse = A.prefill_blockwise(q, k, v, p_quant=A.P_BLOCK_ABSMAX, out_dtype=torch.float32)
    ref, lse_ref = _scalar_block_absmax_prefill(q[0, 0], k[0, 0], v[0, 0], D)
    d = np.abs(out[0, 0].numpy() - ref)
    rms = np.sqrt((ref ** 2).mean())
    assert np.quantile(d, 0.999) < 2e-5 * max(rms, 1.0)
    assert d.max() < 0.05
    assert np.allclose(lse[0, 0].numpy(), lse_ref, atol=2e-5)
    # the mode is not the static scale in disguise on this input
    stat, _ = A.prefill_blockwise(q, k, v, p_quant=A.P_STATIC448, out_dtype=torch.float32)
    assert float((stat - out).abs().max()) > 1e-3 * rms
    # and a per-row or per-128-row group would differ
    for gr in (1, 128):
        other, _ = A.prefill_blockwise(q, k, v, p_quant=A.P_BLOCK_ABSMAX, out_dtype=torch.float32, group_rows=gr)
        assert float((other - out).abs().max()) > 1e-3 * rms, gr


# ------------------------------------------------------------------ the last corners: decode fp8-P, the lazy reference point
def _scalar_fp8_decode(q, k, v, L, D):
    """Independent scalar restatement of attn_triton_decode.py:204-241 with the fp8 option (:232-233) for ONE head: the
    64-token blocks in ascending order, running maximum, the denominator summed from the *unquantised* p, then
    p <- fp16(fp16(e4m3(448 p)) / 448) (the e4m3 cast as a search on the value grid) times the fp32 value rows."""
    f32 = np.float32
    qf = A.fold_scale(q, D).float().numpy()
    kf, vf = k.float().numpy(), v.float().numpy()
    m, l, acc = f32(-np.inf), f32(0.0), np.zeros(D, dtype=np.float64)
    for j0 in range(0, L, 64):
        j1 = min(j0 + 64, L)
        s = np.array([np.dot(qf.astype(np.float64), kf[j].astype(np.float64)) for j in range(j0, j1)], dtype=f32)
        m_new = max(m, s.max())
        p = np.exp2((s - m_new).astype(np.float64)).astype(f32)
        alpha = f32(np.exp2(np.float64(m - m_new)))
        l = f32(l * alpha + p.sum(dtype=f32))
        acc = acc * np.float64(alpha)
        p8 = _e4m3_scalar((p * f32(448.0)).astype(np.float64))
        pq = (p8.astype(np.float16) / np.float16(448.0)).astype(np.float16).astype(np.float64)   # fp16 / fp16 -> fp16
        for c, j in enumerate(range(j0, j1)):
            acc = acc + pq[c] * vf[j].astype(np.float64)
        m = m_new
    return (acc / np.float64(l)).astype(f32), f32(np.log2(l) + m)


def test_decode_fp8_p_matches_scalar_bruteforce():
    """`decode_blockwise(p_quant=P_STATIC448)` -- what the GPU decode test with the fp8 option compares against -- pinned
    by the scalar loop above: quantising before the denominator is summed, quantising the accumulated output instead of
    p, or a bf16 instead of an fp16 round trip each move the result by e4m3 steps (1e-2 of rms) or shift the LSE."""
    B, Hq, Hkv, L, D = 2, 4, 2, 333, 32
    g = torch.Generator().manual_seed(61)
    q = torch.randn(B, Hq, 1, D, generator=g).bfloat16()
    k = torch.randn(B, Hkv, L, D, generator=g).bfloat16()
    v = torch.randn(B, Hkv, L, D, generator=g).bfloat16()
    lens = [333, 130]
    out, lse = A.decode_blockwise(q, k, v, lens, p_quant=A.P_STATIC448)
    plain, lse_plain = A.decode_blockwise(q, k, v, lens)
    for b in range(B):
        for h in range(Hq):
            ref, lref = _scalar_fp8_decode(q[b, h, 0], k[b, h // 2], v[b, h // 2], lens[b], D)
            d = np.abs(out[b, h].numpy() - ref)
            assert d.max() < 3e-5 * max(float(np.abs(ref).max()), 1.0), (b, h, d.max())
            assert abs(float(lse[b, h]) - float(lref)) < 2e-5
    assert torch.equal(lse, lse_plain)                                    # the quantisation never enters the LSE
    rms = float(plain.pow(2).mean().sqrt())
    assert 1e-3 * rms < float((out - plain).abs().max()) < 0.2 * rms      # and it is not a no-op


def _scalar_mx_row(scores, vals):
    """Independent per-row scalar restatement of the `P_MX_ROW` state: scores [blocks][64] (fp32, base-2 logits of one
    query row), vals [blocks][64] (one output channel).  Written from the definition, not from the oracle's tensors:
      * reference point r: the first block's maximum;
      * p = 2^(s - r) whatever the scores; the denominator sums p as it is; with rs = sum(448 p) in [2^(E-1), 2^E) the
        block scale is 2^k, k = 8 - E clamped to [-118, 60]; the product uses e4m3(448 p 2^k) / (448 2^k);
      * after a block with rs > 448 2^16, r goes up by n = E - 9 and numerator and denominator are multiplied by 2^-n;
      * a block whose rs is not below 2^120 is formed again with r = the block's maximum, numerator and denominator
        multiplied by 2^(old r - new r) first."""
    f32 = np.float32
    r, num, den = None, 0.0, f32(0.0)
    moves, redone = [], 0

    def form(s, r):
        with np.errstate(over="ignore"):
            p = np.exp2((np.asarray(s, dtype=f32) - r).astype(np.float64)).astype(f32)
            rs = (p * f32(448.0)).sum(dtype=f32)
        return p, rs

    for s, v in zip(scores, vals):
        if r is None:
            r = f32(max(s))
        p, rs = form(s, r)
        if not rs < f32(2.0 ** 120):
            new_r = f32(max(s))
            alpha = f32(np.exp2(np.float64(r) - np.float64(new_r)))
            num, den = num * float(alpha), f32(den * alpha)
            r = new_r
            redone += 1
            p, rs = form(s, r)
        den = f32(den + p.sum(dtype=f32))
        E = int(np.frexp(np.float64(rs))[1]) if rs > 0 else 0
        kk = min(max(8 - E, -118), 60)
        sc = 448.0 * 2.0 ** kk
        pq = _e4m3_scalar((p.astype(np.float64) * sc).astype(np.float32).astype(np.float64)) / sc
        num = num + float(np.dot(pq, np.asarray(v, dtype=np.float64)))
        if rs > f32(448.0 * 2.0 ** 16):
            n = E - 9
            num, den, r = num * 2.0 ** -n, f32(den * f32(2.0 ** -n)), f32(r + f32(n))
            moves.append(n)
    return num / float(den), float(np.log2(np.float64(den)) + np.float64(r)), moves, redone


def test_lazy_reference_point_matches_scalar_row_loop():
    """`_RowState.update` in `P_MX_ROW` against the scalar loop above, on rows in which one key of the third block leads
    everything before it by 15.0 (block sum below 2^16: the reference point stays), by 16.5 and by 40 (it moves up by a
    whole number of binades), and by 140 (2^(s - r) overflows: the block is formed again against its own maximum); one
    more row creeps up by 6 per block (the sum passes 2^16 at the third step)."""
    g = torch.Generator().manual_seed(71)
    blocks, D = 6, 4
    rises = [15.0, 16.5, 40.0, 140.0, None]
    S = torch.randn(len(rises), blocks, 64, generator=g) * 2.0 - 3.0
    for i, rise in enumerate(rises):
        top0 = float(S[i, 0].max())
        if rise is None:
            for b in range(1, blocks):
                S[i, b, 7] = top0 + 6.0 * b
        else:
            S[i, 1:] = torch.minimum(S[i, 1:], torch.tensor(top0 - 0.5))     # nothing else leads the first block
            S[i, 2, 11] = top0 + rise
    V = torch.randn(blocks, 64, D, generator=g).to(torch.float16).float()
    st = A._RowState(len(rises), D)
    for b in range(blocks):
        st.update(S[:, b].contiguous(), V[b], A.P_MX_ROW, 64)
    out, lse = st.finish()
    # n = E - 9 with the block's sum 448 2^rise (1 + small) = 2^(8.807 + rise) in [2^(E-1), 2^E): rise 16.5 -> E = 26, 40 -> E = 49;
    # the creeping row reaches 2^18 in its fourth block (2^6 and 2^12 before): E = 27
    expect = [([], 0), ([17], 0), ([40], 0), ([], 1), ([18], 0)]
    for i, rise in enumerate(rises):
        for d in range(D):
            ref, lref, moves, redone = _scalar_mx_row(S[i].numpy(), V[:, :, d].numpy())
            assert abs(float(out[i, d]) - ref) <= 2e-5 * max(abs(ref), 1.0), (i, d, float(out[i, d]), ref)
        assert abs(float(lse[i]) - lref) <= 2e-5 * max(abs(lref), 1.0)
        assert (moves, redone) == expect[i], (rise, moves, redone)
    # and against the exact softmax of the same scores: the lazily followed reference point changes no value
    for i in range(len(rises)):
        s = S[i].reshape(-1).double()
        w = torch.softmax(s * math.log(2.0), dim=0)
        exact = w @ V.reshape(-1, D).double()
        assert torch.allclose(out[i].double(), exact, atol=3e-2 * float(exact.abs().max()) + 1e-3)
        assert abs(float(lse[i]) - float(torch.logsumexp(s * math.log(2.0), 0) / math.log(2.0))) < 1e-4
    # the row that rose by 15.0 really kept its reference point, the one that overflowed sits on its block maximum
    assert float(st.m[0]) == float(S[0, 0].max()) and float(st.m[3]) == float(S[3, 2, 11])
    assert float(st.m[1]) == float(S[1, 0].max() + 17.0)      # (the sum in fp32, as the state holds it)
