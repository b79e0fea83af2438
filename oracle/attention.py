"""CPU restatement of the reference's prefill / decode attention arithmetic.

TEST INFRASTRUCTURE ONLY (see `oracle/__init__.py`).  torch-CPU tensors in,
torch-CPU tensors out.  Layout is always HND here (`[B, H, N, D]`); callers
permute NHD inputs first.

Followed reference code:
  * `_attn_fwd_inner`, `_attn_fwd`, `attn_causal`          sqattn/attn_triton.py:10-87, 90-213, 216-315
  * `_attn_decode_fwd`, `attn_unified`                     sqattn/attn_triton_decode.py:175-241, 244-361
  * `attn_fwd_inner` + relative wrapper                    sqattn/attn_triton_mix_relative.py:8-99, 309-483
  * `_attn_fwd_inner` + absolute wrapper                   sqattn/attn_triton_mix_bad.py:9-98, 285-426

Build-defined, no reference counterpart (the reference multiplies fp16 P by fp16 V, attn_triton.py:81-83), so no
reference artefact can pin them: P modes `P_BLOCK_ABSMAX`, `P_STATIC448_GRID`, `P_MX_ROW` and `v_quant="e4m3_channel"`.
tests/test_oracle_attention.py pins each against its written definition instead: hand-derived known answers on the e4m3
grid, an independent scalar (grid-search) rounding loop, the exact power-of-two scale rule and its equivariance, and a
scalar row-group brute force for the block-absmax mode.
"""
from __future__ import annotations

import math
from typing import Optional, Sequence

import torch

LOG2E = 1.44269504  # the literal the reference uses (attn_triton.py:250)
BLOCK_N = 64        # KV block of every reference prefill/decode kernel (attn_triton.py:253)
MASK_ADD = -1000000.0  # additive causal mask (attn_triton.py:71)

P_NONE, P_STATIC448, P_BLOCK_ABSMAX, P_STATIC448_GRID = 0, 1, 2, 3
P_MX_ROW = 5   # e4m3 with one power-of-two scale per query row and 64-key tile (block-scaled fp8 MFMA operand)
MX_LAZY = 16.0  # P_MX_ROW: a row's reference point moves only once the row's sum of a block's probabilities exceeds 2^this
MX_REDO = 2.0 ** 120   # P_MX_ROW: a block sum (times 448) at or beyond this, or not a number, has the block formed again


# --------------------------------------------------------------------------- helpers
def softmax_scale_log2(head_dim: int) -> float:
    """`sm_scale = 1/sqrt(D) * 1.44269504` as a Python double (attn_triton.py:249-250)."""
    return 1.0 / head_dim ** 0.5 * LOG2E


def fold_scale(q: torch.Tensor, head_dim: int) -> torch.Tensor:
    """`q = q * sm_scale` in the input dtype (attn_triton.py:251): the product is formed
    in fp32 with the scalar rounded to fp32, then rounded to q's dtype."""
    s = torch.tensor(softmax_scale_log2(head_dim), dtype=torch.float32)
    return (q.float() * s).to(q.dtype)


def exact_attention(q, k, v, *, causal=True, q_offset=0, kv_lens=None, mask=None, score_scale=None):
    """Closed form in fp64: softmax(q k^T / sqrt(D)) v with GQA mapping kv = h // (Hq/Hkv).

    q [B,Hq,Nq,D], k/v [B,Hkv,Nk,D].  Row i sits at absolute position q_offset+i and sees
    keys j <= q_offset+i when `causal`.  `kv_lens[b]` limits the keys of batch b (decode).
    `mask` (bool, broadcastable to [B,Hq,Nq,Nk], True = attend) replaces the causal rule.
    Returns (out fp64, lse2 fp64) with lse2 = log2(sum exp(s)) in base 2 of the *scaled* scores
    (the convention of attn_triton.py:210-213).  `score_scale` overrides 1/sqrt(D) (use ln 2 with a
    query that already carries the folded log2e/sqrt(D) factor).
    """
    B, Hq, Nq, D = q.shape
    Hkv, Nk = k.shape[1], k.shape[2]
    g = Hq // Hkv
    qd, kd, vd = q.double(), k.double(), v.double()
    kd = kd.repeat_interleave(g, dim=1)
    vd = vd.repeat_interleave(g, dim=1)
    s = qd @ kd.transpose(-1, -2) * (1.0 / math.sqrt(D) if score_scale is None else score_scale)
    if mask is None:
        allow = torch.ones(Nq, Nk, dtype=torch.bool)
        if causal:
            allow = torch.arange(Nk)[None, :] <= (q_offset + torch.arange(Nq))[:, None]
        allow = allow[None, None].expand(B, Hq, Nq, Nk).clone()
        if kv_lens is not None:
            lens = torch.as_tensor(kv_lens).view(B, 1, 1, 1)
            allow &= torch.arange(Nk).view(1, 1, 1, Nk) < lens
    else:
        allow = mask.expand(B, Hq, Nq, Nk)
    s = s.masked_fill(~allow, float("-inf"))
    lse = torch.logsumexp(s, dim=-1)
    p = torch.exp(s - lse[..., None])
    out = p @ vd
    return out, lse * math.log2(math.e)


def _quant_p(p: torch.Tensor, mode: int, group_rows: int = 64) -> torch.Tensor:
    """Quantise a block of probabilities `p` [rows, 64] (fp32, values in [0,1]).

    mode 0: `p.to(fp16)`                                          (attn_triton.py:83)
    mode 1: `fp16( fp16(e4m3(p*448)) / 448 )`                     (attn_triton.py:81-82)
    mode 2: per (64-row group x 64-col block) absmax scale a: `e4m3(p*(448/a)) * (a/448)` then fp16
            (build-defined generalisation; a == 1 reproduces mode 1 up to the fp16 divide).
    mode 3: `e4m3(p*448)/448` kept in fp32 (build-defined: P as the fp8 operand of an fp8 P.V product).
    mode 5: as mode 3 with a power-of-two scale per row of the tile (build-defined, see below).
    Returns fp32 values that are exactly representable in fp16.
    """
    if mode == P_NONE:
        return p.to(torch.float16).float()
    if mode == P_STATIC448:
        p8 = (p * 448.0).to(torch.float8_e4m3fn)
        return (p8.to(torch.float16) / 448).float()
    if mode == P_STATIC448_GRID:   # the e4m3 grid of mode 1 without the fp16 rounding of p/448 (fp8 operand of an fp8 MFMA)
        return (p * 448.0).to(torch.float8_e4m3fn).float() / 448.0
    if mode == P_MX_ROW:
        # build-defined: scale 2^k per row of the tile, taken from the row's SUM rs = sum(448 p) (fp32), which the
        # denominator needs anyway: with rs = f 2^E, f in [1/2, 1) (frexp), k = 8 - E clamped to [-118, 60], so that
        # rs 2^k lies in [128, 256): every scaled probability is below 256 (e4m3 reaches 448) and the row's largest one
        # at least 2.  The dequantised value is e4m3(448 p 2^k) / (448 2^k).
        # (p is taken relative to a reference that may trail the row maximum, see _RowState.update.)
        p448 = p * 448.0
        k = mx_row_exponent(p448.sum(dim=1, keepdim=True))
        return (p448 * torch.exp2(k)).to(torch.float8_e4m3fn).float() / (torch.exp2(k) * 448.0)
    if mode == P_BLOCK_ABSMAX:
        out = torch.empty_like(p)
        for r0 in range(0, p.shape[0], group_rows):
            blk = p[r0:r0 + group_rows]
            a = blk.max()
            if float(a) <= 0.0:
                out[r0:r0 + group_rows] = 0.0
                continue
            sc = (torch.tensor(448.0) / a).float()
            inv = (a / torch.tensor(448.0)).float()
            p8 = (blk * sc).clamp(max=448.0).to(torch.float8_e4m3fn)
            out[r0:r0 + group_rows] = (p8.float() * inv).to(torch.float16).float()
        return out
    raise ValueError(f"unknown p_quant mode {mode}")


def mx_row_exponent(rs448: torch.Tensor) -> torch.Tensor:
    """P_MX_ROW: the block scale's exponent k (as fp32) for rows whose probabilities, times 448, sum to `rs448`."""
    e = torch.frexp(rs448.float()).exponent.float()      # rs448 in [2^(e-1), 2^e); 0 for a zero sum
    return (8.0 - e).clamp(-118.0, 60.0)


class _RowState:
    """Online-softmax state of a tile of query rows (attn_triton.py:165-167)."""

    def __init__(self, rows: int, dim: int):
        self.m = torch.full((rows,), float("-inf"), dtype=torch.float32)
        self.l = torch.ones(rows, dtype=torch.float32)
        self.acc = torch.zeros(rows, dim, dtype=torch.float32)

    def update(self, s: torch.Tensor, vblk: torch.Tensor, p_quant: int, group_rows: int):
        """One KV-block step (attn_triton.py:72-84). `s` fp32 [rows, cols], `vblk` fp32 [cols, D]
        holding fp16-representable values."""
        if p_quant == P_MX_ROW:
            return self._update_mx_row(s, vblk)
        m_new = torch.maximum(self.m, s.max(dim=1).values)
        p = torch.exp2(s - m_new[:, None])
        alpha = torch.exp2(self.m - m_new)
        self.l = self.l * alpha + p.sum(dim=1)
        self.acc = self.acc * alpha[:, None]
        pq = _quant_p(p, p_quant, group_rows)
        self.acc = self.acc + pq @ vblk
        self.m = m_new

    def _update_mx_row(self, s: torch.Tensor, vblk: torch.Tensor):
        """Build-defined (no reference counterpart): the reference point m of a row is not its running maximum and no
        maximum is looked at.  The first block sets m to its row maximum.  Afterwards a block's probabilities are formed
        against the standing m, p = 2^(s - m), whatever the scores are (p may exceed 1: the block scale of `_quant_p`
        absorbs any power of two, and l, acc carry the common factor, which cancels in finish()); the block's sum decides
        what follows:
          * rs = sum(448 p) > 448 2^MX_LAZY: after the block has been added, m goes up by the whole number n = E - 9
            (rs in [2^(E-1), 2^E)), l and acc are multiplied by 2^-n (exactly), so that the block's sum becomes [256, 512);
          * rs >= MX_REDO or not a number (a score 2^100 above everything before it): the row takes the block's maximum
            as m first (l and acc rescaled as in the reference's step) and the block is formed again.
        Mathematically the same softmax; the e4m3 grid points differ."""
        blockmax = s.max(dim=1).values
        first = self.m == float("-inf")
        m = torch.where(first, blockmax, self.m)
        rs = (torch.exp2(s - m[:, None]) * 448.0).sum(dim=1)
        redo = ~(rs < MX_REDO)
        m = torch.where(redo, blockmax, m)
        alpha = torch.where(m == self.m, torch.ones_like(m), torch.exp2(self.m - m))
        p = torch.exp2(s - m[:, None])
        rs = (p * 448.0).sum(dim=1)
        self.l = self.l * alpha + p.sum(dim=1)
        self.acc = self.acc * alpha[:, None] + _quant_p(p, P_MX_ROW) @ vblk
        n = torch.where(rs > 448.0 * 2.0 ** MX_LAZY, torch.frexp(rs).exponent.float() - 9.0, torch.zeros_like(rs))
        down = torch.exp2(-n)
        self.l = self.l * down
        self.acc = self.acc * down[:, None]
        self.m = m + n

    def finish(self):
        out = self.acc / self.l[:, None]
        lse = torch.log2(self.l) + self.m
        return out, lse


def quant_v_e4m3_channel(v: torch.Tensor):
    """Build-defined V operand of the fp8 P.V product (no reference counterpart: the reference multiplies fp16 V,
    attn_triton.py:83).  v [B,Hkv,N,D] -> (`e4m3(v * s) / s` as fp32, s [B,Hkv,1,D]) with one power-of-two scale per
    (batch, kv head, channel): `s = 2^floor(log2(448 / amax))`, amax the channel's largest |v| over the tokens, so that
    amax * s lies in (224, 448]; an all-zero channel takes s = 1 and stays zero."""
    amax = v.float().abs().amax(dim=2, keepdim=True)
    _, ex = torch.frexp(torch.where(amax > 0, 448.0 / amax, torch.ones_like(amax)))   # 448/amax = f * 2^ex, f in [1/2, 1)
    sv = torch.ldexp(torch.ones_like(amax), ex - 1)                                    # 2^floor(log2(448/amax))
    return (v.float() * sv).clamp(-448.0, 448.0).to(torch.float8_e4m3fn).float() / sv, sv


def window_size_relative(ratio: float, kv_len: int) -> int:
    """`ceil128(int(float32(ratio) * kv_len))` (attn_triton_mix_relative.py:43-46)."""
    # the product is formed in fp32 on the device: float32(ratio) * float32(kv_len)
    prod = (torch.tensor(ratio, dtype=torch.float32) * torch.tensor(float(kv_len), dtype=torch.float32))
    raw = int(prod.item())  # cast to int64 truncates toward zero
    return (raw + 127) // 128 * 128


def kv_ranges(qs: int, qe: int, *, sink: int, w8: Optional[int], w4: Optional[int]):
    """The ordered KV ranges one query block [qs, qe) visits.

    Full causal (w8 is None): stage 1 `[0, qs)`, stage 2 `[qs, qe)` masked (attn_triton.py:57-63).
    Windowed: sink / 4-bit window / 8-bit window / diagonal
    (attn_triton_mix_relative.py:36-75, attn_triton_mix_bad.py:37-74).
    Returns a list of (lo, hi, use_4bit_operands, causal_masked).
    """
    if w8 is None:
        return [(0, qs, False, False), (qs, qe, False, True)]
    out = [(0, min(sink, qs), False, False)]
    left4 = max(sink, qe - w4)
    left8 = max(sink, qe - w8)
    out.append((left4, left8, True, False) if left4 < left8 else (0, 0, True, False))
    out.append((left8, qs, False, False) if left8 < qs else (0, 0, False, False))
    out.append((qs, qe, False, True))
    return out


def prefill_blockwise(
    q, k, v, *,
    p_quant: int = P_NONE,
    q_offset: int = 0,
    block_m: int = 128,
    sink: int = 0,
    w8: Optional[Sequence[int]] = None,
    w4: Optional[Sequence[int]] = None,
    q4=None, k4=None,
    out_dtype=torch.bfloat16,
    group_rows: int = 64,
    v_quant: Optional[str] = None,
):
    """Blockwise online-softmax prefill exactly in the reference's order of operations.

    q [B,Hq,Nq,D], k,v [B,Hkv,Nk,D] in bf16/fp16.  Query row i has absolute position q_offset+i
    (the reference only has q_offset == 0 and Nq == Nk, attn_triton.py:272).  `block_m` is the
    query tile whose [qs,qe) defines the KV ranges (128 full-causal/absolute, 64 relative).
    `w8`/`w4` = per-head window sizes in tokens (None = full causal).  `q4`/`k4` are the 4-bit
    fake-quantised operands used in the 4-bit window (default: alias of q/k, which is what the
    relative wrapper passes, attn_triton_mix_relative.py:441-444).
    `v_quant="e4m3_channel"` (build-defined, for the fp8 P.V product): V is replaced by
    `e4m3(v * s_d) / s_d` with the power-of-two scale `s_d = 2^floor(log2(448 / max_n |v[b, kvh, n, d]|))` per
    (batch, kv head, channel).
    Returns (out [B,Hq,Nq,D] out_dtype, lse2 [B,Hq,Nq] fp32).
    """
    B, Hq, Nq, D = q.shape
    Hkv, Nk = k.shape[1], k.shape[2]
    g = Hq // Hkv
    qf = fold_scale(q, D).float()
    q4f = fold_scale(q4, D).float() if q4 is not None else qf
    kf = k.float()
    k4f = k4.float() if k4 is not None else kf
    if v_quant is None:
        vf = v.to(torch.float16).float()
    elif v_quant == "e4m3_channel":
        vf, _ = quant_v_e4m3_channel(v)
    else:
        raise ValueError(f"unknown v_quant {v_quant}")
    out = torch.zeros(B, Hq, Nq, D, dtype=torch.float32)
    lse = torch.zeros(B, Hq, Nq, dtype=torch.float32)
    assert q_offset % block_m == 0
    for b in range(B):
        for h in range(Hq):
            kvh = h // g
            for r0 in range(0, Nq, block_m):
                r1 = min(r0 + block_m, Nq)
                qs = q_offset + r0
                qe = qs + block_m
                rows_abs = torch.arange(qs, qs + (r1 - r0))
                st = _RowState(r1 - r0, D)
                rng = kv_ranges(qs, qe, sink=sink,
                                w8=None if w8 is None else int(w8[h]),
                                w4=None if w4 is None else int(w4[h]))
                for lo, hi, use4, masked in rng:
                    qq = (q4f if use4 else qf)[b, h, r0:r1]
                    kk = (k4f if use4 else kf)[b, kvh]
                    for n0 in range(lo, hi, BLOCK_N):
                        if n0 >= Nk:
                            break  # every key of the block is past kv_len; reference loads zeros
                        n1 = min(n0 + BLOCK_N, Nk)
                        s = qq @ kk[n0:n1].T
                        if n1 - n0 < BLOCK_N:  # masked loads return 0 -> score 0 (attn_triton.py:66-68)
                            s = torch.cat([s, torch.zeros(s.shape[0], BLOCK_N - (n1 - n0))], dim=1)
                        vb = vf[b, kvh, n0:n1]
                        if n1 - n0 < BLOCK_N:
                            vb = torch.cat([vb, torch.zeros(BLOCK_N - (n1 - n0), D)], dim=0)
                        if masked:
                            cols = torch.arange(n0, n0 + BLOCK_N)
                            s = s + torch.where(rows_abs[:, None] >= cols[None, :], 0.0, MASK_ADD)
                        st.update(s, vb, p_quant, group_rows)
                o, ls = st.finish()
                out[b, h, r0:r1] = o
                lse[b, h, r0:r1] = ls
    return out.to(out_dtype), lse


def window_mask(Nq, Nk, *, q_offset, block_m, sink, w8, w4):
    """Explicit [Nq, Nk] bool mask (True = key contributes) equivalent to `kv_ranges` for one head,
    valid when every range bound is a multiple of 64 and ranges do not overlap."""
    allow = torch.zeros(Nq, Nk, dtype=torch.bool)
    for r0 in range(0, Nq, block_m):
        qs = q_offset + r0
        qe = qs + block_m
        for lo, hi, _, masked in kv_ranges(qs, qe, sink=sink, w8=w8, w4=w4):
            for n0 in range(lo, hi, BLOCK_N):
                n1 = min(n0 + BLOCK_N, Nk)
                if n0 >= Nk:
                    break
                r1 = min(r0 + block_m, Nq)
                if masked:
                    rows = torch.arange(qs, qs + (r1 - r0))[:, None]
                    cols = torch.arange(n0, n1)[None, :]
                    allow[r0:r1, n0:n1] |= rows >= cols
                else:
                    allow[r0:r1, n0:n1] = True
    return allow


# --------------------------------------------------------------------------- decode
def decode_blockwise(q, k, v, kv_lens=None, *, p_quant: int = P_NONE, out_dtype=torch.bfloat16,
                     token_range=None):
    """q_len == 1 attention streamed in 64-token blocks (attn_triton_decode.py:204-241), scores
    accumulated in fp32 (the reference reduces bf16 products in bf16, attn_triton_decode.py:221;
    this restatement and the HIP kernel are deliberately more accurate there).

    q [B,Hq,1,D], k/v [B,Hkv,L,D]; `kv_lens[b]` = valid prefix (default L).  `token_range=(t0,t1)`
    restricts to a split of the cache.  Returns (out_normalised fp32 [B,Hq,D], lse2 fp32 [B,Hq]);
    the caller casts.  The per-channel K-mean subtraction of `attn_unified` (:268-269) is *not*
    applied: it shifts every score of a row by the same constant and leaves softmax unchanged.
    """
    B, Hq, _, D = q.shape
    Hkv, L = k.shape[1], k.shape[2]
    g = Hq // Hkv
    qf = fold_scale(q, D).float()[:, :, 0]
    out = torch.zeros(B, Hq, D, dtype=torch.float32)
    lse = torch.full((B, Hq), float("-inf"), dtype=torch.float32)
    for b in range(B):
        Lb = int(kv_lens[b]) if kv_lens is not None else L
        t0, t1 = (0, Lb) if token_range is None else (min(token_range[0], Lb), min(token_range[1], Lb))
        if t1 <= t0:
            continue
        for h in range(Hq):
            kvh = h // g
            st = _RowState(1, D)
            st.l = torch.zeros(1)  # decode starts l at 0 (attn_triton_decode.py:211)
            kk = k[b, kvh, t0:t1].float()
            vv = v[b, kvh, t0:t1].float()  # decode multiplies p by fp32(v) (attn_triton_decode.py:234)
            for n0 in range(0, t1 - t0, BLOCK_N):
                s = qf[b, h][None, :] @ kk[n0:n0 + BLOCK_N].T
                m_new = torch.maximum(st.m, s.max(dim=1).values)
                p = torch.exp2(s - m_new[:, None])
                alpha = torch.exp2(st.m - m_new)
                st.l = st.l * alpha + p.sum(dim=1)
                st.acc = st.acc * alpha[:, None]
                if p_quant == P_STATIC448:
                    p = ((p * 448.0).to(torch.float8_e4m3fn).to(torch.float16) / 448).float()
                st.acc = st.acc + p @ vv[n0:n0 + BLOCK_N]
                st.m = m_new
            o, ls = st.finish()
            out[b, h] = o[0]
            lse[b, h] = ls[0]
    return out, lse


def combine_splits(outs, lses):
    """Merge split-KV partials: `lse = log2 sum_s 2^lse_s`, `o = sum_s 2^(lse_s-lse) o_s`.
    outs [S,B,H,D] fp32 (each normalised), lses [S,B,H] fp32 (-inf for an empty split)."""
    mx = lses.max(dim=0).values
    mx_safe = torch.where(torch.isinf(mx), torch.zeros_like(mx), mx)
    w = torch.exp2(lses - mx_safe[None])
    tot = w.sum(dim=0)
    lse = torch.log2(tot) + mx_safe
    o = (w[..., None] * outs).sum(dim=0) / tot[..., None]
    return o, lse


def decode_selected_exact(q, k, v, token_ids, score_scale=None):
    """Closed form of decode attention over a selection of the cache (build-defined; consumes the ids of
    `kmeans.topk_select`): q [B,Hq,1,D], k/v [B,Hkv,L,D], token_ids int [B*Hkv, n].  Row b*Hkv+kvh lists the tokens
    the q heads of kv head kvh attend to; negative or out-of-range entries are skipped.  Returns (out fp64
    [B,Hq,1,D], lse2 fp64 [B,Hq,1]); a head without valid entries gets zeros and -inf.  Gathers the rows and calls
    `exact_attention` (`score_scale` is passed on), so it is pinned by that function's checks."""
    B, Hq, _, D = q.shape
    Hkv, L = k.shape[1], k.shape[2]
    g = Hq // Hkv
    out = torch.zeros(B, Hq, 1, D, dtype=torch.float64)
    lse = torch.full((B, Hq, 1), float("-inf"), dtype=torch.float64)
    for b in range(B):
        for h in range(Hkv):
            ids = token_ids[b * Hkv + h].long()
            ids = ids[(ids >= 0) & (ids < L)]
            if ids.numel() == 0:
                continue
            o, l2 = exact_attention(q[b:b + 1, h * g:(h + 1) * g], k[b:b + 1, h:h + 1, ids], v[b:b + 1, h:h + 1, ids], causal=False,
                                    score_scale=score_scale)
            out[b, h * g:(h + 1) * g] = o[0]
            lse[b, h * g:(h + 1) * g] = l2[0]
    return out, lse
