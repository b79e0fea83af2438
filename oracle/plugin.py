"""CPU restatement of the plugin closure `mp_triton_wrapper(...).attention_fn`
(sqattn/attn_replacer.py:296-454) and of `repeat_kv` (:281-293).

TEST INFRASTRUCTURE ONLY (see `oracle/__init__.py`).
"""
from __future__ import annotations

import torch

from . import attention as A
from . import fake_quant as FQ


def repeat_kv(x: torch.Tensor, n_rep: int) -> torch.Tensor:
    """[B,N,Hkv,D] -> [B,Hkv*n_rep,N,D], each kv head repeated n_rep times consecutively."""
    x = x.permute(0, 2, 1, 3)
    return x if n_rep == 1 else x.repeat_interleave(n_rep, dim=1)


def _qk_quant(x, qtype: str, bit: int):
    if bit == 4 or qtype == "int":
        return FQ.int_fake_quant(x, bit, True, "per_token")
    if qtype in ("e4m3", "e5m2"):
        return FQ.float_fake_quant(x, qtype, "per_token")
    raise ValueError(f"Invalid quantization type: {qtype}")


def _v_quant(x, qtype: str):
    if qtype == "int":
        return FQ.int_fake_quant(x, 8, True, "per_channel")
    if qtype in ("e4m3", "e5m2"):
        return FQ.float_fake_quant(x, qtype, "per_channel")
    raise ValueError(f"Invalid quantization type: {qtype}")


def key_mean_exact(key_hnd: torch.Tensor) -> torch.Tensor:
    """Token mean of an HND key tensor as the fused pre-pass defines it: the exact sum (fp64; exact for 16-bit
    inputs of ordinary range), divided by N, rounded to fp32 and then to the tensor dtype.  `Tensor.mean` of the
    reference (attn_replacer.py:338-339) accumulates in an implementation-defined order and can differ from it by
    one unit in the last place of the 16-bit result at near-ties."""
    n = key_hnd.shape[2]
    return (key_hnd.double().sum(dim=2, keepdim=True) / n).float().to(key_hnd.dtype)


def int_prepass(query, key, value, want_4bit=True, qk_qtype="int", v_qtype="int"):
    """CPU restatement of the operand pre-pass (attn_replacer.py:334-365) without the GQA expansion (which repeats
    heads and changes no value): inputs NHD `[B,N,H,D]`, outputs NHD `(q8, q4, k8, k4, v8)`; q4/k4 None unless
    `want_4bit`.  `qk_qtype` / `v_qtype` pick the 8-bit quantisers as the closure does (:340-358); the 4-bit ones are
    always the integer quantiser."""
    q, k, v = (t.permute(0, 2, 1, 3) for t in (query, key, value))   # HND views, as the reference quantises them
    kc = k - key_mean_exact(k)
    outs = [_qk_quant(q, qk_qtype, 8), FQ.int_fake_quant(q, 4, True, "per_token") if want_4bit else None,
            _qk_quant(kc, qk_qtype, 8), FQ.int_fake_quant(kc, 4, True, "per_token") if want_4bit else None,
            _v_quant(v, v_qtype)]
    return tuple(None if t is None else t.permute(0, 2, 1, 3).contiguous() for t in outs)


def plugin_attention(query, key, value, *, num_kv_groups, bit8, bit4, sink, relative,
                     qk_qtype="int", v_qtype="int", p_quant=A.P_NONE, int8_qk=False):
    """query [B,N,Hq,D], key/value [B,N,Hkv,D] (bf16) -> [B,N,Hq*D] bf16.

    Steps (attn_replacer.py:334-452): GQA expand + permute to HND; K minus its per-channel token
    mean (in the tensor dtype); 8-/4-bit per-token fake-quant of Q and centred K, 8-bit per-channel
    fake-quant of V; windowed prefill (relative: 64-row blocks, 4-bit operands aliased to the 8-bit
    ones, attn_triton_mix_relative.py:423,441-444; absolute: 128-row blocks, real 4-bit operands,
    attn_triton_mix_bad.py:386-392); back to [B,N,Hq*D].  `bit8`/`bit4` are per-head lists or scalars.

    `int8_qk` (build-defined, relative windows and the integer quantiser only): Q.K^T as a real integer product -- the
    8-bit codes of query and centred key are multiplied and summed exactly and the sum is scaled by the two per-token
    scales and by log2e / sqrt(D) in fp32.  The reference's path rounds `codes * scale` to bf16 (fake_quant.py:85) and
    the scaled query once more (attn_triton.py:251) before its bf16 product; this one does not, which is its only
    difference (restated here by handing the block-wise loop unrounded fp32 operands).
    """
    B, N, Hq, D = query.shape
    k = repeat_kv(key, num_kv_groups)
    v = repeat_kv(value, num_kv_groups)
    q = query.permute(0, 2, 1, 3)
    k = k - key_mean_exact(k)
    q8, q4 = _qk_quant(q, qk_qtype, 8), _qk_quant(q, qk_qtype, 4)
    k8, k4 = _qk_quant(k, qk_qtype, 8), _qk_quant(k, qk_qtype, 4)
    v8 = _v_quant(v, v_qtype)
    per_head = lambda w: [w] * Hq if not isinstance(w, (list, tuple)) else list(w)
    b8, b4 = per_head(bit8), per_head(bit4)
    if int8_qk:
        if not relative or qk_qtype != "int":
            raise ValueError("int8_qk: relative windows and the integer quantiser only")
        qc, qs = FQ.int_quant_codes(q, 8)
        kc, ks = FQ.int_quant_codes(k, 8)
        q8, k8 = qc * qs, kc * ks          # fp32, not rounded to the tensor dtype
    if relative:
        w8 = [A.window_size_relative(float(r), N) for r in b8]
        w4 = [A.window_size_relative(float(r), N) for r in b4]
        out, _ = A.prefill_blockwise(q8, k8, v8, p_quant=p_quant, block_m=64, sink=sink, w8=w8, w4=w4)
    else:
        out, _ = A.prefill_blockwise(q8, k8, v8, p_quant=p_quant, block_m=128, sink=sink,
                                     w8=[int(x) for x in b8], w4=[int(x) for x in b4], q4=q4, k4=k4)
    return out.transpose(1, 2).contiguous().view(B, N, Hq * D)


# ------------------------------------------------------- masked-SDPA emulation (delayed_sdpa_wrapper, attn_replacer.py:36-250)
def mix_bit_mask(kv_len: int, bit8_window, bit4_window, sink: int) -> torch.Tensor:
    """`construct_mix_bit_mask` / `construct_mix_bit_mask_per_head` (attn_replacer.py:63-112) called with
    `seq_len = 2 * kv_len` as the closure does (:152-165): a bool mask [kv_len, 2 * kv_len] (per head: [H, kv_len,
    2 * kv_len] when the windows are lists), True = attend.  Columns [0, kv_len) are the 8-bit keys, columns
    [kv_len, 2 kv_len) the 4-bit copies of the same keys.  Row i attends 8-bit key j iff j <= i and (j < sink or
    j > i - w8), and the 4-bit copy of key j iff j >= sink and i - w8 - w4 < j <= i - w8."""
    per_head = isinstance(bit8_window, (list, tuple)) or isinstance(bit4_window, (list, tuple))
    L = 2 * kv_len
    if per_head:
        w8 = torch.tensor(bit8_window).view(-1, 1, 1)
        w4 = torch.tensor(bit4_window).view(-1, 1, 1)
        q_idx = torch.arange(L).view(1, L, 1)
        kv_idx = torch.arange(L).view(1, 1, L)
    else:
        w8, w4 = bit8_window, bit4_window
        q_idx = torch.arange(L).unsqueeze(1)
        kv_idx = torch.arange(L).unsqueeze(0)
    causal = kv_idx <= q_idx
    fp8 = causal & ((kv_idx < sink) | (kv_idx > q_idx - w8))
    kv4 = kv_idx - L // 2
    int4 = (kv4 >= sink) & (kv4 <= q_idx - w8) & (kv4 > q_idx - w8 - w4)
    is8 = kv_idx < L // 2
    final = (is8 & fp8) | (~is8 & int4)
    return final[..., : L // 2, :]


def masked_sdpa_emulation(q, k, v, *, bit8_window, bit4_window, sink, qk_qtype="int", v_qtype="int"):
    """What the quantised branch of `delayed_sdpa_wrapper`'s closure sets out to compute (attn_replacer.py:123-186; the
    reference's own call passes the unconcatenated operands with the [L, 2L] mask and then stops in a debugger, :173-189):
    exact softmax attention of the 8-bit queries over the concatenation [8-bit keys ; 4-bit keys] with the values
    [v8 ; v8] under `mix_bit_mask`.  q, k, v [B,H,L,D] (heads already expanded).  K is centred over tokens first; V uses
    the asymmetric 8-bit per-channel quantiser of this branch (:141).  fp64, returns [B,H,L,D]."""
    kc = k - k.mean(dim=2, keepdim=True)
    q8 = _qk_quant(q, qk_qtype, 8)
    k8, k4 = _qk_quant(kc, qk_qtype, 8), _qk_quant(kc, qk_qtype, 4)
    v8 = FQ.int_fake_quant(v, 8, False, "per_channel") if v_qtype == "int" else FQ.float_fake_quant(v, v_qtype, "per_channel")
    L = k.shape[2]
    mask = mix_bit_mask(L, bit8_window, bit4_window, sink)[..., -q.shape[2]:, :]
    out, _ = A.exact_attention(q8, torch.cat([k8, k4], dim=2), torch.cat([v8, v8], dim=2), mask=mask if mask.ndim == 2 else mask[None])
    return out
