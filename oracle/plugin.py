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


def int_prepass(query, key, value, want_4bit=True):
    """CPU restatement of the operand pre-pass for the integer quantisers (attn_replacer.py:334-365) without the
    GQA expansion (which repeats heads and changes no value): inputs NHD `[B,N,H,D]`, outputs NHD
    `(q8, q4, k8, k4, v8)`; q4/k4 None unless `want_4bit`."""
    q, k, v = (t.permute(0, 2, 1, 3) for t in (query, key, value))   # HND views, as the reference quantises them
    kc = k - key_mean_exact(k)
    outs = [FQ.int_fake_quant(q, 8, True, "per_token"), FQ.int_fake_quant(q, 4, True, "per_token") if want_4bit else None,
            FQ.int_fake_quant(kc, 8, True, "per_token"), FQ.int_fake_quant(kc, 4, True, "per_token") if want_4bit else None,
            FQ.int_fake_quant(v, 8, True, "per_channel")]
    return tuple(None if t is None else t.permute(0, 2, 1, 3).contiguous() for t in outs)


def plugin_attention(query, key, value, *, num_kv_groups, bit8, bit4, sink, relative,
                     qk_qtype="int", v_qtype="int", p_quant=A.P_NONE):
    """query [B,N,Hq,D], key/value [B,N,Hkv,D] (bf16) -> [B,N,Hq*D] bf16.

    Steps (attn_replacer.py:334-452): GQA expand + permute to HND; K minus its per-channel token
    mean (in the tensor dtype); 8-/4-bit per-token fake-quant of Q and centred K, 8-bit per-channel
    fake-quant of V; windowed prefill (relative: 64-row blocks, 4-bit operands aliased to the 8-bit
    ones, attn_triton_mix_relative.py:423,441-444; absolute: 128-row blocks, real 4-bit operands,
    attn_triton_mix_bad.py:386-392); back to [B,N,Hq*D].  `bit8`/`bit4` are per-head lists or scalars.
    """
    B, N, Hq, D = query.shape
    k = repeat_kv(key, num_kv_groups)
    v = repeat_kv(value, num_kv_groups)
    q = query.permute(0, 2, 1, 3)
    k = k - (key_mean_exact(k) if qk_qtype == "int" and v_qtype == "int" else k.mean(dim=2, keepdim=True))
    q8, q4 = _qk_quant(q, qk_qtype, 8), _qk_quant(q, qk_qtype, 4)
    k8, k4 = _qk_quant(k, qk_qtype, 8), _qk_quant(k, qk_qtype, 4)
    v8 = _v_quant(v, v_qtype)
    per_head = lambda w: [w] * Hq if not isinstance(w, (list, tuple)) else list(w)
    b8, b4 = per_head(bit8), per_head(bit4)
    if relative:
        w8 = [A.window_size_relative(float(r), N) for r in b8]
        w4 = [A.window_size_relative(float(r), N) for r in b4]
        out, _ = A.prefill_blockwise(q8, k8, v8, p_quant=p_quant, block_m=64, sink=sink, w8=w8, w4=w4)
    else:
        out, _ = A.prefill_blockwise(q8, k8, v8, p_quant=p_quant, block_m=128, sink=sink,
                                     w8=[int(x) for x in b8], w4=[int(x) for x in b4], q4=q4, k4=k4)
    return out.transpose(1, 2).contiguous().view(B, N, Hq * D)
