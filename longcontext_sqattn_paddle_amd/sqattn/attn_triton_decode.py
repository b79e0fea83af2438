"""`attn_unified` / `attn_causal` of the reference's sqattn/attn_triton_decode.py:244-375 on the HIP kernels.

`qo_len == 1` runs the split-KV decode kernel (one pass over the cache for all q-heads of a KV group,
LSE combine); anything else runs the prefill kernel.  The module keeps the reference's file name so that
imports keep working; nothing here uses Triton.
"""
from __future__ import annotations

from typing import Optional

import torch

from .. import _native as N
from ._common import pad_head_dim, require_gpu


def attn_decode(q, k, v, tensor_layout="HND", output_dtype=torch.float16, return_lse=False, is_P_fp8_quant=False,
                seqlens: Optional[torch.Tensor] = None, num_splits: int = 0, workspace: Optional[torch.Tensor] = None,
                out: Optional[torch.Tensor] = None):
    """Decode attention: q [B,Hq,1,D] (HND) or [B,1,Hq,D] (NHD) against caches [B,Hkv,L,D] / [B,L,Hkv,D].

    Extensions over the reference (all optional): `seqlens` int32 [B] valid prefix per sequence,
    `num_splits` KV splits, caller-provided `workspace`/`out` so that a serving loop allocates nothing.
    With `num_splits=0` the library chooses, and on a batch with `seqlens` it deals its workgroups to the sequences in
    proportion to their lengths; a positive `num_splits` gives every sequence exactly that many splits, so that a
    sequence's result does not depend on its batch mates.
    """
    if tensor_layout not in N.LAYOUT:
        raise ValueError(f"tensor_layout {tensor_layout} not supported")
    require_gpu(q, k, v)
    head_dim_og = q.size(-1)
    q, k, v = pad_head_dim((q, k, v), head_dim_og)
    assert q.stride(-1) == 1 and k.stride(-1) == 1 and v.stride(-1) == 1
    hdim, ndim = (1, 2) if tensor_layout == "HND" else (2, 1)
    B, Hq, Hkv, L = q.size(0), q.size(hdim), k.size(hdim), k.size(ndim)
    lib = N.lib()
    S = num_splits if num_splits > 0 else lib.sq_decode_num_splits(B, Hkv, L)
    need = lib.sq_decode_workspace_bytes(B, Hq, 128, S)
    if workspace is None:
        workspace = torch.empty(need // 4, dtype=torch.float32, device=q.device)
    o = out if out is not None else torch.empty(q.shape, dtype=output_dtype, device=q.device)
    lse = torch.empty([B, Hq, 1], dtype=torch.float32, device=q.device) if return_lse else None
    params = N.DecodeParams(N.LAYOUT[tensor_layout], N.P_E4M3_STATIC if is_P_fp8_quant else N.P_NONE, max(num_splits, 0), head_dim_og)
    bq, bk, bv, bs, bo, bl, bw = (N.dl(t) for t in (q, k, v, seqlens, o, lse, workspace))
    N.check(lib.sq_decode_fwd(N.ptr(bq), N.ptr(bk), N.ptr(bv), N.ptr(bs), N.ptr(bo), N.ptr(bl), N.ptr(bw),
                              params, N.current_stream(q.device)))
    o = o[..., :head_dim_og]
    return (o, lse) if return_lse else o


def attn_decode_noalloc(q, k, v, out, tensor_layout="NHD", lse: Optional[torch.Tensor] = None, is_P_fp8_quant=False,
                        seqlens: Optional[torch.Tensor] = None, num_splits: int = 0):
    """`attn_decode` for callers that must not allocate device memory (graph capture, serving loops): head_dim 128
    tensors, caller-provided `out` (shape of q) and optional `lse` (fp32, B*Hq elements); the split-KV partials live
    in the library's own 8 MiB device array instead of a workspace tensor.  No reference counterpart.  Calls that
    overlap in time on one GPU share that array and race.  Returns `out`."""
    if tensor_layout not in N.LAYOUT:
        raise ValueError(f"tensor_layout {tensor_layout} not supported")
    require_gpu(q, k, v)
    if q.size(-1) != 128:
        raise ValueError("attn_decode_noalloc needs head_dim 128 tensors (padding would allocate)")
    params = N.DecodeParams(N.LAYOUT[tensor_layout], N.P_E4M3_STATIC if is_P_fp8_quant else N.P_NONE, num_splits, 128)
    b = [N.dl(t) for t in (q, k, v, seqlens, out, lse)]
    N.check(N.lib().sq_decode_fwd_noalloc(*[N.ptr(x) for x in b], params, N.current_stream(q.device)))
    return out


def attn_decode_selected(q, k, v, token_ids, tensor_layout="NHD", output_dtype=torch.float16, return_lse=False,
                         is_P_fp8_quant=False, seqlens: Optional[torch.Tensor] = None, num_splits: int = 0,
                         workspace: Optional[torch.Tensor] = None, out: Optional[torch.Tensor] = None):
    """Decode attention over a selection of the cache (no reference counterpart): `token_ids` int32 [B*Hkv, k]
    lists, per sequence and kv head, the cache rows to attend to -- what `cache_hub.kmeans.topk_select` returns.
    Negative entries (the missing tail of a selection) are skipped.  Other arguments as `attn_decode`."""
    if tensor_layout not in N.LAYOUT:
        raise ValueError(f"tensor_layout {tensor_layout} not supported")
    require_gpu(q, k, v)
    head_dim_og = q.size(-1)
    q, k, v = pad_head_dim((q, k, v), head_dim_og)
    hdim = 1 if tensor_layout == "HND" else 2
    B, Hq, Hkv = q.size(0), q.size(hdim), k.size(hdim)
    lib = N.lib()
    S = num_splits if num_splits > 0 else lib.sq_decode_num_splits(B, Hkv, token_ids.size(1))
    need = lib.sq_decode_workspace_bytes(B, Hq, 128, S)
    if workspace is None:
        workspace = torch.empty(need // 4, dtype=torch.float32, device=q.device)
    o = out if out is not None else torch.empty(q.shape, dtype=output_dtype, device=q.device)
    lse = torch.empty([B, Hq, 1], dtype=torch.float32, device=q.device) if return_lse else None
    params = N.DecodeParams(N.LAYOUT[tensor_layout], N.P_E4M3_STATIC if is_P_fp8_quant else N.P_NONE, max(num_splits, 0), head_dim_og)
    b = [N.dl(t) for t in (q, k, v, token_ids, seqlens, o, lse, workspace)]
    N.check(lib.sq_decode_selected_fwd(*[N.ptr(x) for x in b], params, N.current_stream(q.device)))
    o = o[..., :head_dim_og]
    return (o, lse) if return_lse else o


class DecodePlan:
    """A decode launch prepared once and replayed: every tensor (query, caches, seqlens, output, LSE,
    workspace) is borrowed up front, so `run()` is one C call that allocates nothing.  For serving loops
    whose buffers stay in place between steps (the KV cache grows in place; `seqlens` is updated on device).
    """

    def __init__(self, q, k, v, tensor_layout="NHD", output_dtype=torch.bfloat16, return_lse=False,
                 is_P_fp8_quant=False, seqlens=None, num_splits: int = 0):
        if tensor_layout not in N.LAYOUT:
            raise ValueError(f"tensor_layout {tensor_layout} not supported")
        require_gpu(q, k, v)
        if q.size(-1) != 128:
            raise ValueError("DecodePlan needs head_dim 128 tensors (pad once, outside the loop)")
        hdim, ndim = (1, 2) if tensor_layout == "HND" else (2, 1)
        B, Hq, Hkv, L = q.size(0), q.size(hdim), k.size(hdim), k.size(ndim)
        self._lib = N.lib()
        S = num_splits if num_splits > 0 else self._lib.sq_decode_num_splits(B, Hkv, L)
        self.workspace = torch.empty(self._lib.sq_decode_workspace_bytes(B, Hq, 128, S) // 4, dtype=torch.float32,
                                     device=q.device)
        self.out = torch.empty(q.shape, dtype=output_dtype, device=q.device)
        self.lse = torch.empty([B, Hq, 1], dtype=torch.float32, device=q.device) if return_lse else None
        self._params = N.DecodeParams(N.LAYOUT[tensor_layout], N.P_E4M3_STATIC if is_P_fp8_quant else N.P_NONE, max(num_splits, 0), 128)
        self._b = [N.dl(t) for t in (q, k, v, seqlens, self.out, self.lse, self.workspace)]
        self._ptrs = [N.ptr(x) for x in self._b]
        self._device = q.device

    def run(self, stream=None):
        st = N.current_stream(self._device) if stream is None else stream
        N.check(self._lib.sq_decode_fwd(*self._ptrs, self._params, st))
        return self.out


def attn_unified(q, k, v, tensor_layout="HND", output_dtype=torch.float16, return_lse=False, is_P_fp8_quant=False):
    """Unified interface (attn_triton_decode.py:244-361).

    Decode: the per-channel K-mean subtraction of the reference (:268-269) is skipped in the kernel, it shifts all
    scores of a row equally and cannot change the softmax; a returned log-sum-exp is moved into the reference's frame
    (scores of the centred keys) afterwards.  Prefill: K is centred with tensor ops as in
    the reference (the bf16 rounding of the centred K is part of its result), then the prefill kernel runs.
    """
    if tensor_layout not in N.LAYOUT:
        raise ValueError(f"tensor_layout {tensor_layout} not supported")
    seq_dim = 1 if tensor_layout == "NHD" else 2
    if q.size(seq_dim) == 1:
        res = attn_decode(q, k, v, tensor_layout, output_dtype, return_lse, is_P_fp8_quant)
        if not return_lse:
            return res
        # The reference subtracts the keys' token mean before the kernel (:268-269): the output is unchanged, but every
        # score of a row, and with it the returned base-2 log-sum-exp, is lower by q~ . mean(k) (q~ = q * log2e / sqrt(D)
        # rounded to the tensor dtype).  Put the log-sum-exp into that frame, the one the prefill branch below is in.
        o, lse = res
        head_dim = q.size(-1)
        sm = torch.tensor(1.0 / head_dim ** 0.5 * 1.44269504, dtype=torch.float32, device=q.device)
        q_folded = (q.float() * sm).to(q.dtype).float()
        # one pass over the keys in their own dtype with fp32 accumulation (no fp32 copy of the cache: 4 GB at 1M tokens)
        k_mean = k.mean(dim=seq_dim, dtype=torch.float32)                      # [B, Hkv, D]
        qh = q_folded.squeeze(seq_dim)                                         # [B, Hq, D]
        groups = qh.size(1) // k_mean.size(1)
        shift = (qh.view(qh.size(0), k_mean.size(1), groups, head_dim) * k_mean[:, :, None, :]).sum(-1).reshape(lse.shape)
        return o, lse - shift
    from .attn_triton import attn_causal as _prefill

    k = k - k.mean(dim=seq_dim, keepdim=True)
    return _prefill(q, k, v, tensor_layout, output_dtype, return_lse, is_P_fp8_quant)


def attn_causal(q, k, v, tensor_layout="HND", output_dtype=torch.float16, return_lse=False, is_P_fp8_quant=False):
    """Alias kept by the reference (attn_triton_decode.py:364-375)."""
    return attn_unified(q, k, v, tensor_layout, output_dtype, return_lse, is_P_fp8_quant)
