"""The element-wise helpers of the reference's model_hub/utils.py on the gfx950 kernels (same names and arguments):
`silu_and_mul` (:4-13), `rmsnorm` (:15-19), `apply_rope_with_cos_sin_cache_inplace` (:21-106), plus
`yarn_cos_sin_cache`, the cos | sin table the reference builds in `model_hub/qwen.py:133-198, 227-228`.

Each helper is one kernel launch and writes nothing but its result, where the reference launches one kernel per
tensor operator (the rotary embedding alone peaks at 81 GB of temporaries at 1M tokens by the reference's own
comments, :82-91).  There is no CPU path.
"""
from __future__ import annotations

import math
from typing import Optional

import torch

from .. import _native as N


def _need_gpu(*ts):
    for t in ts:
        if not t.is_cuda:
            raise RuntimeError(f"tensors must live on the MI355X (got {t.device}); there is no CPU path")


def silu_and_mul(hidden_states: torch.Tensor, out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """[..., 2*I] -> [..., I]: `x2 * (x1 * sigmoid(x1))` for the two halves of the last dimension (utils.py:4-13)."""
    _need_gpu(hidden_states)
    two = hidden_states.shape[-1]
    x = hidden_states.reshape(-1, two)
    if x.stride(-1) != 1:
        x = x.contiguous()
    if out is None:
        out = torch.empty(*hidden_states.shape[:-1], two // 2, dtype=hidden_states.dtype, device=hidden_states.device)
    b = [N.dl(x), N.dl(out.view(-1, two // 2))]
    N.check(N.lib().sq_silu_and_mul(N.ptr(b[0]), N.ptr(b[1]), N.current_stream(x.device)))
    return out


LINEAR_ROWS_MAX = 8   # sq_linear_rows takes 1 to 8 activation rows; more is a GEMM


def _norm_fits(norm, rows: int, K: int, fuse_rows: int = 1) -> bool:
    """Should the RMS norm in front of a projection ride inside the projection's kernel?  The kernel takes it for up to
    four rows (8192 elements -- the stand-alone norm's limit -- of one or two rows, 5120 of three or four: the normalised
    rows have to fit its staging buffer), but every workgroup repeats the norm of every row: with one row that saves the
    norm's whole launch (gated projection of the decode step 47.1 -> 42.8 us, fused q/k/v 11.4 -> 10.6 us), with four rows
    it costs more than it saves (52 -> 66 us), hence `fuse_rows`."""
    w = norm[0]
    cap = 8192 if rows <= 2 else 5120 if rows <= 4 else 2048
    return rows <= fuse_rows and K <= cap and w.is_contiguous() and w.data_ptr() % 16 == 0 and w.shape == (K,)


def linear(x: torch.Tensor, weight: torch.Tensor, bias: Optional[torch.Tensor] = None, residual: Optional[torch.Tensor] = None,
           max_rows: int = 4, norm=None, fuse_norm_rows: int = 1) -> torch.Tensor:
    """`x @ weight.T (+ bias) (+ residual)` over the last dimension of x, weight [N, K] (the matmuls of
    model_hub/qwen.py:293-326).  Up to `max_rows` rows of x (a decode step) go through the weight-streaming HIP
    kernel; longer activations (a prompt) are a GEMM and go to the BLAS library.  The kernel takes up to
    LINEAR_ROWS_MAX rows; from five rows on the library's GEMM is as fast, hence the default.

    `norm` = (weight, epsilon): the product is taken of `rmsnorm(x, weight, epsilon)`; with up to `fuse_norm_rows` rows
    on the kernel's route the norm is part of the same pass (same values as the two calls)."""
    _need_gpu(x, weight)
    K = x.shape[-1]
    rows = x.numel() // K
    on_kernel = not (rows > min(max_rows, LINEAR_ROWS_MAX) or K % 8 or weight.stride(-1) != 1 or weight.stride(0) % 8 or weight.data_ptr() % 16)
    if norm is not None and not (on_kernel and _norm_fits(norm, rows, K, fuse_norm_rows)):
        x, norm = rmsnorm(x, norm[0], norm[1]), None
    if not on_kernel:
        y = torch.nn.functional.linear(x, weight, bias)
        return y if residual is None else residual + y
    x2 = x.reshape(rows, K)
    if x2.stride(-1) != 1 or (rows > 1 and x2.stride(0) % 8) or x2.data_ptr() % 16:
        x2 = x2.contiguous()
    n = weight.shape[0]
    out = torch.empty(*x.shape[:-1], n, dtype=x.dtype, device=x.device)
    b = [N.dl(x2), N.dl(weight), N.dl(bias) if bias is not None else None,
         N.dl(residual.reshape(rows, n)) if residual is not None else None, N.dl(out.view(rows, n))]
    tail = (N.ptr(b[1]), N.ptr(b[2]) if b[2] is not None else None, N.ptr(b[3]) if b[3] is not None else None, N.ptr(b[4]),
            N.current_stream(x.device))
    if norm is not None:
        nw = N.dl(norm[0])
        N.check(N.lib().sq_rmsnorm_linear_rows(N.ptr(b[0]), N.ptr(nw), float(norm[1]), *tail))
    else:
        N.check(N.lib().sq_linear_rows(N.ptr(b[0]), *tail))
    return out


def linear_silu_and_mul(x: torch.Tensor, weight: torch.Tensor, bias: Optional[torch.Tensor] = None, max_rows: int = 4, norm=None,
                        fuse_norm_rows: int = 1) -> torch.Tensor:
    """`silu_and_mul(x @ weight.T (+ bias))`, weight [2 I, K] = [gate | up] -> [..., I]: the first half of `mlp`
    (model_hub/qwen.py:320-324).  Up to `max_rows` rows go through one HIP kernel whose waves own both halves of an
    output pair (same values as `silu_and_mul(linear(x, weight, bias))`); longer activations take that route.
    `norm` as in `linear`."""
    _need_gpu(x, weight)
    K = x.shape[-1]
    rows = x.numel() // K
    n = weight.shape[0]
    on_kernel = not (rows > min(max_rows, LINEAR_ROWS_MAX) or K % 8 or n % 2 or weight.stride(-1) != 1 or weight.stride(0) % 8 or weight.data_ptr() % 16)
    if norm is not None and not (on_kernel and _norm_fits(norm, rows, K, fuse_norm_rows)):
        x, norm = rmsnorm(x, norm[0], norm[1]), None
    if not on_kernel:
        return silu_and_mul(torch.nn.functional.linear(x, weight, bias))
    x2 = x.reshape(rows, K)
    if x2.stride(-1) != 1 or (rows > 1 and x2.stride(0) % 8) or x2.data_ptr() % 16:
        x2 = x2.contiguous()
    out = torch.empty(*x.shape[:-1], n // 2, dtype=x.dtype, device=x.device)
    b = [N.dl(x2), N.dl(weight), N.dl(bias), N.dl(out.view(rows, n // 2))]
    if norm is not None:
        nw = N.dl(norm[0])
        N.check(N.lib().sq_rmsnorm_linear_rows_silu_and_mul(N.ptr(b[0]), N.ptr(nw), float(norm[1]), *[N.ptr(t) for t in b[1:]],
                                                            N.current_stream(x.device)))
    else:
        N.check(N.lib().sq_linear_rows_silu_and_mul(*[N.ptr(t) for t in b], N.current_stream(x.device)))
    return out


def linear_rope(x: torch.Tensor, weight: torch.Tensor, bias: Optional[torch.Tensor], position_ids: torch.Tensor, head_dim: int,
                rope_features: int, cos_sin_cache: torch.Tensor, max_rows: int = 4, cache=None, norm=None, fuse_norm_rows: int = 1) -> torch.Tensor:
    """The fused q/k/v projection with the rotary embedding of its first `rope_features` output features (the q and
    k heads) in one pass: x [batch, 1, K] -> [batch, 1, N], position_ids one position per row (model_hub/qwen.py:302-312
    and :352-379 on a decode step).  Same values as `linear` followed by `apply_rope_with_cos_sin_cache_inplace`,
    which is what longer activations (and more than `max_rows` rows) get.

    `cache` = (key_cache, value_cache, valid_length, attend_length) of the layer: the kernel also writes the rotated
    k and the v of every row to row `valid_length` of the caches and sets `attend_length` (what
    `flash_attn_cache.decode_update_kv_cache` does without advancing the length).  Returns None instead of the
    output when `cache` is given but the call cannot go through the kernel: the caller then runs the separate
    passes.  `norm` as in `linear`."""
    _need_gpu(x, weight, position_ids, cos_sin_cache)
    K = x.shape[-1]
    rows = x.numel() // K
    n = weight.shape[0]
    pos = position_ids.reshape(-1)
    if pos.dtype not in (torch.int32, torch.int64):
        pos = pos.to(torch.int64)
    on_kernel = not (rows > min(max_rows, LINEAR_ROWS_MAX) or K % 8 or weight.stride(-1) != 1 or weight.stride(0) % 8 or weight.data_ptr() % 16)
    if not on_kernel and cache is not None:
        return None
    if norm is not None and not (on_kernel and _norm_fits(norm, rows, K, fuse_norm_rows)):
        x, norm = rmsnorm(x, norm[0], norm[1]), None
    if not on_kernel:
        y = torch.nn.functional.linear(x, weight, bias)
        if rope_features > 0:   # the rotation works head by head: any split of the rotated part into two groups of heads will do
            flat = y.view(rows, n)
            cut = max(rope_features - head_dim, head_dim) if rope_features > head_dim else rope_features
            first, second = flat[:, :cut], flat[:, rope_features - head_dim:rope_features]
            r1, r2 = apply_rope_with_cos_sin_cache_inplace(pos.view(rows, 1), first, second, head_dim, cos_sin_cache)
            flat[:, :cut] = r1.reshape(rows, -1)
            flat[:, rope_features - head_dim:rope_features] = r2.reshape(rows, -1)
        return y
    x2 = x.reshape(rows, K)
    if x2.stride(-1) != 1 or (rows > 1 and x2.stride(0) % 8) or x2.data_ptr() % 16:
        x2 = x2.contiguous()
    out = torch.empty(*x.shape[:-1], n, dtype=x.dtype, device=x.device)
    b = [N.dl(x2), N.dl(weight), N.dl(bias), N.dl(pos.contiguous()), N.dl(cos_sin_cache), N.dl(out.view(rows, n))]
    c = [N.dl(t) for t in cache] if cache is not None else [None] * 4
    tail = (N.ptr(b[1]), N.ptr(b[2]), N.ptr(b[3]), N.ptr(b[4]), int(head_dim), int(rope_features), N.ptr(b[5]), *[N.ptr(t) for t in c],
            N.current_stream(x.device))
    if norm is not None:
        nw = N.dl(norm[0])
        N.check(N.lib().sq_rmsnorm_linear_rows_rope(N.ptr(b[0]), N.ptr(nw), float(norm[1]), *tail))
    else:
        N.check(N.lib().sq_linear_rows_rope(N.ptr(b[0]), *tail))
    return out


def rmsnorm(x: torch.Tensor, weight: torch.Tensor, epsilon: float = 1e-6, out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """`x * rsqrt(mean(x^2, -1) + epsilon) * weight` over the last dimension (utils.py:15-19)."""
    _need_gpu(x, weight)
    dim = x.shape[-1]
    x2 = x.reshape(-1, dim)
    if x2.stride(-1) != 1:
        x2 = x2.contiguous()
    if out is None:
        out = torch.empty(x.shape, dtype=x.dtype, device=x.device)
    b = [N.dl(x2), N.dl(weight), N.dl(out.view(-1, dim))]
    N.check(N.lib().sq_rmsnorm(N.ptr(b[0]), N.ptr(b[1]), N.ptr(b[2]), float(epsilon), N.current_stream(x.device)))
    return out


def apply_rope_with_cos_sin_cache_inplace(position_ids: torch.Tensor, query_states: torch.Tensor, key_states: torch.Tensor,
                                          head_dim: int, cos_sin_cache: torch.Tensor, use_cache: bool = True):
    """Rotary embedding (utils.py:21-106).  position_ids [batch, seq_len]; query_states [batch*seq_len, Hq*head_dim];
    key_states [batch*seq_len, Hkv*head_dim]; cos_sin_cache fp32 [max_seq_len, head_dim] (cos | sin).
    Returns `(q_out [batch, seq_len, Hq, head_dim], k_out [batch, seq_len, Hkv, head_dim])` like the reference; the
    inputs are left as they were (the reference overwrites them with values it then discards, :87-90)."""
    _need_gpu(query_states, key_states, position_ids, cos_sin_cache)
    bsz, seq_len = position_ids.shape
    q_out = torch.empty_like(query_states)
    k_out = torch.empty_like(key_states)
    pos = position_ids.reshape(-1)
    if pos.dtype not in (torch.int32, torch.int64):
        pos = pos.to(torch.int64)
    b = [N.dl(t) for t in (query_states, key_states, q_out, k_out, pos.contiguous(), cos_sin_cache)]
    N.check(N.lib().sq_rope(*[N.ptr(x) for x in b], int(head_dim), N.current_stream(query_states.device)))
    return (q_out.view(bsz, seq_len, -1, head_dim), k_out.view(bsz, seq_len, -1, head_dim))


def yarn_cos_sin_cache(head_dim: int, base: float, max_position_embeddings: int, max_length: int, device,
                       yarn_factor: float = 4.0, inv_freq: Optional[torch.Tensor] = None) -> torch.Tensor:
    """The fp32 [max_length, head_dim] cos | sin table of `model_hub/qwen.py:133-198, 227-228`.

    Up to 32768 positions: plain rotary frequencies `base^(-2i/head_dim)` (or the checkpoint's `inv_freq`), scaling 1.
    Beyond: YaRN with factor 4 -- dimensions that turn more than 32 times within the trained context keep their
    frequency, those that turn less than once are divided by the factor, a linear ramp in between, and cos/sin are
    multiplied by `0.1 ln(factor) + 1`.  Host-side set-up work (once per model), plain torch on the target device.
    """
    half = head_dim // 2
    exponent = torch.arange(0, head_dim, 2, dtype=torch.float32, device=device) / head_dim
    scaling = 1.0
    if max_length > 32768:
        def correction_dim(num_rotations):
            return head_dim * math.log(max_position_embeddings / (num_rotations * 2 * math.pi)) / (2 * math.log(base))

        low = max(math.floor(correction_dim(32)), 0)          # beta_fast
        high = min(math.ceil(correction_dim(1)), head_dim - 1)  # beta_slow
        hi = high + 0.001 if low == high else high
        ramp = ((torch.arange(half, dtype=torch.float32, device=device) - low) / (hi - low)).clamp(0, 1)
        keep = 1 - ramp
        pos_freqs = base ** exponent
        inv_freq = (1.0 / (yarn_factor * pos_freqs)) * (1 - keep) + (1.0 / pos_freqs) * keep
        scaling = 0.1 * math.log(yarn_factor) + 1.0
    elif inv_freq is None:
        inv_freq = 1.0 / (base ** exponent)
    inv_freq = inv_freq.to(device=device, dtype=torch.float32)
    t = torch.arange(max_length, device=device, dtype=torch.float32)
    freqs = torch.outer(t, inv_freq)
    return torch.cat((freqs.cos() * scaling, freqs.sin() * scaling), dim=-1).contiguous()
