"""CPU restatement of the reference's element-wise layer helpers -- TEST INFRASTRUCTURE ONLY.

Followed reference code: model_hub/utils.py:4-13 (`silu_and_mul`), :15-19 (`rmsnorm`), :21-106
(`apply_rope_with_cos_sin_cache_inplace`); model_hub/qwen.py:293-326 (the `linear` calls of lm, wqkv, wo, mlp) with
the residual additions of model_hub/LLM.py:88-116.  The reference evaluates them as chains of tensor operators on 16-bit
tensors; every operator computes in fp32 and rounds its result to the tensor dtype, and an operator that meets the
fp32 cos/sin table yields fp32.  The functions below spell out those rounding points one by one.

Pinned in tests/test_oracle_layer.py against torch's own 16-bit CPU operators evaluating the reference's expressions
(an independent implementation of the same operator semantics), against fp64 closed forms, and by invariants (norm
preservation and position 0 of the rotation, scale equivariance of the normalisation).  Parity unpinned: whether
PaddlePaddle's kernels round exactly at these points (it cannot be run here); the order of the fp32 accumulation
inside `mean` (taken as exact here, which differs from any order only when the sum sits on a rounding boundary of
the 16-bit variance).  `linear` is pinned against torch's CPU matmul (fp32 and 16-bit), closed forms (identity and
all-ones weights) and linearity; unpinned: the accumulation order of the reference's GEMM (taken as exact here).
"""
from __future__ import annotations

import torch


def _r(x: torch.Tensor, dtype) -> torch.Tensor:
    """Round an fp32 tensor to `dtype` and return it as fp32 again."""
    return x.to(dtype).float()


def rmsnorm(x: torch.Tensor, weight: torch.Tensor, epsilon: float = 1e-6) -> torch.Tensor:
    """utils.py:17-19 on a 16-bit x [..., dim]."""
    dt = x.dtype
    xf = x.float()
    sq = _r(xf * xf, dt)                                                   # paddle.square
    mean = (sq.double().sum(-1, keepdim=True).float() / float(x.shape[-1]))  # paddle.mean: fp32 sum / n ...
    var = _r(mean, dt)                                                     # ... rounded to the tensor dtype
    ve = _r(var + torch.tensor(epsilon, dtype=torch.float32), dt)          # variance + epsilon
    r = _r(1.0 / torch.sqrt(ve), dt)                                       # paddle.rsqrt
    norm_x = _r(xf * r, dt)                                                # x * rsqrt(...)
    return (norm_x * weight.float()).to(dt)                                # norm_x * weight


def linear(x: torch.Tensor, weight: torch.Tensor, bias: torch.Tensor | None = None, residual: torch.Tensor | None = None) -> torch.Tensor:
    """qwen.py:296-325 on a 16-bit x [..., K], weight [N, K] (the reference passes `w.T` of the same storage): exact
    products and sums, the bias added before the one rounding of the matmul operator; `residual + linear(...)`
    (LLM.py:107, 115) is a second operator and rounds again."""
    dt = x.dtype
    y = x.double() @ weight.double().T
    if bias is not None:
        y = y + bias.double()
    y = y.to(torch.float32).to(dt)
    if residual is not None:
        y = (residual.float() + y.float()).to(dt)
    return y


def silu_and_mul(hidden_states: torch.Tensor) -> torch.Tensor:
    """utils.py:11-13 on a 16-bit [..., 2*I] tensor."""
    dt = hidden_states.dtype
    x1, x2 = hidden_states.float().chunk(2, dim=-1)
    sg = _r(torch.sigmoid(x1), dt)
    inner = _r(x1 * sg, dt)
    return (x2 * inner).to(dt)


def rope(position_ids: torch.Tensor, query_states: torch.Tensor, key_states: torch.Tensor, head_dim: int,
         cos_sin_cache: torch.Tensor):
    """utils.py:44-49, 74-85: q/k [T, H*head_dim] 16-bit, cos_sin_cache fp32 [max, head_dim] (cos | sin), position_ids
    any integer tensor of T entries.  Returns (q_out, k_out) with the inputs' shapes.  The products and the sum are
    separate fp32 operators (no fused multiply-add); one rounding to the tensor dtype at the end."""
    half = head_dim // 2
    pos = position_ids.reshape(-1).long()
    cos = cos_sin_cache[pos, :half].float()[:, None, :]
    sin = cos_sin_cache[pos, half:].float()[:, None, :]
    outs = []
    for x in (query_states, key_states):
        T = x.shape[0]
        xf = x.float().view(T, -1, head_dim)
        x1, x2 = xf[..., :half], xf[..., half:]
        o1 = (x1 * cos) - (x2 * sin)
        o2 = (x1 * sin) + (x2 * cos)
        outs.append(torch.cat([o1, o2], dim=-1).to(x.dtype).view(x.shape))
    return outs[0], outs[1]
