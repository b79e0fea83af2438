"""Fake quantisers with the reference's class names and arguments (sqattn/fake_quant.py), on torch tensors.

`IntegerQuantizer(bit, symmetric, granularity)` / `FloatQuantizer("e4m3"|"e5m2", True, granularity)` and
their `fake_quant_tensor` / `real_quant_tensor` behave like the reference's: ranges per tensor, per
"channel" (reduced over dims 0 and 1, fake_quant.py:30-32) or per token (last dim), rounding half away
from zero as `paddle.round` does, and the home-made float simulation of fake_quant.py:151-204 including
its quirks (largest e4m3 output 240, no subnormals).  These are elementwise tensor passes that feed the
HIP attention kernels; they run wherever the tensor lives.
"""
from __future__ import annotations

import torch


def _round(x: torch.Tensor) -> torch.Tensor:
    return torch.sign(x) * torch.floor(torch.abs(x) + 0.5)


class BaseQuantizer(object):
    def __init__(self, bit, symmetric, granularity, **kwargs):
        self.bit = bit
        self.sym = symmetric
        self.granularity = granularity
        self.kwargs = kwargs
        if self.granularity == "per_group":
            self.group_size = self.kwargs["group_size"]
        self.calib_algo = self.kwargs.get("calib_algo", "minmax")

    def get_tensor_range(self, tensor):
        if self.calib_algo == "minmax":
            return self.get_minmax_range(tensor)
        if self.calib_algo == "mse":
            raise NotImplementedError
        raise ValueError(f"Unsupported calibration algorithm: {self.calib_algo}")

    def get_minmax_range(self, tensor):
        if tensor.dtype in (torch.bfloat16, torch.float16):
            tensor = tensor.float()
        if self.granularity == "per_tensor":
            return tensor.min(), tensor.max()
        if self.granularity == "per_channel":
            return tensor.amin(dim=(0, 1), keepdim=True), tensor.amax(dim=(0, 1), keepdim=True)
        return tensor.amin(dim=-1, keepdim=True), tensor.amax(dim=-1, keepdim=True)

    def get_qparams(self, tensor_range, device):
        min_val, max_val = tensor_range
        qmin, qmax = self.qmin.to(device), self.qmax.to(device)
        if self.sym:
            abs_max = torch.maximum(max_val.abs(), min_val.abs()).clamp(min=1e-05)
            scales = abs_max / qmax
            zeros = torch.tensor(0.0, device=device)
        else:
            scales = (max_val - min_val).clamp(min=1e-05) / (qmax - qmin)
            zeros = torch.minimum(torch.maximum(qmin - _round(min_val / scales), qmin), qmax)
        return scales, zeros, qmax, qmin

    def reshape_tensor(self, tensor, allow_padding=False):
        return tensor.reshape(-1, self.group_size) if self.granularity == "per_group" else tensor

    def restore_tensor(self, tensor, shape):
        return tensor if tensor.shape == shape else tensor.reshape(shape)

    def get_tensor_qparams(self, tensor):
        tensor = self.reshape_tensor(tensor)
        tensor_range = self.get_tensor_range(tensor)
        scales, zeros, qmax, qmin = self.get_qparams(tensor_range, tensor.device)
        return tensor, scales, zeros, qmax, qmin

    def fake_quant_tensor(self, tensor):
        org_shape, org_dtype = tensor.shape, tensor.dtype
        tensor, scales, zeros, qmax, qmin = self.get_tensor_qparams(tensor)
        tensor = self.quant_dequant(tensor.float(), scales, zeros, qmax, qmin)
        return self.restore_tensor(tensor, org_shape).to(org_dtype)

    def real_quant_tensor(self, tensor):
        org_shape = tensor.shape
        tensor, scales, zeros, qmax, qmin = self.get_tensor_qparams(tensor)
        tensor = self.quant(tensor.float(), scales, zeros, qmax, qmin)
        tensor = self.restore_tensor(tensor, org_shape)
        return tensor, scales, (None if self.sym else zeros)

    def quant_dequant(self, tensor, scales, zeros, qmax, qmin):
        return self.dequant(self.quant(tensor, scales, zeros, qmax, qmin), scales, zeros)

    def dequant(self, tensor, scales, zeros):
        return (tensor - zeros) * scales


class IntegerQuantizer(BaseQuantizer):
    def __init__(self, bit, symmetric, granularity, **kwargs):
        super().__init__(bit, symmetric, granularity, **kwargs)
        if "int_range" in self.kwargs:
            qmin, qmax = self.kwargs["int_range"]
        elif self.sym:
            qmin, qmax = -(2 ** (self.bit - 1)), 2 ** (self.bit - 1) - 1
        else:
            qmin, qmax = 0.0, 2 ** self.bit - 1
        self.qmin = torch.tensor(float(qmin))
        self.qmax = torch.tensor(float(qmax))
        self.dst_nbins = 2 ** bit

    def quant(self, tensor, scales, zeros, qmax, qmin):
        return torch.minimum(torch.maximum(_round(tensor / scales) + zeros, qmin), qmax)


def float_quantize(x, e_bits=5, m_bits=10, rounding="nearest"):
    """Float simulation of fake_quant.py:151-204 (nearest or stochastic mantissa rounding)."""
    assert rounding in ["nearest", "stochastic"]
    bias = 2 ** (e_bits - 1) - 1
    eps = 2.0 ** (-m_bits)
    max_exp = 2 ** (e_bits - 1) - 1
    min_exp = 1 - bias
    sign = torch.sign(x)
    x = torch.abs(x)
    zero_mask = x == 0
    exp = torch.floor(torch.log2(x + 1e-30))
    frac = x / (2.0 ** exp) - 1.0
    exp_clamped = exp.clamp(min_exp, max_exp)
    if rounding == "nearest":
        frac_q = _round(frac / eps) * eps
    else:
        frac_q = torch.floor(frac / eps + torch.rand_like(frac)) * eps
    frac_q = frac_q.clamp(0.0, 1.0 - eps)
    x_q = (1.0 + frac_q) * (2.0 ** exp_clamped) * sign
    max_val = (2 - 2 ** (-m_bits)) * (2.0 ** max_exp)
    x_q = x_q.clamp(-max_val, max_val)
    return torch.where(zero_mask, torch.zeros_like(x_q), x_q)


class FloatQuantizer(BaseQuantizer):
    def __init__(self, bit, symmetric, granularity, **kwargs):
        super().__init__(bit, symmetric, granularity, **kwargs)
        assert self.bit in ["e4m3", "e5m2"], f"Unsupported bit configuration: {self.bit}"
        assert self.sym
        self.e_bits, self.m_bits, fmax = (4, 3, 448.0) if self.bit == "e4m3" else (5, 2, 57344.0)
        self.qmin, self.qmax = torch.tensor(-fmax), torch.tensor(fmax)

    def quant(self, tensor, scales, zeros, qmax, qmin):
        scaled = torch.minimum(torch.maximum(tensor / scales + zeros, qmin), qmax)
        return float_quantize(scaled.float(), self.e_bits, self.m_bits, rounding="nearest")


def fused_int_prepass(query, key, value, want_4bit=True, tensor_layout="NHD", qk_qtype="int", v_qtype="int", skip_query=False):
    """The operand pre-pass of `mp_triton_wrapper`'s closure (attn_replacer.py:334-365) as one call into the HIP
    library: key centring, per-token 8-bit (and integer 4-bit) fake quantisation of query and centred key, per-channel
    8-bit fake quantisation of value -- without expanding the kv heads.  `qk_qtype` / `v_qtype` pick the 8-bit
    quantisers as the closure does (:340-358): "int", "e4m3" or "e5m2".

    query [B,N,Hq,D], key/value [B,N,Hkv,D] for "NHD" ([B,H,N,D] for "HND"), bf16 or fp16, D == 128.
    Returns (q8, q4, k8, k4, v8) in the layout of the inputs; q4 and k4 are None unless `want_4bit`.  With `skip_query`
    the query is left alone and q8 is None (the attention kernel applies the 8-bit integer quantiser while it loads the
    rows, `q_quant=8`); not together with `want_4bit`.
    """
    from .. import _native as N
    from ._common import require_gpu

    if tensor_layout not in N.LAYOUT:
        raise ValueError(f"tensor_layout {tensor_layout} not supported")
    require_gpu(query, key, value)
    assert query.stride(-1) == 1 and key.stride(-1) == 1 and value.stride(-1) == 1, "Last dim of qkv must be contiguous."
    if query.size(-1) != 128:
        raise ValueError(f"Unsupported head_dim for the fused pre-pass: {query.size(-1)}")
    hdim, ndim = (1, 2) if tensor_layout == "HND" else (2, 1)
    B, Hkv, Nk = key.size(0), key.size(hdim), key.size(ndim)
    lib = N.lib()
    if skip_query and want_4bit:
        raise ValueError("skip_query leaves no query to derive the 4-bit operands from")
    q8 = None if skip_query else torch.empty_like(query)
    k8, v8 = torch.empty_like(key), torch.empty_like(value)
    q4 = torch.empty_like(query) if want_4bit else None
    k4 = torch.empty_like(key) if want_4bit else None
    need = lib.sq_fake_quant_prepass_workspace_bytes(B, Hkv, Nk)
    ws = torch.empty((need + 7) // 8, dtype=torch.float64, device=query.device)
    b = [N.dl(t) for t in (query, key, value, q8, q4, k8, k4, v8, ws)]
    for name in (qk_qtype, v_qtype):
        if name not in N.QTYPE:
            raise ValueError(f"Invalid quantization type: {name}")
    N.check(lib.sq_fake_quant_prepass_typed(*[N.ptr(x) for x in b], N.LAYOUT[tensor_layout], N.QTYPE[qk_qtype], N.QTYPE[v_qtype],
                                            N.current_stream(query.device)))
    return q8, q4, k8, k4, v8


def fused_int8qk_prepass(query, key, value, tensor_layout="NHD"):
    """The operand pre-pass for the integer Q.K^T path (`attn_int8qk_relative_window`): key centring, then the 8-bit
    per-token codes of the centred key (int8, laid out like `key`) and their fp32 scales `[B, Hkv, N rounded up to 64]`
    (the tail zero), and the per-channel 8-bit fake quantisation of value.  The query passes through untouched.
    Returns (k_codes, k_scale, v8)."""
    from .. import _native as N
    from ._common import require_gpu

    if tensor_layout not in N.LAYOUT:
        raise ValueError(f"tensor_layout {tensor_layout} not supported")
    require_gpu(query, key, value)
    assert query.stride(-1) == 1 and key.stride(-1) == 1 and value.stride(-1) == 1, "Last dim of qkv must be contiguous."
    if query.size(-1) != 128:
        raise ValueError(f"Unsupported head_dim for the fused pre-pass: {query.size(-1)}")
    hdim, ndim = (1, 2) if tensor_layout == "HND" else (2, 1)
    B, Hkv, Nk = key.size(0), key.size(hdim), key.size(ndim)
    lib = N.lib()
    k_codes = torch.empty(key.shape, dtype=torch.int8, device=key.device)
    k_scale = torch.zeros(B, Hkv, (Nk + 63) // 64 * 64, dtype=torch.float32, device=key.device)
    v8 = torch.empty_like(value)
    need = lib.sq_fake_quant_prepass_workspace_bytes(B, Hkv, Nk)
    ws = torch.empty((need + 7) // 8, dtype=torch.float64, device=query.device)
    b = [N.dl(t) for t in (query, key, value, k_codes, k_scale, v8, ws)]
    N.check(lib.sq_fake_quant_prepass_int8qk(*[N.ptr(x) for x in b], N.LAYOUT[tensor_layout], N.current_stream(query.device)))
    return k_codes, k_scale, v8
