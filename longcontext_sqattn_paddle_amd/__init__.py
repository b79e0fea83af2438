"""MI355X (gfx950) implementation of SQAttn's attention hot path.

Sub-packages mirror the reference's module paths so that the entry points are drop-in:
`sqattn.attn_replacer`, `sqattn.attn_triton`, `sqattn.attn_triton_decode`,
`sqattn.attn_triton_mix_relative`, `sqattn.attn_triton_mix_bad`, `sqattn.fake_quant`,
`cache_hub.kmeans`.  All compute goes through `libsqattn_hip.so` (hand-written HIP kernels).
"""
from . import _native  # noqa: F401

__all__ = ["_native"]
