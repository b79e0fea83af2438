"""Host-side helpers shared by the kernel-level wrappers."""
from __future__ import annotations

import torch

KERNEL_HEAD_DIM = 128


def pad_head_dim(tensors, head_dim_og: int):
    """Zero-pad the last dimension to the kernels' head_dim of 128.

    The reference pads to 64 or 128 (attn_triton.py:236-244); zero channels add nothing to q.k and
    produce zero output channels that are sliced off again, so padding to 128 gives the same result.
    """
    if head_dim_og > KERNEL_HEAD_DIM:
        raise ValueError(f"Unsupported head_dim: {head_dim_og}")
    if head_dim_og == KERNEL_HEAD_DIM:
        return list(tensors)
    pad = KERNEL_HEAD_DIM - head_dim_og
    return [None if t is None else torch.nn.functional.pad(t, (0, pad)) for t in tensors]


def require_gpu(*tensors):
    for t in tensors:
        if t is not None and not t.is_cuda:
            raise RuntimeError("SQAttn kernels need tensors on the MI355X (tensor is on %s); there is no CPU path" % t.device)
