"""Quantize a ``(T, H, D)`` attention operand to e4m3 with ue8m0 blocks along D.

Counterpart of ``src/kohakuwullm/kernels/mxfp8/attention_quant.py`` (``column_mean`` :78-80,
``quantize_heads`` :83-118): scale blocks run along the head dimension, the contraction axis of
``QK^T``; ``mu`` is subtracted in fp32 registers, so no widened or shifted copy of the operand
reaches memory.  An operand with unit stride along D (a slice of a fused projection output, for
instance) is read where it lies; any other layout is made contiguous first.

Differences from the reference, on purpose: any ``head_dim`` that is a multiple of 32 is taken
(the reference also needs ``head_dim / 32`` to be a power of two, a limit of its tile shapes),
``block_m`` is accepted and ignored, and the tensors must live on the GPU.
"""

from __future__ import annotations

import torch

from kohakuwullm_amd import _lib
from kohakuwullm_amd.kernels.mxfp8.quantize import BLOCK_SCALE


def column_mean(x: torch.Tensor) -> torch.Tensor:
    """Per-head, per-channel mean of a ``(T, H, D)`` operand as ``(H, D)`` fp32."""
    return x.mean(dim=0, dtype=torch.float32)


def quantize_heads(x: torch.Tensor, mu: torch.Tensor | None = None, block_m: int = 32):
    """``(T, H, D)`` -> ``(e4m3 (T, H, D), ue8m0 (T, H, D // 32))``.

    ``mu`` is an ``(H, D)`` fp32 mean subtracted before quantizing.
    """
    del block_m
    if x.dim() != 3:
        raise ValueError(f"x must be (T, H, D), got shape {tuple(x.shape)}")
    t, heads, head_dim = x.shape
    if head_dim % BLOCK_SCALE:
        raise ValueError(f"head_dim={head_dim} must be a multiple of {BLOCK_SCALE}")
    if x.dtype not in _lib.MX_DTYPE:
        raise ValueError(f"x.dtype={x.dtype} is not one of {tuple(_lib.MX_DTYPE)}")
    _lib.require_gpu(x, "x")
    if mu is not None:
        if mu.shape != (heads, head_dim) or mu.dtype != torch.float32 or mu.device != x.device:
            raise ValueError(f"mu must be ({heads}, {head_dim}) float32 on {x.device}")
        mu = mu.contiguous()
    unit = 16 // x.element_size()
    if t and heads and (x.stride(2) != 1 or x.stride(0) % unit or x.stride(1) % unit or x.data_ptr() % 16
                        or (heads > 1 and x.stride(1) < head_dim)):
        x = x.contiguous()
    q = torch.empty(t, heads, head_dim, device=x.device, dtype=torch.float8_e4m3fn)
    s = torch.empty(t, heads, head_dim // BLOCK_SCALE, device=x.device, dtype=torch.uint8)
    if q.numel():
        _lib.invoke("mx_quantize_heads", q.numel() * (x.element_size() + 1 + 1 / BLOCK_SCALE), x,
                    x.data_ptr(), _lib.MX_DTYPE[x.dtype], t, heads, head_dim, x.stride(0), x.stride(1),
                    0 if mu is None else mu.data_ptr(), q.data_ptr(), s.data_ptr())
    return q, s
