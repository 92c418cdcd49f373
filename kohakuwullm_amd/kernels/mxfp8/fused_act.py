"""Activation epilogue that emits MXFP8 directly, so the consumer GEMM needs no cast.

Mirrors ``swiglu_mx`` (``src/kohakuwullm/kernels/mxfp8/fused_act.py:69-101``) and ``rmsnorm_mx``
(``:146-175``) of the reference.
"""

from __future__ import annotations

import torch

from kohakuwullm_amd import _lib
from kohakuwullm_amd.kernels.mxfp8.quantize import BLOCK_SCALE


def swiglu_mx(gate: torch.Tensor, up: torch.Tensor):
    """``silu(gate) * up`` as ``(e4m3 (M,K), ue8m0 (M, K//32))``; K a multiple of 32.

    The product is kept in fp32 and quantized from there.
    """
    if gate.shape != up.shape:
        raise ValueError(f"gate {tuple(gate.shape)} != up {tuple(up.shape)}")
    if gate.shape[-1] % BLOCK_SCALE:
        raise ValueError(f"K={gate.shape[-1]} must be a multiple of {BLOCK_SCALE}")
    if gate.dtype != up.dtype or gate.dtype not in (torch.bfloat16, torch.float16):
        raise ValueError(f"gate/up must share a 16-bit dtype, got {gate.dtype}, {up.dtype}")
    _lib.require_gpu(gate, "gate")
    shape = gate.shape
    g2, u2 = gate.reshape(-1, shape[-1]), up.reshape(-1, shape[-1])
    # chunked halves of one projection are accepted through their row pitch
    if g2.stride(1) != 1:
        g2 = g2.contiguous()
    if u2.stride(1) != 1:
        u2 = u2.contiguous()
    m, k = g2.shape
    q = torch.empty(m, k, device=gate.device, dtype=torch.float8_e4m3fn)
    s = torch.empty(m, k // BLOCK_SCALE, device=gate.device, dtype=torch.uint8)
    if m and k:
        _lib.invoke(
            "mx_swiglu_quantize_rows", m * k * (2 * gate.element_size() + 1 + 1 / BLOCK_SCALE), gate,
            g2.data_ptr(), u2.data_ptr(), _lib.MX_DTYPE[gate.dtype], m, k, g2.stride(0), u2.stride(0),
            q.data_ptr(), k, s.data_ptr(), k // BLOCK_SCALE,
        )
    return q, s


def rmsnorm_mx(x: torch.Tensor, weight: torch.Tensor, eps: float = 1e-6):
    """RMSNorm as ``(e4m3 (M,K), ue8m0 (M, K//32))``; K a multiple of 32.  The 16-bit output is not written."""
    from kohakuwullm_amd.kernels.elementwise.rmsnorm import _check, launch_rmsnorm

    if x.shape[-1] % BLOCK_SCALE:
        raise ValueError(f"K={x.shape[-1]} must be a multiple of {BLOCK_SCALE}")
    _check(x, weight, True)
    x2 = x.contiguous().reshape(-1, x.shape[-1])
    m, k = x2.shape
    q = torch.empty(m, k, device=x.device, dtype=torch.float8_e4m3fn)
    s = torch.empty(m, k // BLOCK_SCALE, device=x.device, dtype=torch.uint8)
    if m and k:
        launch_rmsnorm(x2, None if weight is None else weight.contiguous(), eps, None, None, q, s)
    return q, s
