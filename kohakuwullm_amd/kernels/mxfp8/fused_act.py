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


def rmsnorm_mx_dual(x: torch.Tensor, weight: torch.Tensor | None, eps: float = 1e-6, stage_major_t: bool = False):
    """RMSNorm as both MXFP8 operands of the linear layer behind it: ``(q, s, qT, sT, rstd)``.

    ``(q, s)`` ``(M,K)``, ``(M,K//32)`` is ``rmsnorm_mx(x, weight, eps)`` bit for bit (the layer's forward operand);
    ``(qT, sT)`` ``(K,M)``, ``(K,M//32)`` is the same fp32 ``x * rstd * weight`` quantized along the tokens (the operand
    of its weight gradient: what ``quantize_mx_cols`` would make of it); ``rstd`` ``(M,)`` fp32 is what the norm's
    backward takes.  The normalized activation itself is never written.  ``M`` and ``K`` multiples of 32.
    ``stage_major_t``: ``qT`` as ``(M/128, K, 128)`` panels (``M % 128 == 0``), the layout the GEMM reads fastest on long
    token axes.  The reference has the row-axis half only (``rmsnorm_mx``, ``fused_act.py:146-175``).
    """
    from kohakuwullm_amd.kernels.elementwise.rmsnorm import _check

    _check(x, weight, True)
    x2 = x.contiguous().reshape(-1, x.shape[-1])
    m, k = x2.shape
    if m % BLOCK_SCALE or k % BLOCK_SCALE:
        raise ValueError(f"rows={m} and K={k} must be multiples of {BLOCK_SCALE}")
    if stage_major_t and (m % 128 or m <= 128):
        raise ValueError(f"stage_major_t needs a multiple of 128 tokens above 128, got {m}")
    dev, f8 = x.device, torch.float8_e4m3fn
    q = torch.empty(m, k, device=dev, dtype=f8)
    s = torch.empty(m, k // BLOCK_SCALE, device=dev, dtype=torch.uint8)
    qt = torch.empty((m // 128, k, 128) if stage_major_t else (k, m), device=dev, dtype=f8)
    st = torch.empty(k, m // BLOCK_SCALE, device=dev, dtype=torch.uint8)
    rstd = torch.empty(m, device=dev, dtype=torch.float32)
    if m and k:
        w = None if weight is None else weight.contiguous()
        _lib.invoke(
            "mx_rmsnorm_quantize_dual", m * k * (2 * x.element_size() + 2 * (1 + 1 / BLOCK_SCALE)), x2,
            x2.data_ptr(), _lib.MX_DTYPE[x2.dtype], m, k, x2.stride(0), 0 if w is None else w.data_ptr(),
            0 if w is None else _lib.MX_DTYPE[w.dtype], float(eps), rstd.data_ptr(), q.data_ptr(), k, s.data_ptr(),
            k // BLOCK_SCALE, qt.data_ptr(), 128 if stage_major_t else m, st.data_ptr(), m // BLOCK_SCALE,
        )
    return q, s, qt, st, rstd
