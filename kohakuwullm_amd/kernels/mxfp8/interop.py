"""The reference's vendor MXFP8 interface on MI355X: swizzled scales in, natural scales inside.

Counterpart of ``src/kohakuwullm/kernels/mxfp8/interop.py`` (``swizzle_mx_scales`` :24-41,
``expected_swizzled_numel`` :44-48, ``vendor_mxfp8_matmul_swizzled`` :51-75, ``as_vendor_scales``
:78-80, ``vendor_mxfp8_matmul`` :83-103, ``mxfp8_mm_swizzled`` + fake :106-122) and of
``quantize_mx_vendor`` (``quantize.py:140-215``).  There the swizzle is the layout cuBLAS reads;
the gfx950 MFMA kernels read the natural ``(rows, K//32)`` layout, so here the swizzled form is
an exchange format: it is produced on request and converted back in front of the GEMM, which
costs one pass over the scales (1/32 of the operand bytes).
"""

from __future__ import annotations

import torch

from kohakuwullm_amd import _lib
from kohakuwullm_amd.kernels.mxfp8.quantize import BLOCK_SCALE, mxfp8_matmul_pq, quantize_mx

SCALE_ROW_TILE = 128
SCALE_COL_TILE = 4
VENDOR_K_ALIGN = SCALE_COL_TILE * BLOCK_SCALE
_E8M0 = getattr(torch, "float8_e8m0fnu", torch.uint8)


def _ceil_div(a: int, b: int) -> int:
    return -(-a // b)


def expected_swizzled_numel(rows: int, k: int) -> int:
    """Bytes of the flat swizzled scale buffer of a ``(rows, k)`` operand."""
    return _ceil_div(rows, SCALE_ROW_TILE) * SCALE_ROW_TILE * _ceil_div(_ceil_div(k, BLOCK_SCALE), SCALE_COL_TILE) * SCALE_COL_TILE


def swizzle_mx_scales(scales: torch.Tensor) -> torch.Tensor:
    """``(rows, K//32)`` ue8m0 bytes -> the flat ``SWIZZLE_32_4_4`` layout, zero padded to whole tiles."""
    if scales.dim() != 2 or scales.element_size() != 1:
        raise ValueError(f"scales must be a 2-D byte tensor, got {tuple(scales.shape)} {scales.dtype}")
    _lib.require_gpu(scales, "scales")
    if scales.stride(1) != 1:
        scales = scales.contiguous()
    rows, cols = scales.shape
    out = torch.empty(expected_swizzled_numel(rows, cols * BLOCK_SCALE), device=scales.device, dtype=torch.uint8)
    if out.numel():
        _lib.invoke("mx_swizzle_scales", rows * cols + out.numel(), scales,
                    scales.data_ptr(), rows, cols, scales.stride(0), out.data_ptr())
    return out


def unswizzle_mx_scales(swizzled: torch.Tensor, rows: int, k: int) -> torch.Tensor:
    """The inverse: flat swizzled bytes of a ``(rows, k)`` operand -> natural ``(rows, k//32)``."""
    cols = k // BLOCK_SCALE
    if swizzled.element_size() != 1 or swizzled.numel() != expected_swizzled_numel(rows, k):
        raise ValueError(
            f"swizzled scales hold {swizzled.numel()} bytes, a ({rows}, {k}) operand needs {expected_swizzled_numel(rows, k)}"
        )
    _lib.require_gpu(swizzled, "swizzled")
    flat = swizzled.contiguous().view(torch.uint8).reshape(-1)
    out = torch.empty(rows, cols, device=swizzled.device, dtype=torch.uint8)
    if out.numel():
        _lib.invoke("mx_unswizzle_scales", rows * cols + flat.numel(), flat, flat.data_ptr(), rows, cols, out.data_ptr(), cols)
    return out


def as_vendor_scales(scales: torch.Tensor) -> torch.Tensor:
    """``(rows, K//32)`` uint8 -> the swizzled e8m0 tensor the vendor entry points take."""
    return swizzle_mx_scales(scales).view(_E8M0)


def quantize_mx_vendor(x: torch.Tensor) -> tuple[torch.Tensor, torch.Tensor]:
    """``quantize_mx`` with the scales in the flat swizzled e8m0 layout.  ``K % 128 == 0``.

    Same codes as :func:`quantize_mx`; a singly-strided (transposed) view is read in place.
    """
    if x.shape[-1] % VENDOR_K_ALIGN:
        raise ValueError(f"K={x.shape[-1]} must be a multiple of {VENDOR_K_ALIGN}")
    q, s = quantize_mx(x)
    return q, as_vendor_scales(s)


def vendor_mxfp8_matmul_swizzled(aq, a_swizzled, bq, b_swizzled, out_dtype: torch.dtype = torch.bfloat16) -> torch.Tensor:
    """``aq @ bq.T`` from operands whose scales are already swizzled."""
    if aq.dim() != 2 or bq.dim() != 2 or aq.shape[1] != bq.shape[1]:
        raise ValueError(f"contraction mismatch: {tuple(aq.shape)} @ {tuple(bq.shape)}.T")
    k = aq.shape[1]
    if k % BLOCK_SCALE:
        raise ValueError(f"K={k} must be a multiple of {BLOCK_SCALE}")
    a_scale = unswizzle_mx_scales(a_swizzled, aq.shape[0], k)
    b_scale = unswizzle_mx_scales(b_swizzled, bq.shape[0], k)
    return mxfp8_matmul_pq(aq, a_scale, bq, b_scale, out_dtype)


def vendor_mxfp8_matmul(aq, a_scale, bq, b_scale, out_dtype: torch.dtype = torch.bfloat16) -> torch.Tensor:
    """Convenience wrapper: swizzle the natural-layout scales, then multiply (for correctness checks)."""
    return vendor_mxfp8_matmul_swizzled(aq, as_vendor_scales(a_scale), bq, as_vendor_scales(b_scale), out_dtype)


@torch.library.custom_op("kohakuwullm_amd::mxfp8_mm_swizzled", mutates_args=())
def mxfp8_mm_swizzled(
    aq: torch.Tensor,
    a_scale: torch.Tensor,
    bq: torch.Tensor,
    b_scale: torch.Tensor,
    out_dtype: torch.dtype = torch.bfloat16,
) -> torch.Tensor:
    """:func:`vendor_mxfp8_matmul_swizzled` as an opaque op, so a graph compiler traces past it."""
    return vendor_mxfp8_matmul_swizzled(aq, a_scale, bq, b_scale, out_dtype)


@mxfp8_mm_swizzled.register_fake
def _mxfp8_mm_swizzled_fake(aq, a_scale, bq, b_scale, out_dtype=torch.bfloat16):
    return aq.new_empty((aq.shape[0], bq.shape[0]), dtype=out_dtype)
