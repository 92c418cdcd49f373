"""MXFP8: e4m3 values with a UE8M0 power-of-two scale per 32 elements.

The names re-exported here are the ones ``kohakuwullm.kernels.mxfp8`` exports
(``src/kohakuwullm/kernels/mxfp8/__init__.py:17-35`` of the reference), so
``from kohakuwullm_amd.kernels.mxfp8 import quantize_mx`` is the drop-in spelling.
"""

from kohakuwullm_amd.kernels.mxfp8.quantize import (
    BLOCK_SCALE,
    E4M3_MAX,
    mxfp8_matmul,
    mxfp8_matmul_pq,
    mxfp8_matmul_pq_batch,
    quantize_mx,
    quantize_mx_cols,
    quantize_mx_dual,
    quantize_mx_dual_batch,
)



def quantize_mx_vendor(x):
    """``quantize_mx`` with swizzled e8m0 scales (``quantize.py:140-215`` of the reference); see :mod:`interop`."""
    from kohakuwullm_amd.kernels.mxfp8.interop import quantize_mx_vendor as impl

    return impl(x)


__all__ = [
    "BLOCK_SCALE",
    "E4M3_MAX",
    "mxfp8_matmul",
    "mxfp8_matmul_pq",
    "mxfp8_matmul_pq_batch",
    "quantize_mx",
    "quantize_mx_cols",
    "quantize_mx_dual",
    "quantize_mx_dual_batch",
    "quantize_mx_vendor",
]
