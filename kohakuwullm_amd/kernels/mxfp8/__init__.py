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
)

__all__ = [
    "BLOCK_SCALE",
    "E4M3_MAX",
    "mxfp8_matmul",
    "mxfp8_matmul_pq",
    "mxfp8_matmul_pq_batch",
    "quantize_mx",
    "quantize_mx_cols",
    "quantize_mx_dual",
]
