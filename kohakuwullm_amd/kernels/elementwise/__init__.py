"""Elementwise producers of the MXFP8 path (the norm in front of a projection)."""

from kohakuwullm_amd.kernels.elementwise.rmsnorm import rms_norm, rms_norm_mx, rms_norm_mx_vendor

__all__ = ["rms_norm", "rms_norm_mx", "rms_norm_mx_vendor"]
