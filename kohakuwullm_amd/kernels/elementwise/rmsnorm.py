"""RMSNorm that can hand the next projection its MXFP8 operand: ``(out, e4m3, ue8m0)`` from one pass.

Counterpart of ``src/kohakuwullm/kernels/elementwise/rmsnorm.py`` (``_RMSNorm`` :130-229,
``rms_norm`` :232-236, ``rms_norm_mx`` :239-246, ``rms_norm_mx_vendor`` :249-258).  The fp8 pair is
quantized from the fp32 normalized row, not from the rounded 16-bit ``out``, and carries no
gradient: dgrad reaches the norm through ``out``.

Differences from the reference, on purpose: the tensors must live on the GPU (there is no ATen
route here, so ``rms_norm`` on a CPU tensor raises instead of falling back), any row width that is
a multiple of 8 is taken (no 16384 cap), and the sum of squares is accumulated in fp64.
"""

from __future__ import annotations

import torch

from kohakuwullm_amd import _lib
from kohakuwullm_amd.kernels.mxfp8.quantize import BLOCK_SCALE

_FP8 = torch.float8_e4m3fn
_E8M0 = getattr(torch, "float8_e8m0fnu", torch.uint8)
_ACT = (torch.bfloat16, torch.float16)
# Partial weight-gradient rows = workgroups of the backward kernel.  The reference fixes 512 (rmsnorm.py:206); here the
# kernel holds three waves per SIMD, i.e. three workgroups per CU, and fewer leave a third of the latency hiding unused
# (32768 x 2048 bf16 on 256 CUs: 110 us with 512, 94 us with 768, 115 us with 1024, which runs a ragged second round).
BWD_WORKGROUPS_PER_CU = 3


def backward_partial_rows(device) -> int:
    return BWD_WORKGROUPS_PER_CU * torch.cuda.get_device_properties(device).multi_processor_count


def launch_rmsnorm(x2d, weight, eps: float, out, rstd, q, s) -> None:
    """One launch of ``mx_rmsnorm_quantize``; any of ``out``, ``rstd``, ``(q, s)`` may be ``None``."""
    m, k = x2d.shape
    written = (0 if out is None else x2d.element_size()) + (0 if q is None else 1 + 1 / BLOCK_SCALE)
    _lib.invoke(
        "mx_rmsnorm_quantize", m * k * (x2d.element_size() + written), x2d,
        x2d.data_ptr(), _lib.MX_DTYPE[x2d.dtype], m, k, x2d.stride(0),
        0 if weight is None else weight.data_ptr(), 0 if weight is None else _lib.MX_DTYPE[weight.dtype], float(eps),
        0 if out is None else out.data_ptr(), 0 if out is None else out.stride(0),
        0 if rstd is None else rstd.data_ptr(),
        0 if q is None else q.data_ptr(), 0 if q is None else q.stride(0),
        0 if s is None else s.data_ptr(), 0 if s is None else s.stride(0),
    )


def _check(x: torch.Tensor, weight: torch.Tensor | None, quant: bool) -> None:
    _lib.require_gpu(x, "x")
    k = x.shape[-1]
    if x.dtype not in _ACT:
        raise ValueError(f"x.dtype={x.dtype} is not one of {_ACT}")
    if weight is not None:
        _lib.require_gpu(weight, "weight")
        if weight.shape != (k,):
            raise ValueError(f"weight {tuple(weight.shape)} does not match the row width {k}")
        if weight.dtype not in (x.dtype, torch.float32):
            raise ValueError(f"weight.dtype={weight.dtype} must be {x.dtype} or float32")
    if quant and k % BLOCK_SCALE:
        raise ValueError(f"quant needs n_cols % {BLOCK_SCALE} == 0, got {k}")


class _RMSNorm(torch.autograd.Function):
    @staticmethod
    def forward(ctx, x, weight, eps, quant=False, write_out=True, swizzle=False):
        _check(x, weight, quant)
        shape = x.shape
        x2d = x.reshape(-1, shape[-1]).contiguous()
        n_rows, n_cols = x2d.shape
        if swizzle and n_cols % (4 * BLOCK_SCALE):
            raise ValueError(f"swizzle needs n_cols % {4 * BLOCK_SCALE} == 0")
        if weight is not None:
            weight = weight.contiguous()
        dev = x2d.device
        rstd = torch.empty(n_rows, dtype=torch.float32, device=dev)
        out = torch.empty_like(x2d) if write_out else None
        q = s = None
        if quant:
            q = torch.empty(n_rows, n_cols, dtype=_FP8, device=dev)
            s = torch.empty(n_rows, n_cols // BLOCK_SCALE, dtype=torch.uint8, device=dev)
        if n_rows and n_cols:
            launch_rmsnorm(x2d, weight, eps, out, rstd, q, s)
        ctx.save_for_backward(x2d, weight, rstd)
        # without this autograd would fill zero "gradients" for the fp8 pair on every backward
        ctx.set_materialize_grads(False)
        if out is None:
            out = x2d.new_empty(0)
        elif write_out:
            out = out.reshape(shape)
        if not quant:
            return out
        if swizzle:
            from kohakuwullm_amd.kernels.mxfp8.interop import swizzle_mx_scales

            s = swizzle_mx_scales(s)  # flat, zero padded to whole 128-row tiles
        # the fp8 pair carries no gradient; dgrad reaches the norm through `out`
        ctx.mark_non_differentiable(q, s)
        return out, q, s

    @staticmethod
    def backward(ctx, dout, *_unused_fp8_grads):
        if dout is None:
            return None, None, None, None, None, None
        x2d, weight, rstd = ctx.saved_tensors
        shape = dout.shape
        dout2d = dout.reshape(-1, shape[-1]).contiguous()
        n_rows, n_cols = x2d.shape
        dx = torch.empty_like(x2d)
        has_w = weight is not None and ctx.needs_input_grad[1]
        parts = max(1, min((n_rows + 3) // 4, backward_partial_rows(x2d.device)))
        dw_part = torch.empty(parts, n_cols, dtype=torch.float32, device=x2d.device) if has_w else None
        if n_cols:
            _lib.invoke(
                "mx_rmsnorm_backward", n_rows * n_cols * 3 * x2d.element_size(), x2d,
                x2d.data_ptr(), _lib.MX_DTYPE[x2d.dtype], n_rows, n_cols, x2d.stride(0),
                0 if weight is None else weight.data_ptr(), 0 if weight is None else _lib.MX_DTYPE[weight.dtype],
                dout2d.data_ptr(), dout2d.stride(0), rstd.data_ptr(), dx.data_ptr(), dx.stride(0),
                0 if dw_part is None else dw_part.data_ptr(), parts,
            )
        dw = dw_part.sum(0).to(weight.dtype) if has_w else None
        return dx.reshape(shape), dw, None, None, None, None


def rms_norm(x: torch.Tensor, weight: torch.Tensor | None, eps: float = 1e-6) -> torch.Tensor:
    """Fused RMSNorm on the GPU (no MXFP8 output)."""
    return _RMSNorm.apply(x, weight, eps)


def rms_norm_mx(x: torch.Tensor, weight: torch.Tensor | None, eps: float = 1e-6):
    """Fused RMSNorm returning ``(out, e4m3, ue8m0)``, the fp8 pair K-blocked: ``(rows, K)``, ``(rows, K//32)``."""
    return _RMSNorm.apply(x, weight, eps, True, True)


def rms_norm_mx_vendor(x: torch.Tensor, weight: torch.Tensor | None, eps: float = 1e-6):
    """RMSNorm emitting scales in the flat ``SWIZZLE_32_4_4`` exchange layout (zero padded to 128-row tiles)."""
    out, q, s = _RMSNorm.apply(x, weight, eps, True, True, True)
    return out, q, s.view(_E8M0)
