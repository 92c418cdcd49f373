"""MXFP8 linear: fp8 FPROP, DGRAD and WGRAD on the gfx950 block-scaled MFMA GEMM.

Same surface as the reference's ``MXFP8Linear``
(``src/kohakuwullm/kernels/mxfp8/linear.py:77-126``): a bias-free ``nn.Linear`` stand-in
whose quantized weight copies are plain attributes (never buffers, so they stay out of
``state_dict``), rebuilt by ``refresh_quantized_weight()`` after every optimizer step and
dropped by any ``_apply``.  ``in_features`` must be a multiple of 128; ``out_features`` is
zero-padded to one for DGRAD's contraction, which is exact.  Compute and output dtype
follow autocast, never the weight.

One difference from the reference, on purpose: WGRAD also runs in MXFP8
(``dW = Qcol(dY) . Qcol(X)^T`` with 32-token blocks), where the reference multiplies in
16 bits (``linear.py:72-73``).  A token count that is not a multiple of 32 is padded with
zero rows in front of the quantizers: zero rows add nothing to ``dW``, and their rows of
the output and of ``dX`` are dropped.
"""

from __future__ import annotations

import torch
import torch.nn.functional as F

from kohakuwullm_amd.kernels.mxfp8.quantize import (
    BLOCK_SCALE,
    mxfp8_matmul_pq,
    mxfp8_matmul_pq_batch,
    quantize_mx,
    quantize_mx_cols,
    quantize_mx_dual,
    stage_major_ok,
)

# Alignment of FPROP's contraction axis (kept at the reference's value so `swap_mxfp8`
# accepts and refuses exactly the same layers).
VENDOR_K_ALIGN = 128


def compute_dtype(x: torch.Tensor) -> torch.dtype:
    """The dtype ``nn.Linear`` would compute in for this input (autocast, else the input's)."""
    if torch.is_autocast_enabled("cuda"):
        return torch.get_autocast_dtype("cuda")
    return x.dtype


class _PadLastAxis:
    """Zero-pads the last axis by ``width`` columns; ``width == 0`` returns the tensor itself.

    A picklable callable: the module that owns it must survive ``copy.deepcopy`` and
    ``torch.save``.
    """

    __slots__ = ("width",)

    def __init__(self, width: int) -> None:
        self.width = int(width)

    def __call__(self, tensor: torch.Tensor) -> torch.Tensor:
        return F.pad(tensor, (0, self.width)) if self.width else tensor


def pad_tokens(x2d: torch.Tensor) -> torch.Tensor:
    """``x2d`` with zero rows appended up to the next multiple of 32 tokens (itself when it already is one)."""
    extra = -x2d.shape[0] % BLOCK_SCALE
    return F.pad(x2d, (0, 0, 0, extra)) if extra else x2d


class _MXFP8Linear(torch.autograd.Function):
    @staticmethod
    def forward(ctx, x, weight, wq_f, ws_f, wq_d, ws_d, pad_k):
        compute = compute_dtype(x)
        shape = x.shape
        x2d = x.reshape(-1, shape[-1]).to(compute)
        if x2d.stride(-1) != 1:
            x2d = x2d.contiguous()
        tokens = x2d.shape[0]
        need_dw = ctx.needs_input_grad[1] and tokens > 0
        # WGRAD contracts over the tokens (tens of thousands): its operands are written stage-major, a
        # K stage of a tile in one contiguous run, when tokens come in whole panels and dout needs no padding
        stage_major = need_dw and stage_major_ok(tokens) and pad_k.width == 0
        if need_dw:
            # One pass over x gives FPROP's operand and WGRAD's (blocks of 32 along the tokens).
            xq, xs, xtq, xts = quantize_mx_dual(pad_tokens(x2d), stage_major_t=stage_major)
            saved_x = (xtq, xts)
        else:
            xq, xs = quantize_mx(x2d)
            saved_x = (None, None)
        out = mxfp8_matmul_pq(xq, xs, wq_f, ws_f, compute)[:tokens]
        ctx.save_for_backward(*saved_x, wq_d, ws_d)
        ctx.stage_major = stage_major
        ctx.pad_k = pad_k
        ctx.x_dtype = x.dtype
        ctx.compute = compute
        ctx.out_features = weight.shape[0]
        return out.reshape(*shape[:-1], out.shape[-1])

    @staticmethod
    def backward(ctx, dout):
        xtq, xts, wq_d, ws_d = ctx.saved_tensors
        shape = dout.shape
        d2d = dout.reshape(-1, shape[-1]).to(ctx.compute).contiguous()
        tokens = d2d.shape[0]
        need_dx, need_dw = ctx.needs_input_grad[0], ctx.needs_input_grad[1] and xtq is not None
        dx = dw = None
        padded = ctx.pad_k(d2d)
        if need_dw:
            dq, ds, dtq, dts = quantize_mx_dual(pad_tokens(padded), stage_major_t=ctx.stage_major)
            n = ctx.out_features
            # dW (out,in) = dY^T (out,tokens) . (X^T (in,tokens))^T, contraction over tokens.
            wgrad = (dtq if ctx.stage_major else dtq[:n], dts[:n], xtq, xts)
            if need_dx and ctx.x_dtype == ctx.compute:
                # few tiles with a long K beside many with a short one: one launch shares the GPU
                dx, dw = mxfp8_matmul_pq_batch([(dq, ds, wq_d, ws_d), wgrad], ctx.compute)
                dx = dx[:tokens]
                return dx.reshape(*shape[:-1], dx.shape[-1]), dw, None, None, None, None, None
            dw = mxfp8_matmul_pq(*wgrad, ctx.compute)
        elif ctx.needs_input_grad[1]:
            dw = torch.zeros(ctx.out_features, wq_d.shape[0], device=d2d.device, dtype=ctx.compute)  # no tokens
            dq, ds = quantize_mx(padded) if need_dx else (None, None)
        else:
            dq, ds = quantize_mx(padded) if need_dx else (None, None)
        if need_dx:
            dx = mxfp8_matmul_pq(dq, ds, wq_d, ws_d, ctx.x_dtype)[:tokens]
            dx = dx.reshape(*shape[:-1], dx.shape[-1])
        return dx, dw, None, None, None, None, None


class MXFP8Linear(torch.nn.Module):
    """``nn.Linear`` (no bias) computing FPROP, DGRAD and WGRAD in MXFP8.

    ``refresh_quantized_weight`` must be called after every optimizer step.  ``dw`` comes
    back in the compute dtype and autograd casts it during accumulation.
    """

    def __init__(self, in_features: int, out_features: int, dtype=torch.bfloat16):
        super().__init__()
        if in_features % VENDOR_K_ALIGN:
            raise ValueError(
                f"in_features={in_features} must be a multiple of {VENDOR_K_ALIGN}; "
                "it is FPROP's contraction axis and is shared with the activation "
                "cast, so it cannot be padded without padding every input"
            )
        self.in_features = in_features
        self.out_features = out_features
        padded = -(-out_features // VENDOR_K_ALIGN) * VENDOR_K_ALIGN
        self.padded_out_features = padded
        self._pad_k = _PadLastAxis(padded - out_features)
        self.weight = torch.nn.Parameter(torch.empty(out_features, in_features, dtype=dtype))
        torch.nn.init.normal_(self.weight, std=in_features**-0.5)
        self._cache: tuple[torch.Tensor, ...] | None = None

    @torch.no_grad()
    def refresh_quantized_weight(self) -> None:
        wq_f, ws_f = quantize_mx(self.weight)
        if self._pad_k.width == 0:
            # Blocks along out_features without materialising the transpose.
            wq_d, ws_d = quantize_mx_cols(self.weight)
        else:
            wq_d, ws_d = quantize_mx(self._pad_k(self.weight.t()))
        self._cache = (wq_f, ws_f, wq_d, ws_d)

    def mxfp8_refresh_plan(self) -> list[torch.Tensor] | None:
        """The matrices whose row + column quantization is this module's cache, for a batched refresh.

        ``None`` when the cache is not a plain dual quantization of the weight (padded
        ``out_features``); ``refresh_mxfp8_weights`` then calls ``refresh_quantized_weight``.
        """
        if self._pad_k.width or self.out_features % BLOCK_SCALE or not self.weight.is_cuda:
            return None
        return [self.weight.detach()]

    def mxfp8_install(self, copies) -> None:
        """Take the ``(q, s, qT, sT)`` a batched refresh made of the planned matrix."""
        (self._cache,) = copies

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        if self._cache is None:
            self.refresh_quantized_weight()
        return _MXFP8Linear.apply(x, self.weight, *self._cache, self._pad_k)

    def _apply(self, *args, **kwargs):
        """Any device or dtype transform drops the quantized cache; ``forward`` rebuilds it."""
        self._cache = None
        return super()._apply(*args, **kwargs)

    def extra_repr(self) -> str:
        return f"in_features={self.in_features}, out_features={self.out_features}, mxfp8=True"
