"""Dense SwiGLU feed-forward in MXFP8 with the activation fused into the quantizers.

The reference's dense ``GLUMLP`` runs ``w_out(silu(gate) * value)`` as two ``MXFP8Linear``
calls around an eager 16-bit activation (``src/kohakuwullm/models/components/mlp.py:68-73``)
and names the fused cast ``swiglu_mx`` (``kernels/mxfp8/fused_act.py:69-101``) as the
producer epilogue it wants.  This function is that fusion for the whole layer:

forward   X --dual quantize--> GU = Xq . Wq_in^T --SwiGLU + dual quantize--> Y = Hq . Wq_out^T
backward  dY --dual quantize--> dH = dYq . Wq_out_d^T --SwiGLU' + dual quantize--> dX = dPq . Wq_in_d^T
          dW_out = dY^T . H^T-blocks,  dW_in = dP^T . X^T-blocks   (contraction over tokens)

``h`` and ``dpre`` never exist in 16 bits: the SwiGLU kernels read the GEMM output once and
emit the row-blocked operand for the next GEMM and the token-blocked operand for WGRAD.
"""

from __future__ import annotations

import torch

from kohakuwullm_amd import _lib
from kohakuwullm_amd.kernels.mxfp8.linear import compute_dtype, pad_tokens
from kohakuwullm_amd.kernels.mxfp8.quantize import (
    BLOCK_SCALE,
    PANEL,
    mxfp8_matmul_pq,
    mxfp8_matmul_pq_batch,
    quantize_mx_dual,
    stage_major_ok,
)

_FP8 = torch.float8_e4m3fn

# The two projection outputs that only the SwiGLU quantizers read (`gu`, `dh`) are allocated with 128 spare
# elements per row.  Their natural pitches (16 KiB and 8 KiB at the benchmark shape) put the 128 rows a quantizer
# tile reads at once on a few memory channels; 256 bytes more spread them.  Measured in the step at 16384 x 1536 x
# 4096: SwiGLU 75.6 -> 73.1 us, SwiGLU' 135.0 -> 129.4 us, the GEMM that writes `gu` 183.7 -> 186.0 us (64 or 256
# elements: no gain).
_PITCH_PAD = 128


def swiglu_mx_dual(gu: torch.Tensor, stage_major_t: bool = False):
    """``h = silu(gu[:, :H]) * gu[:, H:]`` as ``(q, s, qT, sT)``: blocks along H and along tokens.

    ``stage_major_t``: ``qT`` as ``(tokens // 128, H, 128)`` (see :func:`quantize_mx_dual`).
    """
    m, two_h = gu.shape
    h = two_h // 2
    if two_h % 2 or h % BLOCK_SCALE or m % BLOCK_SCALE:
        raise ValueError(f"gu {tuple(gu.shape)}: tokens and hidden must be multiples of {BLOCK_SCALE}")
    if stage_major_t and not stage_major_ok(m):
        raise ValueError(f"stage_major_t needs the token count {m} to be a positive multiple of {PANEL}")
    _lib.require_gpu(gu, "gu")
    q = torch.empty(m, h, device=gu.device, dtype=_FP8)
    s = torch.empty(m, h // BLOCK_SCALE, device=gu.device, dtype=torch.uint8)
    qt = torch.empty((m // PANEL, h, PANEL) if stage_major_t else (h, m), device=gu.device, dtype=_FP8)
    st = torch.empty(h, m // BLOCK_SCALE, device=gu.device, dtype=torch.uint8)
    _lib.invoke(
        "mx_swiglu_quantize_dual", m * h * (2 * gu.element_size() + 2 * (1 + 1 / BLOCK_SCALE)), gu,
        gu.data_ptr(), _lib.MX_DTYPE[gu.dtype], m, h, gu.stride(0), q.data_ptr(), h, s.data_ptr(), h // BLOCK_SCALE,
        qt.data_ptr(), PANEL if stage_major_t else m, st.data_ptr(), m // BLOCK_SCALE,
    )
    return q, s, qt, st


def swiglu_bwd_mx_dual(dh: torch.Tensor, gu: torch.Tensor, stage_major: bool = False):
    """SwiGLU backward emitted straight in MXFP8: ``dpre = [dgate | dup]`` as ``(q, s, qT, sT)``.

    ``stage_major``: ``q`` as ``(2H // 128, tokens, 128)`` and ``qT`` as ``(tokens // 128, 2H, 128)``
    (tokens and H multiples of 128; see :func:`quantize_mx_dual`).
    """
    m, two_h = gu.shape
    h = two_h // 2
    if dh.shape != (m, h) or h % BLOCK_SCALE or m % BLOCK_SCALE:
        raise ValueError(f"dh {tuple(dh.shape)} does not match gu {tuple(gu.shape)}")
    if stage_major and not (stage_major_ok(m) and stage_major_ok(h)):
        raise ValueError(f"stage_major needs tokens={m} and H={h} to be positive multiples of {PANEL}")
    _lib.require_gpu(gu, "gu")
    q = torch.empty((two_h // PANEL, m, PANEL) if stage_major else (m, two_h), device=gu.device, dtype=_FP8)
    s = torch.empty(m, two_h // BLOCK_SCALE, device=gu.device, dtype=torch.uint8)
    qt = torch.empty((m // PANEL, two_h, PANEL) if stage_major else (two_h, m), device=gu.device, dtype=_FP8)
    st = torch.empty(two_h, m // BLOCK_SCALE, device=gu.device, dtype=torch.uint8)
    _lib.invoke(
        "mx_swiglu_bwd_quantize_dual", m * h * (3 * gu.element_size() + 4 * (1 + 1 / BLOCK_SCALE)), gu,
        dh.data_ptr(), dh.stride(0), gu.data_ptr(), gu.stride(0), _lib.MX_DTYPE[gu.dtype], m, h,
        q.data_ptr(), PANEL if stage_major else two_h, s.data_ptr(), two_h // BLOCK_SCALE,
        qt.data_ptr(), PANEL if stage_major else m, st.data_ptr(), m // BLOCK_SCALE,
    )
    return q, s, qt, st


_WHOLE_RANGE: dict = {}


def _whole_range(device, rows: int) -> torch.Tensor:
    """``[0, rows]`` as the offset table of a single "expert" that owns every row (cached: built once)."""
    key = (device, rows)
    if key not in _WHOLE_RANGE:
        _WHOLE_RANGE[key] = torch.tensor([0, rows], dtype=torch.int32, device=device)
    return _WHOLE_RANGE[key]


def fused_swiglu_projection(xq, xs, wq, ws, out_dtype):
    """``gu = x . w_in^T`` with SwiGLU and both casts of ``h`` in the GEMM's epilogue.

    Returns ``gu (M, 2H)`` in ``out_dtype`` (the rounded accumulators, saved for the backward),
    ``h`` quantized along H ``(hq, hs)`` and along the tokens ``(htq, hts)``.  ``h`` is computed
    from the rounded ``gu``, exactly as :func:`swiglu_mx_dual` does on the stored tensor.
    Needs ``M % 128 == 0`` (token-axis tiles) and a 128-multiple contraction.
    """
    from kohakuwullm_amd.kernels.mxfp8.moe import launch_gemm1

    m, k = xq.shape
    hidden = wq.shape[0] // 2
    dev = xq.device
    gu = torch.empty(m, 2 * hidden, device=dev, dtype=out_dtype)
    hq = torch.empty(m, hidden, device=dev, dtype=_FP8)
    hs = torch.empty(m, hidden // BLOCK_SCALE, device=dev, dtype=torch.uint8)
    htq = torch.empty(hidden, m, device=dev, dtype=_FP8)
    hts = torch.empty(hidden, m // BLOCK_SCALE, device=dev, dtype=torch.uint8)
    launch_gemm1(xq, xs, None, wq.unsqueeze(0), ws.unsqueeze(0), hq, hs, gu, _whole_range(dev, m), hidden, k, out_dtype,
                 htq, hts)
    return gu, hq, hs, htq, hts


class _MXFP8SwiGLUMLP(torch.autograd.Function):
    @staticmethod
    def forward(ctx, x, w_in, w_out, in_f, in_d, out_f, out_d):
        compute = compute_dtype(x)
        shape = x.shape
        x2d = x.reshape(-1, shape[-1]).to(compute)
        if x2d.stride(-1) != 1:
            x2d = x2d.contiguous()
        tokens = x2d.shape[0]
        x2d = pad_tokens(x2d)  # whole 32-token blocks for WGRAD; zero rows change no gradient
        # The operands of the three backward products that go down in one launch (contractions of
        # 8192 and 16384) are written stage-major: each K stage of a tile is then one contiguous run.
        sm = x.dtype == compute and stage_major_ok(tokens) and stage_major_ok(w_out.shape[1])
        xq, xs, xtq, xts = quantize_mx_dual(x2d, stage_major_t=sm)
        # GEMM, then one bandwidth-bound pass for SwiGLU and both casts: measured faster at the
        # benchmark shape (220 + 89 us) than the same work in the GEMM's epilogue
        # (fused_swiglu_projection: 329 us), whose vector ALU work cannot overlap the MFMAs.
        gu = mxfp8_matmul_pq(xq, xs, *in_f, compute, out_pad=_PITCH_PAD)
        hq, hs, htq, hts = swiglu_mx_dual(gu, stage_major_t=sm)
        y = mxfp8_matmul_pq(hq, hs, *out_f, compute)
        if any(ctx.needs_input_grad):
            ctx.save_for_backward(xtq, xts, gu, htq, hts, *in_d, *out_d)
            ctx.compute = compute
            ctx.x_dtype = x.dtype
            ctx.stage_major = sm
        return y[:tokens].reshape(*shape[:-1], y.shape[-1])

    @staticmethod
    def backward(ctx, dout):
        xtq, xts, gu, htq, hts, win_dq, win_ds, wout_dq, wout_ds = ctx.saved_tensors
        shape = dout.shape
        d2d = dout.reshape(-1, shape[-1]).to(ctx.compute).contiguous()
        tokens = d2d.shape[0]
        dq, ds, dtq, dts = quantize_mx_dual(pad_tokens(d2d), stage_major_t=ctx.stage_major)
        dh = mxfp8_matmul_pq(dq, ds, wout_dq, wout_ds, ctx.compute, out_pad=_PITCH_PAD)
        pq, ps, ptq, pts = swiglu_bwd_mx_dual(dh, gu, stage_major=ctx.stage_major)
        # The last three products are independent and none fills the GPU alone (dW has few
        # tiles with a long K): they go down together and share the GPU by work.
        wanted = [
            (pq, ps, win_dq, win_ds) if ctx.needs_input_grad[0] else None,
            (ptq, pts, xtq, xts) if ctx.needs_input_grad[1] else None,
            (dtq, dts, htq, hts) if ctx.needs_input_grad[2] else None,
        ]
        grads = [None, None, None]
        if ctx.x_dtype == ctx.compute:
            live = [i for i, w in enumerate(wanted) if w is not None]
            for i, g in zip(live, mxfp8_matmul_pq_batch([wanted[i] for i in live], ctx.compute)):
                grads[i] = g
        else:
            for i, w in enumerate(wanted):
                if w is not None:
                    grads[i] = mxfp8_matmul_pq(*w, ctx.x_dtype if i == 0 else ctx.compute)
        dx, dw_in, dw_out = grads
        if dx is not None:
            dx = dx[:tokens].reshape(*shape[:-1], -1)
        return dx, dw_in, dw_out, None, None, None, None


def mxfp8_swiglu_mlp(x, w_in, w_out, packed) -> torch.Tensor:
    """``(silu(x W_g^T) * (x W_u^T)) W_out^T`` with ``w_in = [W_g; W_u]`` ``(2H, dim)``, ``w_out`` ``(dim, H)``.

    ``packed`` is ``(in_fwd, in_dgrad, out_fwd, out_dgrad)``, each a ``(codes, scales)`` pair:
    the weights blocked along their contraction axis for FPROP and along the other axis for
    DGRAD.  ``w_in``/``w_out`` are passed so autograd routes ``dW`` to the master parameters.
    ``dim`` and ``H`` must be multiples of 32; any token count is taken (it is padded with zero
    rows to whole 32-token blocks, which changes no result).
    """
    if w_in.shape[0] != 2 * w_out.shape[1] or w_in.shape[1] != x.shape[-1] or w_out.shape[0] != x.shape[-1]:
        raise ValueError(f"shape mismatch: x {tuple(x.shape)}, w_in {tuple(w_in.shape)}, w_out {tuple(w_out.shape)}")
    return _MXFP8SwiGLUMLP.apply(x, w_in, w_out, *packed)
