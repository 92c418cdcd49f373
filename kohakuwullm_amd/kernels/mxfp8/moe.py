"""The routed-expert path in MXFP8: the fused four-kernel graph, its weights, and the unfused twin.

Counterpart of the reference's ``src/kohakuwullm/kernels/mxfp8/moe.py`` (``MXFP8ExpertWeights``
:34-61, ``_MXFP8Experts`` :181-336, ``mxfp8_moe_experts`` :374-405,
``mxfp8_moe_experts_reference`` :408-433) and ``moe_unfused.py``
(``mxfp8_moe_experts_unfused`` :119-158).

forward   quantize x once per token -> GEMM1 (gather + both halves + SwiGLU + requantize)
          -> GEMM2 (gate scale + scatter-add into the zeroed output)
backward  quantize dout -> GEMM2-DGRAD (dgate, SwiGLU', dpre + requantize) -> GEMM1-DGRAD
          (scatter-add into dx) -> two MXFP8 WGRADs on token-axis blocks inside each expert
"""

from __future__ import annotations

import torch

from kohakuwullm_amd import _lib
from kohakuwullm_amd.kernels.moe.moe_dispatch import combine_routed
from kohakuwullm_amd.kernels.mxfp8.grouped import (
    grouped_mxfp8_gemm,
    grouped_mxfp8_wgrad,
    padded_rows,
    token_axis_buffers,
    token_axis_pitch,
    quantize_mx_cols_grouped,
)
from kohakuwullm_amd.kernels.mxfp8.quantize import BLOCK_SCALE, quantize_mx, quantize_mx_cols

_FP8 = torch.float8_e4m3fn
_ACT_DTYPES = (torch.bfloat16, torch.float16)
# The token-axis operands of the expert WGRADs (h, dpre, gathered x, gate-scaled dout) are written stage-major,
# (Mpad // 128, rows, 128): a K stage of a WGRAD tile is then one contiguous run instead of 256 rows ~100 KB apart.
TOKEN_AXIS_STAGE_MAJOR = True


def _quantize_stacked(w: torch.Tensor):
    """Quantize ``(E, N, K)`` row by row, keeping the expert axis.  Blocks along K."""
    e, n, k = w.shape
    q, s = quantize_mx(w.reshape(e * n, k))
    return q.view(e, n, k), s.view(e, n, k // BLOCK_SCALE)


def _quantize_stacked_t(w: torch.Tensor):
    """``_quantize_stacked(w.transpose(1, 2))`` without materialising the transpose: blocks along N.

    With ``N % 128 == 0`` the whole stack is one column-axis launch over ``(E*N, K)`` (32-row
    blocks never straddle two experts); the result ``(K, E*N)`` is viewed as ``(E, K, N)``, whose
    rows are ``E*N`` apart.  The kernels take the expert and row strides as given.
    """
    e, n, k = w.shape
    if n % 128 == 0 and w.is_contiguous():
        q, s = quantize_mx_cols(w.reshape(e * n, k))
        return q.view(k, e, n).permute(1, 0, 2), s.view(k, e, n // BLOCK_SCALE).permute(1, 0, 2)
    qs, ss = [], []
    for i in range(e):
        q, s = quantize_mx_cols(w[i])
        qs.append(q)
        ss.append(s)
    return torch.stack(qs), torch.stack(ss)


class MXFP8ExpertWeights:
    """The four fp8 copies of one MoE layer's expert matrices (not a module: nothing enters ``state_dict``)."""

    __slots__ = ("in_fwd", "in_dgrad", "out_fwd", "out_dgrad")

    def __init__(self, w_in: torch.Tensor | None = None, w_out: torch.Tensor | None = None) -> None:
        if w_in is not None:
            self.refresh(w_in, w_out)

    @torch.no_grad()
    def refresh(self, w_in: torch.Tensor, w_out: torch.Tensor) -> None:
        """Rebuild every copy from the 16-bit masters.  Call after each optimizer step."""
        self.in_fwd = _quantize_stacked(w_in)  # (E, 2H, dim), K = dim
        self.out_fwd = _quantize_stacked(w_out)  # (E, dim, H), K = H
        self.in_dgrad = _quantize_stacked_t(w_in)  # (E, dim, 2H), K = 2H
        self.out_dgrad = _quantize_stacked_t(w_out)  # (E, H, dim), K = dim

    @staticmethod
    def plan(w_in: torch.Tensor, w_out: torch.Tensor) -> list[torch.Tensor] | None:
        """The two stacks as ``(E*N, K)`` matrices whose dual quantization holds all four copies.

        ``None`` when a stack cannot be taken as one matrix (rows per expert not a multiple of
        128, or a non-contiguous stack): ``refresh`` is the way then.
        """
        for w in (w_in, w_out):
            if w.shape[1] % 128 or w.shape[2] % BLOCK_SCALE or not w.is_contiguous() or not w.is_cuda:
                return None
        return [w.detach().reshape(w.shape[0] * w.shape[1], w.shape[2]) for w in (w_in, w_out)]

    def install(self, copies, num_experts: int) -> None:
        """Take the dual quantizations of ``plan``'s matrices, viewed per expert as ``refresh`` lays them out."""
        views = []
        for q, s, qt, st in copies:
            en, k = q.shape
            n = en // num_experts
            views.append((q.view(num_experts, n, k), s.view(num_experts, n, k // BLOCK_SCALE)))
            views.append((qt.view(k, num_experts, n).permute(1, 0, 2),
                          st.view(k, num_experts, n // BLOCK_SCALE).permute(1, 0, 2)))
        self.in_fwd, self.in_dgrad, self.out_fwd, self.out_dgrad = views


def _w_args(wq, ws):
    return (wq.data_ptr(), ws.data_ptr(), wq.stride(0), wq.stride(1), ws.stride(0), ws.stride(1))


def launch_gemm1(xq, xs, token_of, wq, ws, hq, hs, pre, offsets, hidden, dim, act_dtype, htq=None, hts=None) -> None:
    """GEMM1 with its epilogue; ``token_of=None`` reads row m of ``xq`` for sorted row m.

    ``htq``/``hts`` ``(H, Mpad)``/``(H, Mpad//32)``, when given, receive ``h`` quantized along the tokens
    (``htq`` may be stage-major, ``(Mpad//128, H, 128)``).
    """
    m = hq.shape[0]
    _lib.invoke(
        "mx_experts_gemm1", 2.0 * m * 2 * hidden * dim, xq,
        xq.data_ptr(), xs.data_ptr(), xq.shape[0], xq.stride(0), xs.stride(0),
        0 if token_of is None else token_of.data_ptr(), *_w_args(wq, ws),
        offsets.data_ptr(), wq.shape[0], hq.data_ptr(), hq.stride(0), hs.data_ptr(), hs.stride(0),
        0 if pre is None else pre.data_ptr(), 0 if pre is None else pre.stride(0),
        0 if htq is None else htq.data_ptr(), 0 if htq is None else token_axis_pitch(htq),
        0 if hts is None else hts.data_ptr(), 0 if hts is None else hts.stride(0),
        _lib.MX_DTYPE[act_dtype], m, hidden, dim,
    )


def launch_scatter_gemm(aq, a_s, wq, ws, out, token_of, order, gate, offsets, index=None) -> None:
    m = token_of.numel()
    n, k = wq.shape[1], wq.shape[2]
    _lib.invoke(
        "mx_experts_scatter_gemm", 2.0 * m * n * k, aq,
        aq.data_ptr(), a_s.data_ptr(), aq.shape[0], aq.stride(0), a_s.stride(0), 0 if index is None else index.data_ptr(),
        *_w_args(wq, ws), offsets.data_ptr(), wq.shape[0], token_of.data_ptr(), 0 if order is None else order.data_ptr(),
        0 if gate is None else gate.data_ptr(), 0 if gate is None else _lib.MX_DTYPE[gate.dtype],
        out.data_ptr(), _lib.MX_DTYPE[out.dtype], out.stride(0), m, n, k,
    )


def combine_sorted_rows(y, order, offsets, num_experts, gate, tokens: int, top_k: int, positions=None,
                        return_positions: bool = False):
    """``out[t] = sum_k gate[t*top_k+k] * y[position of pair t*top_k+k]``: the scatter-add as a gather.

    ``order`` must be the pair index ``token * top_k + slot`` (what ``expert_sort`` produces).
    Deterministic; every row of the result is written.  ``positions``: the pair -> sorted position
    table an earlier call for the same routing returned (``return_positions=True``); with it the
    call skips rebuilding the table from ``order``.
    """
    m, n = y.shape
    out = torch.empty(tokens, n, device=y.device, dtype=y.dtype)
    reuse = positions is not None
    if reuse and (positions.numel() != tokens * top_k or positions.dtype != torch.int32 or positions.device != y.device):
        raise ValueError(f"positions {tuple(positions.shape)} {positions.dtype} does not fit {tokens} tokens x top_k {top_k}")
    inv = positions if reuse else torch.empty(tokens * top_k, device=y.device, dtype=torch.int32)
    _lib.invoke(
        "mx_experts_combine", y.element_size() * n * (tokens * top_k + tokens), y,
        y.data_ptr(), y.stride(0), 0 if reuse else order.data_ptr(), offsets.data_ptr(), num_experts,
        0 if gate is None else gate.data_ptr(), 0 if gate is None else _lib.MX_DTYPE[gate.dtype], inv.data_ptr(),
        tokens, top_k, out.data_ptr(), _lib.MX_DTYPE[out.dtype], out.stride(0), m, n,
    )
    return (out, inv) if return_positions else out


def _routed_product(aq, a_s, wq, ws, token_of, order, gate, offsets, tokens: int, top_k: int, dtype, positions=None,
                    return_positions: bool = False):
    """``out[token] += scale * (a[m] . w[e(m)]^T)`` over the sorted rows.

    When ``order`` is a pair index (``top_k`` > 0) the rows are written once by the grouped GEMM
    and gathered per token; otherwise the scatter GEMM adds them into a zeroed output with
    16-bit atomics, as the reference does.
    """
    n = wq.shape[1]
    if top_k > 0 and n % 8 == 0:
        y = grouped_mxfp8_gemm(aq, a_s, wq, ws, offsets, out_dtype=dtype, rows=token_of.numel())
        return combine_sorted_rows(y, order, offsets, wq.shape[0], gate, tokens, top_k, positions, return_positions)
    out = torch.zeros(tokens, n, device=aq.device, dtype=dtype)
    launch_scatter_gemm(aq, a_s, wq, ws, out, token_of, order if gate is not None else None, gate, offsets)
    return (out, None) if return_positions else out


def launch_gemm2_dgrad(dq, ds, token_of, order, gate, wq, ws, hq, hs, pre, dpre, dpq, dps, dgate, offsets,
                       ptq=None, pts=None) -> None:
    """DGRAD through GEMM2 with its epilogue.

    ``ptq``/``pts`` ``(2H, Mpad)``/``(2H, Mpad//32)``, when given, receive ``dpre`` quantized along the
    tokens; ``dpre`` may then be ``None``.
    """
    m = token_of.numel()
    hidden, dim = wq.shape[1], wq.shape[2]
    _lib.invoke(
        "mx_experts_gemm2_dgrad", 2.0 * m * hidden * dim, dq,
        dq.data_ptr(), ds.data_ptr(), dq.shape[0], dq.stride(0), ds.stride(0), token_of.data_ptr(), order.data_ptr(),
        gate.data_ptr(), _lib.MX_DTYPE[gate.dtype], *_w_args(wq, ws), offsets.data_ptr(), wq.shape[0],
        hq.data_ptr(), hq.stride(0), hs.data_ptr(), hs.stride(0), pre.data_ptr(),
        0 if dpre is None else dpre.data_ptr(), pre.stride(0),
        dpq.data_ptr(), dpq.stride(0), dps.data_ptr(), dps.stride(0),
        0 if ptq is None else ptq.data_ptr(), 0 if ptq is None else token_axis_pitch(ptq),
        0 if pts is None else pts.data_ptr(), 0 if pts is None else pts.stride(0),
        dgate.data_ptr(), _lib.MX_DTYPE[pre.dtype], m, hidden, dim,
    )


class _MXFP8Experts(torch.autograd.Function):
    @staticmethod
    def forward(ctx, x, w_in, w_out, gate, token_of, order, offsets, packed, hidden):
        del w_in, w_out  # present so autograd routes dW to the master parameters
        rows, dim = x.shape
        m = token_of.numel()
        # `ctx.needs_input_grad`, not `torch.is_grad_enabled()`: autograd runs forward under no_grad
        needs_grad = any(ctx.needs_input_grad)
        xq, xs = quantize_mx(x)  # once per token; the gather happens inside GEMM1
        hq = torch.empty(m, hidden, device=x.device, dtype=_FP8)
        hs = torch.empty(m, hidden // BLOCK_SCALE, device=x.device, dtype=torch.uint8)
        pre = torch.empty(m, 2 * hidden, device=x.device, dtype=x.dtype) if needs_grad else None
        htq = hts = None
        if ctx.needs_input_grad[2]:
            # h along the tokens, for dW_out: written by GEMM1's epilogue instead of a pass over `pre`
            mpad = padded_rows(m, packed.in_fwd[0].shape[0])
            htq, hts = token_axis_buffers(hidden, mpad, x.device, TOKEN_AXIS_STAGE_MAJOR)
        launch_gemm1(xq, xs, token_of, *packed.in_fwd, hq, hs, pre, offsets, hidden, dim, x.dtype, htq, hts)
        # pairs per token when `order` is the pair index token * top_k + slot; 0 = unknown layout
        top_k = gate.numel() // rows if rows and gate.numel() % rows == 0 else 0
        # the pair -> sorted position table of the combine serves the backward's combine too
        out, positions = _routed_product(hq, hs, *packed.out_fwd, token_of, order, gate, offsets, rows, top_k, x.dtype,
                                         return_positions=True)
        if needs_grad:
            ctx.positions = positions
            ctx.save_for_backward(x, hq, hs, pre, gate, token_of, order, offsets, htq, hts)
            ctx.packed = packed
            ctx.shapes = (hidden, dim, m, rows, top_k)
        return out

    @staticmethod
    def backward(ctx, dout):
        x, hq, hs, pre, gate, token_of, order, offsets, htq, hts = ctx.saved_tensors
        packed = ctx.packed
        hidden, dim, m, rows, top_k = ctx.shapes
        dev = dout.device
        dout = dout.contiguous()
        dq, ds = quantize_mx(dout)
        dpq = torch.empty(m, 2 * hidden, device=dev, dtype=_FP8)
        dps = torch.empty(m, 2 * hidden // BLOCK_SCALE, device=dev, dtype=torch.uint8)
        # fp32 and zeroed: this reduction crosses workgroups through an atomic
        dgate = torch.zeros(gate.numel(), device=dev, dtype=torch.float32)
        ptq = pts = None
        if ctx.needs_input_grad[1]:
            # dpre along the tokens, for dW_in: written by the epilogue; dpre itself never reaches memory
            mpad = padded_rows(m, packed.in_fwd[0].shape[0])
            ptq, pts = token_axis_buffers(2 * hidden, mpad, dev, TOKEN_AXIS_STAGE_MAJOR)
        dpre = None if ptq is not None else torch.empty(m, 2 * hidden, device=dev, dtype=dout.dtype)
        launch_gemm2_dgrad(dq, ds, token_of, order, gate, *packed.out_dgrad, hq, hs, pre, dpre, dpq, dps, dgate, offsets,
                           ptq, pts)
        dx = _routed_product(dpq, dps, *packed.in_dgrad, token_of, order, None, offsets, rows, top_k, dout.dtype,
                             positions=ctx.positions)

        dw_in = dw_out = None
        if ctx.needs_input_grad[2]:
            # dW_out[e] = (gate-scaled dout rows of e).T @ h rows of e; h is rebuilt from `pre`
            dtq, dts = quantize_mx_cols_grouped(dout, offsets, m, index=token_of, row_scale=gate, scale_index=order,
                                                stage_major=TOKEN_AXIS_STAGE_MAJOR)
            dw_out = grouped_mxfp8_wgrad(dtq, dts, htq, hts, offsets, m, dout.dtype)
        if ctx.needs_input_grad[1]:
            # dW_in[e] = dpre rows of e .T @ x rows of e
            xtq, xts = quantize_mx_cols_grouped(x, offsets, m, index=token_of, stage_major=TOKEN_AXIS_STAGE_MAJOR)
            dw_in = grouped_mxfp8_wgrad(ptq, pts, xtq, xts, offsets, m, dout.dtype)
        return dx, dw_in, dw_out, dgate.to(gate.dtype), None, None, None, None, None


def _validate_expert_call(x, w_in, w_out, token_of, order) -> int:
    """Shared contract of the fused and unfused entry points; returns ``hidden``.

    ``x`` must be unit-stride on its last axis and 16-bit; both are refused rather than repaired.
    """
    hidden = w_out.shape[2]
    if w_in.shape[1] != 2 * hidden:
        raise ValueError(f"w_in {tuple(w_in.shape)} is not 2x w_out's hidden {hidden}")
    if w_in.shape[2] != x.shape[1] or w_out.shape[1] != x.shape[1]:
        raise ValueError(f"width mismatch: x {tuple(x.shape)} vs {tuple(w_in.shape)}")
    for name, value in (("dim", x.shape[1]), ("hidden", hidden)):
        if value % BLOCK_SCALE:
            raise ValueError(f"{name}={value} must be a multiple of {BLOCK_SCALE}")
    if token_of.numel() != order.numel():
        raise ValueError(f"token_of {token_of.numel()} != order {order.numel()}")
    if x.stride(-1) != 1:
        raise ValueError(
            f"x must be contiguous along its last axis, got strides {x.stride()}; "
            "WGRAD indexes the contraction axis without a stride"
        )
    if x.dtype not in _ACT_DTYPES:
        raise ValueError(
            f"x.dtype={x.dtype} is not one of {_ACT_DTYPES}; the compute dtype is the caller's to choose"
        )
    return hidden


def mxfp8_moe_experts(x, w_in, w_out, gate, token_of, order, offsets, packed: MXFP8ExpertWeights) -> torch.Tensor:
    """The whole routed-expert path in MXFP8: gather, SwiGLU MLP, gate, combine.

    Args:
        x: ``(T, dim)`` activations, one row per token, **not** gathered.
        w_in: ``(E, 2H, dim)`` master weights.  Passed for the gradient only; the forward reads ``packed``.
        w_out: ``(E, dim, H)`` master weights, likewise.
        gate: ``(T*top_k,)`` gate weights indexed by pair index.
        token_of: ``(M,)`` int32, sorted position -> token index.
        order: ``(M,)`` int32, sorted position -> pair index.
        offsets: ``(E+1,)`` int32 exclusive prefix sum of per-expert row counts, truncated to the
            real experts, so a sentinel bucket's rows fall outside every tile.  Never read on the host.
        packed: the four quantized copies, refreshed after each optimizer step.
    """
    hidden = _validate_expert_call(x, w_in, w_out, token_of, order)
    return _MXFP8Experts.apply(x, w_in, w_out, gate, token_of, order, offsets, packed, hidden)


def mxfp8_moe_experts_reference(x, w_in, w_out, gate, token_of, order, offsets) -> torch.Tensor:
    """Autograd-composed equivalent in the input dtype, with no quantization (reads ``offsets`` on the host)."""
    rows = x.index_select(0, token_of.long())
    off = offsets.tolist()
    outs = []
    for e in range(w_in.shape[0]):
        block = rows[off[e] : off[e + 1]]
        gate_h, value = (block @ w_in[e].T).chunk(2, dim=-1)
        outs.append((torch.nn.functional.silu(gate_h) * value) @ w_out[e].T)
    sorted_out = torch.cat(outs, dim=0)
    real = sorted_out.shape[0]
    scaled = sorted_out * gate.index_select(0, order[:real].long()).reshape(-1, 1)
    out = torch.zeros(x.shape[0], x.shape[1], dtype=x.dtype, device=x.device)
    return out.index_add(0, token_of[:real].long(), scaled)


# ---------------------------------------------------------------------------------------------
# The unfused twin: the same arithmetic composed out of the grouped GEMM, for A/B runs.
# ---------------------------------------------------------------------------------------------


class _GroupedExpertMatmul(torch.autograd.Function):
    """``out[m] = x[index[m]] @ w[e(m)].T`` over expert-sorted rows, in MXFP8 (fwd, dgrad and wgrad)."""

    @staticmethod
    def forward(ctx, x, w, wq, ws, wtq, wts, offsets, index, sentinel):
        del w
        xq, xs = quantize_mx(x)
        rows = xq.shape[0] if index is None else index.numel()
        out = grouped_mxfp8_gemm(xq, xs, wq, ws, offsets, index=index, out_dtype=x.dtype,
                                 out=_maybe_zeros(sentinel, rows, wq.shape[1], x))
        if any(ctx.needs_input_grad):
            ctx.save_for_backward(x, wtq, wts, offsets, index)
            ctx.shape = wq.shape
            ctx.sentinel = sentinel
            ctx.rows = rows
        return out

    @staticmethod
    def backward(ctx, dout):
        x, wtq, wts, offsets, index = ctx.saved_tensors
        num_experts, n, k = ctx.shape
        dout = dout.contiguous()
        dx = dw = None
        if ctx.needs_input_grad[0]:
            dq, ds = quantize_mx(dout)
            dx_sorted = grouped_mxfp8_gemm(dq, ds, wtq, wts, offsets, out_dtype=dout.dtype,
                                           out=_maybe_zeros(ctx.sentinel, dout.shape[0], k, dout))
            dx = dx_sorted if index is None else torch.zeros_like(x).index_add_(0, index.long(), dx_sorted)
        if ctx.needs_input_grad[1]:
            dtq, dts = quantize_mx_cols_grouped(dout, offsets, ctx.rows, stage_major=TOKEN_AXIS_STAGE_MAJOR)
            xtq, xts = quantize_mx_cols_grouped(x, offsets, ctx.rows, index=index, stage_major=TOKEN_AXIS_STAGE_MAJOR)
            dw = grouped_mxfp8_wgrad(dtq, dts, xtq, xts, offsets, ctx.rows, dout.dtype)
        return dx, dw, None, None, None, None, None, None, None


def _maybe_zeros(sentinel: bool, rows: int, cols: int, like: torch.Tensor):
    """A zeroed ``(rows, cols)`` buffer when a sentinel bucket exists (its rows are never written), else ``None``."""
    if not sentinel:
        return None
    return torch.zeros(rows, cols, device=like.device, dtype=like.dtype)


def mxfp8_moe_experts_unfused(x, w_in, w_out, gate, token_of, order, offsets, packed: MXFP8ExpertWeights,
                              valid_rows=None) -> torch.Tensor:
    """The routed-expert path in MXFP8 as separate launches instead of the fused graph; same signature and arithmetic."""
    _validate_expert_call(x, w_in, w_out, token_of, order)
    sentinel = valid_rows is not None
    pre = _GroupedExpertMatmul.apply(x, w_in, *packed.in_fwd, *packed.in_dgrad, offsets, token_of, sentinel)
    gate_h, value = pre.chunk(2, dim=-1)
    h = torch.nn.functional.silu(gate_h) * value
    out_sorted = _GroupedExpertMatmul.apply(h, w_out, *packed.out_fwd, *packed.out_dgrad, offsets, None, sentinel)
    return combine_routed(out_sorted, gate, order, token_of, x.shape[0], valid_rows)
