"""Grouped MXFP8 GEMM: block-scaled fp8 with a variable row count per expert, and its WGRAD.

Function-for-function counterpart of the reference's
``src/kohakuwullm/kernels/mxfp8/grouped.py`` (``grouped_mxfp8_gemm`` :254-327,
``grouped_mxfp8_reference`` :330-350, WGRAD :152-247).  ``offsets`` stays on the device and is
never read on the host: the launch is bounded from host-known ``M`` and ``E`` alone.

WGRAD here is MXFP8 as well (the reference multiplies in 16 bits): both operands are
quantized along the token axis inside each expert's segment by ``quantize_mx_cols_grouped`` and
contracted by ``grouped_mxfp8_wgrad``.
"""

from __future__ import annotations

import torch

from kohakuwullm_amd import _lib
from kohakuwullm_amd.kernels.mxfp8.quantize import BLOCK_SCALE

_FP8 = torch.float8_e4m3fn
WGRAD_ROW_TILE = 128  # an expert's rows start on a multiple of this in the padded token axis
SCALE_ROW_SLACK = 16  # spare bytes behind each token-axis scale row (see token_axis_buffers)


def _check_offsets(offsets: torch.Tensor, num_experts: int) -> None:
    if offsets.dtype != torch.int32 or offsets.numel() != num_experts + 1 or not offsets.is_contiguous():
        raise ValueError(f"offsets must be a contiguous int32 ({num_experts + 1},) tensor, got {offsets.dtype} {tuple(offsets.shape)}")


def _check_index(index, name: str) -> None:
    if index is not None and (index.dtype != torch.int32 or not index.is_contiguous()):
        raise ValueError(f"{name} must be a contiguous int32 tensor")


def grouped_mxfp8_gemm(
    xq: torch.Tensor,
    x_scale: torch.Tensor,
    wq: torch.Tensor,
    w_scale: torch.Tensor,
    offsets: torch.Tensor,
    index: torch.Tensor | None = None,
    out_dtype: torch.dtype = torch.bfloat16,
    rows: int | None = None,
    out: torch.Tensor | None = None,
) -> torch.Tensor:
    """``out[m] = xq[index[m]] @ wq[e(m)].T`` for expert-sorted rows, in MXFP8.

    Args:
        xq / x_scale: ``(R, K)`` e4m3 and ``(R, K//32)`` ue8m0, blocks along K.
        wq / w_scale: ``(E, N, K)`` e4m3 and ``(E, N, K//32)`` ue8m0.
        offsets: ``(E+1,)`` int32 exclusive prefix sum of per-expert row counts.  Never read on the host.
        index: ``(M,)`` int32 source row per sorted position, or ``None`` for the identity.
        rows: output row count ``M`` when it differs from ``xq``'s / ``index``'s.
        out: destination, or ``None`` to allocate.  Pass a zeroed buffer when a sentinel bucket
            leaves rows outside every expert's range: those rows are not written.
    """
    num_experts, n, k = wq.shape
    if k % BLOCK_SCALE:
        raise ValueError(f"K={k} must be a multiple of {BLOCK_SCALE}")
    if w_scale.shape != (num_experts, n, k // BLOCK_SCALE):
        raise ValueError(f"w_scale {tuple(w_scale.shape)} does not match {wq.shape}")
    if xq.shape[1] != k:
        raise ValueError(f"contraction mismatch: xq {tuple(xq.shape)} vs K={k}")
    if x_scale.shape != (xq.shape[0], k // BLOCK_SCALE):
        raise ValueError(f"x_scale {tuple(x_scale.shape)} does not match {tuple(xq.shape)}")
    _check_offsets(offsets, num_experts)
    _check_index(index, "index")
    m = xq.shape[0] if index is None else index.numel()
    if rows is not None:
        m = rows
    if out is None:
        out = torch.empty(m, n, device=xq.device, dtype=out_dtype)
    elif out.shape != (m, n):
        raise ValueError(f"out {tuple(out.shape)} does not match ({m}, {n})")
    _lib.require_gpu(xq, "xq")
    if wq.stride(2) != 1 or w_scale.stride(2) != 1 or xq.stride(1) != 1 or x_scale.stride(1) != 1 or out.stride(1) != 1:
        raise ValueError("operands must be contiguous along their last axis")
    if m and n:
        _lib.invoke(
            "mx_grouped_gemm_nt", 2.0 * m * n * k, xq,
            xq.data_ptr(), x_scale.data_ptr(), xq.shape[0], xq.stride(0), x_scale.stride(0),
            0 if index is None else index.data_ptr(),
            wq.data_ptr(), w_scale.data_ptr(), wq.stride(0), wq.stride(1), w_scale.stride(0), w_scale.stride(1),
            offsets.data_ptr(), num_experts, out.data_ptr(), _lib.MX_DTYPE[out.dtype], out.stride(0), m, n, k,
        )
    return out


def grouped_mxfp8_reference(xq, x_scale, wq, w_scale, offsets, index=None) -> torch.Tensor:
    """Per-expert fp64 matmul on dequantized operands: the precision oracle (reads ``offsets`` on the host)."""
    scale = torch.exp2(x_scale.double() - 127.0).repeat_interleave(BLOCK_SCALE, dim=-1)
    xd = xq.double() * scale
    if index is not None:
        xd = xd.index_select(0, index.long())
    off = offsets.tolist()
    outs = []
    for e in range(wq.shape[0]):
        ws = torch.exp2(w_scale[e].double() - 127.0).repeat_interleave(BLOCK_SCALE, dim=-1)
        outs.append(xd[off[e] : off[e + 1]] @ (wq[e].double() * ws).T)
    return torch.cat(outs, dim=0)


def padded_rows(rows: int, num_experts: int) -> int:
    """Length of the padded token axis the grouped token-axis quantizer writes."""
    return (-(-rows // WGRAD_ROW_TILE) + num_experts) * WGRAD_ROW_TILE


# Extra bytes in the row pitch of the token-axis code buffers, see `token_axis_buffers`.
TOKEN_PITCH_PAD = 0


def token_axis_buffers(cols: int, mpad: int, device, stage_major: bool = False):
    """``(cols, mpad)`` codes and ``(cols, mpad // 32)`` scales for a token-axis quantization, as views of wider rows.

    ``stage_major``: the codes as ``(mpad // 128, cols, 128)`` instead -- the 128 positions of a K stage of every row
    together, so that a tile of the expert WGRAD reads one contiguous run per stage (measured on 98304 routed rows:
    the two WGRAD calls of a step 4 % faster).  Scales stay ``(cols, mpad // 32)``.
    """
    pitch = mpad + TOKEN_PITCH_PAD
    if stage_major:
        qt = torch.empty(mpad // WGRAD_ROW_TILE, cols, WGRAD_ROW_TILE, device=device, dtype=_FP8)
    else:
        qt = torch.empty(cols, pitch, device=device, dtype=_FP8)[:, :mpad]
    # 16 spare bytes behind every scale row: the expert WGRAD then fetches a row's scales 16 bytes at a
    # time from wherever an expert's token range starts (it may read 12 bytes past the row's last stage)
    st = torch.empty(cols, mpad // BLOCK_SCALE + SCALE_ROW_SLACK, device=device, dtype=torch.uint8)[:, : mpad // BLOCK_SCALE]
    return qt, st


def token_axis_pitch(qt: torch.Tensor) -> int:
    """The leading dimension to hand the library for token-axis codes: the row pitch, or 128 for the stage-major form."""
    if qt.dim() == 3:
        if qt.shape[2] != WGRAD_ROW_TILE or not qt.is_contiguous():
            raise ValueError(f"stage-major token-axis codes are contiguous (Mpad//128, C, 128), got {tuple(qt.shape)}")
        return WGRAD_ROW_TILE
    return qt.stride(0)


def quantize_mx_cols_grouped(
    x: torch.Tensor,
    offsets: torch.Tensor,
    rows: int,
    index: torch.Tensor | None = None,
    row_scale: torch.Tensor | None = None,
    scale_index: torch.Tensor | None = None,
    swiglu: bool = False,
    stage_major: bool = False,
):
    """Token-axis MXFP8 of expert-sorted rows: ``(C, Mpad)`` codes and ``(C, Mpad//32)`` scales.

    ``stage_major``: the codes as ``(Mpad // 128, C, 128)`` (see :func:`token_axis_buffers`); same bytes.

    Sorted position ``m`` (``m < rows``) takes row ``x[index[m] or m]``, optionally times
    ``row_scale[scale_index[m] or m]``; with ``swiglu`` the row is ``silu(x[:, :C]) * x[:, C:]``.
    Expert ``e``'s rows start at padded position ``128 * (tiles of the experts before it)``
    and are zero-padded to a multiple of 128, so no 32-row block mixes two experts.
    """
    num_experts = offsets.numel() - 1
    _check_offsets(offsets, num_experts)
    _check_index(index, "index")
    _check_index(scale_index, "scale_index")
    if x.dim() != 2 or x.stride(1) != 1 or x.dtype not in (torch.bfloat16, torch.float16):
        raise ValueError(f"x must be a 16-bit matrix contiguous along its last axis, got {x.dtype} {tuple(x.shape)}")
    _lib.require_gpu(x, "x")
    cols = x.shape[1] // 2 if swiglu else x.shape[1]
    mpad = padded_rows(rows, num_experts)
    qt, st = token_axis_buffers(cols, mpad, x.device, stage_major)
    scale_dt = 0 if row_scale is None else _lib.MX_DTYPE[row_scale.dtype]
    _lib.invoke(
        "mx_quantize_cols_grouped", rows * cols * ((4 if swiglu else 2) + 1 + 1 / BLOCK_SCALE), x,
        x.data_ptr(), _lib.MX_DTYPE[x.dtype], x.stride(0), cols, 1 if swiglu else 0,
        0 if index is None else index.data_ptr(), 0 if row_scale is None else row_scale.data_ptr(), scale_dt,
        0 if scale_index is None else scale_index.data_ptr(), offsets.data_ptr(), num_experts, rows,
        qt.data_ptr(), token_axis_pitch(qt), st.data_ptr(), st.stride(0),
    )
    return qt, st


def grouped_mxfp8_wgrad(atq, ats, btq, bts, offsets, rows: int, out_dtype=torch.bfloat16) -> torch.Tensor:
    """``dW[e] = A[rows(e)].T @ B[rows(e)]`` from the token-axis quantizations of A ``(N, Mpad)`` and B ``(K, Mpad)``.

    Either operand's codes may be stage-major, ``(Mpad // 128, N, 128)`` (see :func:`token_axis_buffers`).
    Returns ``(E, N, K)``; an expert without rows gets zeros.
    """
    num_experts = offsets.numel() - 1
    n, k = ats.shape[0], bts.shape[0]
    mpad = padded_rows(rows, num_experts)
    for name, q, r in (("A", atq, n), ("B", btq, k)):
        ok = q.shape == (mpad // WGRAD_ROW_TILE, r, WGRAD_ROW_TILE) if q.dim() == 3 else q.shape == (r, mpad)
        if not ok:
            raise ValueError(f"operand {name} must span {r} rows of the padded token axis {mpad}, got {tuple(q.shape)}")
    dw = torch.empty(num_experts, n, k, device=atq.device, dtype=out_dtype)
    ws = _lib.gemm_workspace(atq)
    _lib.invoke(
        "mx_grouped_wgrad_nt", 2.0 * rows * n * k, atq,
        atq.data_ptr(), ats.data_ptr(), token_axis_pitch(atq), ats.stride(0), btq.data_ptr(), bts.data_ptr(),
        token_axis_pitch(btq), bts.stride(0), offsets.data_ptr(), num_experts, rows, dw.data_ptr(), _lib.MX_DTYPE[out_dtype],
        dw.stride(0), dw.stride(1), n, k, ws.data_ptr(), ws.numel(),
    )
    return dw
