"""MXFP8 quantizers and the pre-quantized GEMM, on hand-written gfx950 kernels.

Same names, arguments, return dtypes and errors as the reference module
``src/kohakuwullm/kernels/mxfp8/quantize.py`` (``quantize_mx`` :106-137,
``mxfp8_matmul_pq`` :328-371, ``mxfp8_matmul`` :433-473), plus the column-axis and
dual quantizers the MXFP8 wgrad needs (the reference realises the column axis as
``quantize_mx(x.t())``: ``linear.py:111``, ``moe.py:58-61``).

Block scales run along the contraction axis and the scale exponent rounds up.
Accumulation is fp32 always; the output dtype is the caller's.
"""

from __future__ import annotations

import ctypes

import torch

from kohakuwullm_amd import _lib

E4M3_MAX = 448.0
BLOCK_SCALE = 32

_FP8 = torch.float8_e4m3fn


def _check_2d(x: torch.Tensor, name: str) -> None:
    if x.dim() != 2:
        raise ValueError(f"{name} must be 2-D, got shape {tuple(x.shape)}")
    if x.dtype not in _lib.MX_DTYPE:
        raise ValueError(f"{name}.dtype={x.dtype} is not one of {tuple(_lib.MX_DTYPE)}")
    _lib.require_gpu(x, name)


def quantize_mx(x: torch.Tensor) -> tuple[torch.Tensor, torch.Tensor]:
    """``(M,K)`` -> ``(e4m3 (M,K), ue8m0 (M, K//32))``, blocks along the last axis.

    Bandwidth-bound.  ``K`` must be a multiple of 32.  Any strides are accepted; a
    transposed view is quantized in place of a copy (the column-axis kernel runs on
    the matrix underneath it).
    """
    if x.shape[-1] % BLOCK_SCALE:
        raise ValueError(f"K={x.shape[-1]} must be a multiple of {BLOCK_SCALE}")
    _check_2d(x, "x")
    m, k = x.shape
    q = torch.empty(m, k, device=x.device, dtype=_FP8)
    s = torch.empty(m, k // BLOCK_SCALE, device=x.device, dtype=torch.uint8)
    if m and k:
        _lib.invoke(
            "mx_quantize_rows", m * k * (x.element_size() + 1 + 1 / BLOCK_SCALE), x,
            x.data_ptr(), _lib.MX_DTYPE[x.dtype], m, k, x.stride(0), x.stride(1),
            q.data_ptr(), k, s.data_ptr(), k // BLOCK_SCALE,
        )
    return q, s


def quantize_mx_cols(x: torch.Tensor) -> tuple[torch.Tensor, torch.Tensor]:
    """``(M,K)`` -> ``(e4m3 (K,M), ue8m0 (K, M//32))``: blocks of 32 along ``M``.

    Equal, bit for bit, to ``quantize_mx(x.t().contiguous())`` without the copy.
    ``M`` must be a multiple of 32.
    """
    if x.shape[0] % BLOCK_SCALE:
        raise ValueError(f"M={x.shape[0]} must be a multiple of {BLOCK_SCALE}")
    _check_2d(x, "x")
    if x.stride(1) != 1:
        x = x.contiguous()
    m, k = x.shape
    qt = torch.empty(k, m, device=x.device, dtype=_FP8)
    st = torch.empty(k, m // BLOCK_SCALE, device=x.device, dtype=torch.uint8)
    if m and k:
        _lib.invoke(
            "mx_quantize_cols", m * k * (x.element_size() + 1 + 1 / BLOCK_SCALE), x,
            x.data_ptr(), _lib.MX_DTYPE[x.dtype], m, k, x.stride(0),
            qt.data_ptr(), m, st.data_ptr(), m // BLOCK_SCALE,
        )
    return qt, st


PANEL = 128  # columns per panel of the stage-major code layout


def stage_major_ok(cols: int) -> bool:
    """Whether a code matrix with ``cols`` columns can be stored stage-major (whole 128-column panels)."""
    return cols % PANEL == 0 and cols > 0


def rows_of_stage_major(codes: torch.Tensor) -> torch.Tensor:
    """The ``(rows, cols)`` matrix a stage-major ``(cols // 128, rows, 128)`` code tensor holds (a copy)."""
    panels, rows, width = codes.shape
    return codes.permute(1, 0, 2).reshape(rows, panels * width)


def quantize_mx_dual(x: torch.Tensor, stage_major_t: bool = False):
    """Row- and column-axis quantization of ``x`` in one pass over it.

    Returns ``(q, s, qT, sT)`` with ``(q, s) == quantize_mx(x)`` and
    ``(qT, sT) == quantize_mx_cols(x)``.  Both ``M`` and ``K`` must be multiples of 32.

    ``stage_major_t``: ``qT`` comes back as ``(M // 128, K, 128)`` -- 128-token panels, each holding
    every row -- instead of ``(K, M)``; the GEMM wrappers take either.  A WGRAD tile then reads
    each of its K stages as one contiguous run (a few percent faster on long contractions).
    ``M`` must be a multiple of 128.
    """
    if x.shape[-1] % BLOCK_SCALE or x.shape[0] % BLOCK_SCALE:
        raise ValueError(f"shape {tuple(x.shape)}: both axes must be multiples of {BLOCK_SCALE}")
    _check_2d(x, "x")
    if x.stride(1) != 1:
        x = x.contiguous()
    m, k = x.shape
    if stage_major_t and not stage_major_ok(m):
        raise ValueError(f"stage_major_t needs M={m} to be a positive multiple of {PANEL}")
    q = torch.empty(m, k, device=x.device, dtype=_FP8)
    s = torch.empty(m, k // BLOCK_SCALE, device=x.device, dtype=torch.uint8)
    qt = torch.empty((m // PANEL, k, PANEL) if stage_major_t else (k, m), device=x.device, dtype=_FP8)
    st = torch.empty(k, m // BLOCK_SCALE, device=x.device, dtype=torch.uint8)
    if m and k:
        _lib.invoke(
            "mx_quantize_dual", m * k * (x.element_size() + 2 * (1 + 1 / BLOCK_SCALE)), x,
            x.data_ptr(), _lib.MX_DTYPE[x.dtype], m, k, x.stride(0),
            q.data_ptr(), k, s.data_ptr(), k // BLOCK_SCALE,
            qt.data_ptr(), PANEL if stage_major_t else m, st.data_ptr(), m // BLOCK_SCALE,
        )
    return q, s, qt, st


def quantize_mx_dual_batch(xs: list[torch.Tensor]) -> list[tuple[torch.Tensor, torch.Tensor, torch.Tensor, torch.Tensor]]:
    """``quantize_mx_dual`` of every matrix of ``xs`` behind one launch per 24 matrices.

    For the once-per-optimizer-step requantization of a model's weights, where a launch and four
    allocations per matrix cost more than the bytes moved.  The matrices must share device and
    dtype; the codes of one call are views of one allocation, the scale bytes of another.  Same
    bytes as ``quantize_mx_dual`` on each.
    """
    if not xs:
        return []
    for x in xs:
        _check_2d(x, "x")
        if x.shape[0] % BLOCK_SCALE or x.shape[1] % BLOCK_SCALE:
            raise ValueError(f"shape {tuple(x.shape)}: both axes must be multiples of {BLOCK_SCALE}")
        if x.device != xs[0].device or x.dtype != xs[0].dtype:
            raise ValueError("quantize_mx_dual_batch: the matrices must share one device and one dtype")
    xs = [x if x.stride(1) == 1 else x.contiguous() for x in xs]
    # sizes are multiples of 1024 (codes) and 32 (scale bytes): every piece starts 16-byte aligned
    n_codes = [x.shape[0] * x.shape[1] for x in xs]
    n_scales = [n // BLOCK_SCALE for n in n_codes]
    codes = torch.empty(2 * sum(n_codes), device=xs[0].device, dtype=_FP8)
    scales = torch.empty(2 * sum(n_scales), device=xs[0].device, dtype=torch.uint8)
    code_views = codes.split_with_sizes([n for n in n_codes for _ in (0, 1)])
    scale_views = scales.split_with_sizes([n for n in n_scales for _ in (0, 1)])
    problems = (_lib.QuantProblem * len(xs))()
    out, at_code, at_scale, work = [], codes.data_ptr(), scales.data_ptr(), 0.0
    for j, x in enumerate(xs):
        m, k = x.shape
        kb, mb = k // BLOCK_SCALE, m // BLOCK_SCALE
        problems[j] = _lib.QuantProblem(x.data_ptr(), at_code, at_scale, at_code + n_codes[j], at_scale + n_scales[j],
                                        m, k, x.stride(0), k, kb, m, mb)
        out.append((code_views[2 * j].view(m, k), scale_views[2 * j].view(m, kb),
                    code_views[2 * j + 1].view(k, m), scale_views[2 * j + 1].view(k, mb)))
        at_code += 2 * n_codes[j]
        at_scale += 2 * n_scales[j]
        work += n_codes[j] * (x.element_size() + 2 * (1 + 1 / BLOCK_SCALE))
    if codes.numel():
        _lib.invoke("mx_quantize_dual_batch", work, xs[0], ctypes.byref(problems), len(xs), _lib.MX_DTYPE[xs[0].dtype])
    return out


def _gemm_nt_into(aq, a_scale, bq, b_scale, out) -> None:
    m, k = aq.shape
    n = bq.shape[0]
    ws = _lib.gemm_workspace(aq)
    _lib.invoke(
        "mx_gemm_nt", 2.0 * m * n * k, aq,
        aq.data_ptr(), a_scale.data_ptr(), bq.data_ptr(), b_scale.data_ptr(), out.data_ptr(),
        _lib.MX_DTYPE[out.dtype], m, n, k, aq.stride(0), a_scale.stride(0), bq.stride(0), b_scale.stride(0),
        out.stride(0), 0, ws.data_ptr(), ws.numel(),
    )


def mxfp8_matmul_pq(
    aq: torch.Tensor,
    a_scale: torch.Tensor,
    bq: torch.Tensor,
    b_scale: torch.Tensor,
    out_dtype: torch.dtype = torch.bfloat16,
    out_pad: int = 0,
) -> torch.Tensor:
    """``aq @ bq.T`` from pre-quantized operands, fp32 accumulate.

    ``aq (M,K)``, ``bq (N,K)`` e4m3 and ``a_scale (M,K//32)``, ``b_scale (N,K//32)``
    ue8m0 in the natural layout ``quantize_mx`` produces.  Needs only ``K % 32 == 0``.
    A 3-D ``(K // 128, rows, 128)`` code tensor is a stage-major operand (``quantize_mx_dual``).
    ``out_pad``: the result is a view of an allocation with that many spare elements per row (a row
    pitch of ``N + out_pad``), for callers that know what pitch suits the kernel reading it next.
    """
    if out_pad < 0:
        raise ValueError(f"out_pad={out_pad} must not be negative")
    if aq.dim() == 3 or bq.dim() == 3:
        return mxfp8_matmul_pq_batch([(aq, a_scale, bq, b_scale)], out_dtype)[0]
    if aq.dim() != 2 or bq.dim() != 2 or aq.shape[1] != bq.shape[1]:
        raise ValueError(f"contraction mismatch: {tuple(aq.shape)} @ {tuple(bq.shape)}.T")
    m, k = aq.shape
    n = bq.shape[0]
    if k % BLOCK_SCALE:
        raise ValueError(f"K={k} must be a multiple of {BLOCK_SCALE}")
    if a_scale.shape != (m, k // BLOCK_SCALE) or b_scale.shape != (n, k // BLOCK_SCALE):
        raise ValueError(
            f"scale shapes {tuple(a_scale.shape)}, {tuple(b_scale.shape)} do not match operands "
            f"{tuple(aq.shape)}, {tuple(bq.shape)}"
        )
    if out_dtype not in _lib.MX_DTYPE:
        raise ValueError(f"out_dtype={out_dtype} is not one of {tuple(_lib.MX_DTYPE)}")
    _lib.require_gpu(aq, "aq")
    tensors = []
    for t in (aq, a_scale, bq, b_scale):
        if t.element_size() != 1:
            raise ValueError(f"codes and scales must be 1-byte tensors, got {t.dtype}")
        tensors.append(t if t.stride(1) == 1 else t.contiguous())
    out = torch.empty(m, n + out_pad, device=aq.device, dtype=out_dtype)[:, :n]
    if m and n:
        _gemm_nt_into(*tensors, out)
    return out


def mxfp8_matmul_pq_batch(problems, out_dtype: torch.dtype = torch.bfloat16) -> list[torch.Tensor]:
    """``[aq @ bq.T for (aq, a_scale, bq, b_scale) in problems]`` behind as few launches as possible.

    For products that are ready together and do not fill the GPU one by one (DGRAD and WGRAD
    of one layer): the library divides the GPU among them instead of running them in turn.
    Same operand contract and same results as :func:`mxfp8_matmul_pq`.
    """
    if out_dtype not in _lib.MX_DTYPE:
        raise ValueError(f"out_dtype={out_dtype} is not one of {tuple(_lib.MX_DTYPE)}")
    if not problems:
        return []
    descs = (_lib.GemmProblem * len(problems))()
    outs, keep, flops = [], [], 0.0
    for d, (aq, a_scale, bq, b_scale) in zip(descs, problems):
        # a 3-D operand (K // 128, rows, 128) is a stage-major code matrix (quantize_mx_dual(..., stage_major_t=True))
        shape_a = (aq.shape[1], aq.shape[0] * PANEL) if aq.dim() == 3 and aq.shape[2] == PANEL else tuple(aq.shape)
        shape_b = (bq.shape[1], bq.shape[0] * PANEL) if bq.dim() == 3 and bq.shape[2] == PANEL else tuple(bq.shape)
        if len(shape_a) != 2 or len(shape_b) != 2 or shape_a[1] != shape_b[1]:
            raise ValueError(f"contraction mismatch: {tuple(aq.shape)} @ {tuple(bq.shape)}.T")
        m, k = shape_a
        n = shape_b[0]
        if k % BLOCK_SCALE:
            raise ValueError(f"K={k} must be a multiple of {BLOCK_SCALE}")
        if a_scale.shape != (m, k // BLOCK_SCALE) or b_scale.shape != (n, k // BLOCK_SCALE):
            raise ValueError(
                f"scale shapes {tuple(a_scale.shape)}, {tuple(b_scale.shape)} do not match operands "
                f"{tuple(aq.shape)}, {tuple(bq.shape)}"
            )
        _lib.require_gpu(aq, "aq")
        ts = []
        for t in (aq, a_scale, bq, b_scale):
            if t.element_size() != 1:
                raise ValueError(f"codes and scales must be 1-byte tensors, got {t.dtype}")
            if t.dim() == 3:
                ts.append(t.contiguous())
            else:
                ts.append(t if t.stride(1) == 1 else t.contiguous())
        out = torch.empty(m, n, device=aq.device, dtype=out_dtype)
        keep.append(ts)
        outs.append(out)
        flops += 2.0 * m * n * k
        d.aq, d.a_scale, d.bq, d.b_scale, d.c = (t.data_ptr() for t in (*ts, out))
        d.M, d.N, d.K = m, n, k
        d.lda = PANEL if ts[0].dim() == 3 else ts[0].stride(0)
        d.ldb = PANEL if ts[2].dim() == 3 else ts[2].stride(0)
        d.ldas, d.ldbs, d.ldc = ts[1].stride(0), ts[3].stride(0), n
    ws = _lib.gemm_workspace(outs[0])
    _lib.invoke("mx_gemm_nt_batch", flops, outs[0], ctypes.addressof(descs), len(problems), _lib.MX_DTYPE[out_dtype],
                ws.data_ptr(), ws.numel())
    return outs


def mxfp8_matmul(a: torch.Tensor, b: torch.Tensor, out_dtype: torch.dtype | None = None) -> torch.Tensor:
    """``a @ b.T`` in MXFP8 with fp32 accumulation: quantize both, then multiply.

    Args:
        a: ``(M, K)`` activations in fp16/bf16.
        b: ``(N, K)`` weights in fp16/bf16, K-minor as a linear layer stores them.
        out_dtype: output dtype; defaults to ``a``'s.
    """
    if a.shape[-1] != b.shape[-1]:
        raise ValueError(f"contraction mismatch: {a.shape} @ {b.shape}.T")
    if a.shape[-1] % BLOCK_SCALE:
        raise ValueError(f"K={a.shape[-1]} must be a multiple of {BLOCK_SCALE}")
    aq, a_scale = quantize_mx(a)
    bq, b_scale = quantize_mx(b)
    return mxfp8_matmul_pq(aq, a_scale, bq, b_scale, out_dtype or a.dtype)
