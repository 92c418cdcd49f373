"""CPU oracle for the MXFP8 linear path.  TEST INFRASTRUCTURE ONLY.

Python face of ``mx_oracle.c`` (the scalar restatement of the quantizer) plus the
dequantize-then-matmul definitions every GEMM of the path is judged against.  Only
``tests/``, the smoke entry and the ``cpu_baseline`` leg of ``bench.py`` may import
this module; the product package never does.

Reference lines followed (paths relative to the reference tree):

* quantizer ............... ``src/kohakuwullm/kernels/mxfp8/quantize.py:39-56,106-137``
* dequantize .............. ``src/kohakuwullm/kernels/mxfp8/grouped.py:51-62``
* dense / grouped oracle .. ``src/kohakuwullm/kernels/mxfp8/grouped.py:330-350``
* grouped WGRAD semantics . ``src/kohakuwullm/kernels/mxfp8/grouped.py:152-247``
* expert path ............. ``src/kohakuwullm/kernels/mxfp8/experts.py:57-135,166-222``,
  ``src/kohakuwullm/kernels/mxfp8/experts_bwd.py:67-164,193-247``,
  ``src/kohakuwullm/kernels/mxfp8/moe.py:408-433``
* error metrics ........... ``src/kohakuwullm/bench/core/timing.py:201-228``
* expert sort (CPU) ....... ``src/kohakuwullm/kernels/moe/moe_dispatch.py:264-282``
* attention operand ....... ``src/kohakuwullm/kernels/mxfp8/attention_quant.py:17-118``
* expert counts, combine .. ``src/kohakuwullm/models/components/moe.py:38-46``,
  ``src/kohakuwullm/kernels/moe/moe_dispatch.py:60-131,203-220``
* RMSNorm -> MXFP8 ........ ``src/kohakuwullm/kernels/elementwise/rmsnorm.py:20-128``,
  ``src/kohakuwullm/kernels/mxfp8/fused_act.py:104-143``

All tensors are CPU tensors.  Codes travel as ``torch.uint8`` (bit patterns of
``float8_e4m3fn``) unless stated otherwise.
"""

from __future__ import annotations

import ctypes
import os
import subprocess

import torch

BLOCK_SCALE = 32
E4M3_MAX = 448.0

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "libmx_oracle.so")
_DT = {torch.bfloat16: 0, torch.float16: 1, torch.float32: 2}


def build() -> str:
    """Compile ``mx_oracle.c`` with gcc (idempotent)."""
    subprocess.run(["make", "-C", _HERE, "-s"], check=True)
    return _LIB_PATH


def _load() -> ctypes.CDLL:
    if not os.path.exists(_LIB_PATH):
        build()
    lib = ctypes.CDLL(_LIB_PATH)
    i64, p, ci = ctypes.c_int64, ctypes.c_void_p, ctypes.c_int
    lib.ora_quantize_rows.argtypes = [p, ci, i64, i64, i64, i64, p, i64, p, i64]
    lib.ora_quantize_rows.restype = ci
    lib.ora_quantize_cols.argtypes = [p, ci, i64, i64, i64, i64, p, i64, p, i64]
    lib.ora_quantize_cols.restype = ci
    lib.ora_swiglu_quantize_rows.argtypes = [p, p, ci, i64, i64, i64, i64, p, i64, p, i64]
    lib.ora_swiglu_quantize_rows.restype = ci
    lib.ora_dequant.argtypes = [p, i64, p, i64, i64, i64, p, i64]
    lib.ora_dequant.restype = None
    lib.ora_gemm_nt_f64.argtypes = [p, i64, p, i64, p, i64, p, i64, i64, i64, i64, p, i64]
    lib.ora_gemm_nt_f64.restype = None
    lib.ora_swizzle_32_4_4.argtypes = [p, i64, i64, i64, p]
    lib.ora_swizzle_32_4_4.restype = None
    lib.ora_e4m3_from_f32.argtypes = [ctypes.c_float]
    lib.ora_e4m3_from_f32.restype = ctypes.c_uint8
    lib.ora_e4m3_to_f32.argtypes = [ctypes.c_uint8]
    lib.ora_e4m3_to_f32.restype = ctypes.c_float
    lib.ora_scale_byte.argtypes = [ctypes.c_float]
    lib.ora_scale_byte.restype = ctypes.c_uint8
    lib.ora_scale_byte_literal.argtypes = [ctypes.c_float]
    lib.ora_scale_byte_literal.restype = ctypes.c_uint8
    lib.ora_bf16_from_f32.argtypes = [ctypes.c_float]
    lib.ora_bf16_from_f32.restype = ctypes.c_uint16
    return lib


_lib: ctypes.CDLL | None = None


def lib() -> ctypes.CDLL:
    global _lib
    if _lib is None:
        _lib = _load()
    return _lib


# --------------------------------------------------------------------------- quantizer


def quantize_rows(x: torch.Tensor) -> tuple[torch.Tensor, torch.Tensor]:
    """``(M,K)`` -> codes ``(M,K)`` uint8, scales ``(M,K//32)`` uint8; blocks along K.

    Accepts any strides (the C loop takes both).  ``K % 32`` -> ValueError, like
    ``quantize.py:111-112``.
    """
    if x.dim() != 2 or x.dtype not in _DT:
        raise ValueError(f"expected a 2-D bf16/fp16/fp32 tensor, got {tuple(x.shape)} {x.dtype}")
    m, k = x.shape
    if k % BLOCK_SCALE:
        raise ValueError(f"K={k} must be a multiple of {BLOCK_SCALE}")
    q = torch.empty(m, k, dtype=torch.uint8)
    s = torch.empty(m, k // BLOCK_SCALE, dtype=torch.uint8)
    rc = lib().ora_quantize_rows(
        x.data_ptr(), _DT[x.dtype], m, k, x.stride(0), x.stride(1), q.data_ptr(), k, s.data_ptr(), k // BLOCK_SCALE
    )
    assert rc == 0
    return q, s


def quantize_cols(x: torch.Tensor) -> tuple[torch.Tensor, torch.Tensor]:
    """``(M,K)`` -> codes ``(K,M)``, scales ``(K,M//32)``; blocks of 32 along M."""
    if x.dim() != 2 or x.dtype not in _DT:
        raise ValueError(f"expected a 2-D bf16/fp16/fp32 tensor, got {tuple(x.shape)} {x.dtype}")
    m, k = x.shape
    if m % BLOCK_SCALE:
        raise ValueError(f"M={m} must be a multiple of {BLOCK_SCALE}")
    q = torch.empty(k, m, dtype=torch.uint8)
    s = torch.empty(k, m // BLOCK_SCALE, dtype=torch.uint8)
    rc = lib().ora_quantize_cols(
        x.data_ptr(), _DT[x.dtype], m, k, x.stride(0), x.stride(1), q.data_ptr(), m, s.data_ptr(), m // BLOCK_SCALE
    )
    assert rc == 0
    return q, s


def swiglu_quantize_rows(gate: torch.Tensor, up: torch.Tensor) -> tuple[torch.Tensor, torch.Tensor]:
    """``quantize_rows(silu(gate) * up)`` with the product kept in fp32 (fused_act.py:44-56)."""
    if gate.shape != up.shape:
        raise ValueError(f"gate {tuple(gate.shape)} != up {tuple(up.shape)}")
    m, k = gate.shape
    if k % BLOCK_SCALE:
        raise ValueError(f"K={k} must be a multiple of {BLOCK_SCALE}")
    assert gate.stride(1) == 1 and up.stride(1) == 1 and gate.dtype == up.dtype
    q = torch.empty(m, k, dtype=torch.uint8)
    s = torch.empty(m, k // BLOCK_SCALE, dtype=torch.uint8)
    rc = lib().ora_swiglu_quantize_rows(
        gate.data_ptr(), up.data_ptr(), _DT[gate.dtype], m, k, gate.stride(0), up.stride(0),
        q.data_ptr(), k, s.data_ptr(), k // BLOCK_SCALE,
    )
    assert rc == 0
    return q, s


def quantize_heads(x: torch.Tensor, mu: torch.Tensor | None = None):
    """``(T, H, D)`` -> codes ``(T, H, D)`` uint8, scales ``(T, H, D // 32)``; blocks along D (attention_quant.py:17-118).

    ``mu`` ``(H, D)`` fp32 is subtracted in fp32 before the block maximum is taken.
    """
    t, h, d = x.shape
    y = x.float() if mu is None else x.float() - mu.float()[None]
    q, s = quantize_rows(y.reshape(t, h * d).contiguous())
    return q.view(t, h, d), s.view(t, h, d // BLOCK_SCALE)


def quantize_rows_torch(x: torch.Tensor) -> tuple[torch.Tensor, torch.Tensor]:
    """The reference's own pure-torch statement of the quantizer, extended to return the byte.

    ``scripts/bench/moe/kernel_ladder.py:184-188``.  Independent of the C code: torch's
    ``log2``/``ceil``/``exp2`` and torch's CPU ``float8_e4m3fn`` cast do the arithmetic.
    Used to pin the C oracle and as the vectorised CPU baseline.
    """
    m, k = x.shape
    blocks = x.reshape(m, k // BLOCK_SCALE, BLOCK_SCALE).float()
    amax = blocks.abs().amax(dim=-1, keepdim=True)
    exponent = torch.ceil(torch.log2(amax.clamp_min(1e-30) / E4M3_MAX)).clamp_min(-127.0)
    q = (blocks / torch.exp2(exponent)).to(torch.float8_e4m3fn).view(torch.uint8).reshape(m, k)
    s = (exponent + 127.0).to(torch.uint8).reshape(m, k // BLOCK_SCALE)
    return q, s


def e4m3_decode_table() -> torch.Tensor:
    """fp32 value of each of the 256 e4m3fn bit patterns (0x7F/0xFF are NaN)."""
    return torch.tensor([lib().ora_e4m3_to_f32(c) for c in range(256)], dtype=torch.float32)


def dequant(q: torch.Tensor, s: torch.Tensor, dtype: torch.dtype = torch.float64) -> torch.Tensor:
    """``q * 2^(s-127)`` broadcast over blocks of 32 of the last axis (grouped.py:335-336)."""
    q = q.view(torch.uint8) if q.dtype != torch.uint8 else q
    vals = e4m3_decode_table().to(dtype)[q.long()]
    scale = torch.exp2(s.view(torch.uint8).to(dtype) - 127.0).repeat_interleave(BLOCK_SCALE, dim=-1)
    return vals * scale


def swizzle_32_4_4(s: torch.Tensor) -> torch.Tensor:
    rows, cols = s.shape
    s = s.contiguous()
    out = torch.empty(-(-rows // 128) * 128 * -(-cols // 4) * 4, dtype=torch.uint8)
    lib().ora_swizzle_32_4_4(s.data_ptr(), rows, cols, cols, out.data_ptr())
    return out


# --------------------------------------------------------------------------- GEMM


def gemm_nt(aq, a_scale, bq, b_scale, dtype: torch.dtype = torch.float64) -> torch.Tensor:
    """``deq(A) @ deq(B).T`` in ``dtype`` (fp64 = the precision oracle; fp32 = the timed CPU path)."""
    return dequant(aq, a_scale, dtype) @ dequant(bq, b_scale, dtype).T


def gemm_nt_scalar(aq, a_scale, bq, b_scale) -> torch.Tensor:
    """The same product by the scalar C triple loop (tiny sizes; pins ``gemm_nt``)."""
    m, k = aq.shape
    n = bq.shape[0]
    aq, a_scale, bq, b_scale = (t.view(torch.uint8).contiguous() for t in (aq, a_scale, bq, b_scale))
    c = torch.empty(m, n, dtype=torch.float64)
    lib().ora_gemm_nt_f64(
        aq.data_ptr(), k, a_scale.data_ptr(), k // BLOCK_SCALE, bq.data_ptr(), k, b_scale.data_ptr(),
        k // BLOCK_SCALE, m, n, k, c.data_ptr(), n,
    )
    return c


def grouped_gemm_nt(xq, x_scale, wq, w_scale, offsets, index=None, dtype=torch.float64) -> torch.Tensor:
    """Per-expert loop over the offset table (grouped.py:330-350).  Returns only the real rows."""
    xd = dequant(xq, x_scale, dtype)
    if index is not None:
        xd = xd.index_select(0, index.long())
    off = [int(v) for v in offsets.tolist()]
    outs = []
    for e in range(wq.shape[0]):
        outs.append(xd[off[e] : off[e + 1]] @ dequant(wq[e], w_scale[e], dtype).T)
    return torch.cat(outs, dim=0)


def grouped_wgrad(a, b, offsets, a_index=None, b_index=None, row_scale=None, dtype=torch.float64) -> torch.Tensor:
    """``dW[e] = A[rows(e)].T @ B[rows(e)]`` (grouped.py:152-247), operands as given (already rounded).

    ``row_scale`` multiplies A's rows in fp32 before the cast back to A's dtype
    (grouped.py:218-221).  Empty experts give zeros.
    """
    off = [int(v) for v in offsets.tolist()]
    num_experts = len(off) - 1
    n, k = a.shape[1], b.shape[1]
    dw = torch.zeros(num_experts, n, k, dtype=dtype)
    for e in range(num_experts):
        rows = torch.arange(off[e], off[e + 1])
        ar = a[a_index[rows].long()] if a_index is not None else a[rows]
        br = b[b_index[rows].long()] if b_index is not None else b[rows]
        if row_scale is not None:
            ar = (ar.float() * row_scale[rows].float()[:, None]).to(a.dtype)
        dw[e] = ar.to(dtype).T @ br.to(dtype)
    return dw


# --------------------------------------------------------------------------- metrics / routing


def rel_error(got: torch.Tensor, ref: torch.Tensor) -> float:
    """``||got - ref|| / ||ref||`` in fp64 (bench/core/timing.py:201-206)."""
    got = got.detach().double()
    ref = ref.detach().double()
    return ((got - ref).norm() / ref.norm().clamp_min(1e-30)).item()


def expert_sort(flat_expert: torch.Tensor, num_experts: int, top_k: int):
    """Stable argsort + cumsum (moe_dispatch.py:264-282): ``(offsets, order, token_of)`` int32."""
    order = torch.argsort(flat_expert.long(), stable=True).to(torch.int32)
    counts = torch.bincount(flat_expert.long(), minlength=num_experts)
    offsets = torch.zeros(num_experts + 1, dtype=torch.int32)
    offsets[1:] = counts.cumsum(0).to(torch.int32)
    return offsets, order, (order // top_k).to(torch.int32)


def expert_counts(flat_idx: torch.Tensor, num_buckets: int) -> torch.Tensor:
    """``(num_buckets,)`` int32 histogram of the picks (models/components/moe.py:38-46, a scatter_add of ones)."""
    return torch.bincount(flat_idx.long(), minlength=num_buckets)[:num_buckets].to(torch.int32)


def combine_routed(rows: torch.Tensor, weight: torch.Tensor, order: torch.Tensor, token_of: torch.Tensor,
                   num_tokens: int, valid_rows: int | None = None) -> torch.Tensor:
    """``out[token_of[p]] += rows[p] * weight[order[p]]`` over the sorted rows (moe_dispatch.py:203-220).

    The product is taken in fp32 and rounded to ``rows.dtype`` (``_combine_fwd`` :85-88); the
    additions run in ascending sorted position with the sum rounded to ``rows.dtype`` after each,
    which is what an ``index_add`` into a 16-bit tensor does.  Written as one vectorized step per
    "n-th row of its token" so that it does not lean on the loop order inside ``index_add``.
    """
    n = rows.shape[0]
    scaled = (rows.float() * weight.float()[order.long()][:, None]).to(rows.dtype)
    keep = torch.arange(n) < (n if valid_rows is None else int(valid_rows))
    tok = token_of.long()
    out = torch.zeros(num_tokens, rows.shape[1], dtype=rows.dtype)
    # nth[p] = how many kept rows of the same token sit at lower sorted positions
    nth = torch.zeros(n, dtype=torch.long)
    seen = torch.zeros(num_tokens, dtype=torch.long)
    for p in torch.nonzero(keep).flatten().tolist():
        nth[p] = seen[tok[p]]
        seen[tok[p]] += 1
    for r in range(int(seen.max()) if n else 0):
        sel = keep & (nth == r)
        out[tok[sel]] = (out[tok[sel]].float() + scaled[sel].float()).to(rows.dtype)
    return out


def combine_routed_grads(grad_out: torch.Tensor, rows: torch.Tensor, weight: torch.Tensor, order: torch.Tensor,
                         token_of: torch.Tensor, valid_rows: int | None = None):
    """``(grad_rows, grad_weight)`` of the combine (``_combine_bwd``, moe_dispatch.py:93-131).

    ``grad_rows`` in ``rows.dtype`` (one fp32 product, one rounding: exact), ``grad_weight`` per
    pair in fp64 (the kernel sums in fp32; compare with a tolerance).
    """
    n = rows.shape[0]
    keep = torch.arange(n) < (n if valid_rows is None else int(valid_rows))
    g = grad_out[token_of.long()]
    grad_rows = (g.float() * weight.float()[order.long()][:, None]).to(rows.dtype)
    grad_rows[~keep] = 0
    dots = (g.double() * rows.double()).sum(dim=1)
    dots[~keep] = 0
    grad_weight = torch.zeros(weight.numel(), dtype=torch.float64)
    grad_weight[order.long()] = dots
    return grad_rows, grad_weight


def silu(x: torch.Tensor) -> torch.Tensor:
    return x * torch.sigmoid(x)


# --------------------------------------------------------------------------- RMSNorm producer


def rms_norm_mx(x: torch.Tensor, weight: torch.Tensor | None, eps: float = 1e-6):
    """``(out, rstd, q, s)`` of ``_rmsnorm_fwd`` with QUANT (rmsnorm.py:52-84).

    ``rstd = 1 / sqrt(sum(x^2) / K + eps)`` with the sum taken in fp64 (exact for 16-bit inputs, so
    every summation order agrees on the fp32 it rounds to) and the remaining steps in fp32 in the
    reference's order; ``y = x * rstd * w`` in fp32; ``out`` is ``y`` rounded to ``x.dtype``; the
    codes are quantized from the fp32 ``y`` (K % 32 == 0, else ``q = s = None``).
    """
    import numpy as np

    m, k = x.shape
    ss = x.double().square().sum(dim=1).numpy()
    # each fp32 step as "fp64 operation, rounded once to fp32": for fp32 operands that is the correctly
    # rounded fp32 result (53 >= 2 * 24 + 2 bits) and it does not depend on which vector code path a
    # CPU build of torch picks for float sqrt and divide (they were seen to differ between hosts)
    mean = (ss.astype(np.float32).astype(np.float64) / np.float64(np.float32(k))).astype(np.float32) + np.float32(eps)
    root = np.sqrt(mean.astype(np.float64)).astype(np.float32)
    rstd = torch.from_numpy((1.0 / root.astype(np.float64)).astype(np.float32))
    y = x.float() * rstd[:, None]
    if weight is not None:
        y = y * weight.float()[None, :]
    q = s = None
    if k % BLOCK_SCALE == 0:
        q, s = quantize_rows(y.contiguous())
    return y.to(x.dtype), rstd, q, s


def rms_norm_grads(x: torch.Tensor, weight: torch.Tensor | None, dout: torch.Tensor, eps: float = 1e-6):
    """``(dx, dw)`` in fp64 by automatic differentiation of torch's own ``rms_norm`` (rmsnorm.py:87-128 computes the same)."""
    xd = x.double().requires_grad_(True)
    wd = None if weight is None else weight.double().requires_grad_(True)
    out = torch.nn.functional.rms_norm(xd, (x.shape[1],), wd, eps)
    out.backward(dout.double())
    return xd.grad, None if wd is None else wd.grad
