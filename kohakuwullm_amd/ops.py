"""The HIP entry points as opaque ``torch.library`` operators, each with a fake (meta) kernel.

A graph compiler cannot look inside a ``ctypes`` call; registered as custom operators the kernels
are leaves it traces past, the convention the reference uses for its vendor GEMM
(``kohakuwullm::mxfp8_mm_swizzled``, ``src/kohakuwullm/kernels/mxfp8/interop.py:104-122``; that
operator's counterpart lives in ``kernels/mxfp8/interop.py``).  The eager modules do not go
through these wrappers (an operator dispatch costs more host time than a launch); they are for
callers that compile a region around the kernels:

    torch.ops.kohakuwullm_amd.quantize_mx(x) -> (q, s)

Forward-only leaves: the autograd wiring of the path lives in the modules' ``autograd.Function``s.
"""

from __future__ import annotations

import torch

from kohakuwullm_amd.kernels.elementwise.rmsnorm import rms_norm_mx as _rms_norm_mx
from kohakuwullm_amd.kernels.moe import moe_dispatch as _dispatch
from kohakuwullm_amd.kernels.mxfp8 import fused_act as _fused_act
from kohakuwullm_amd.kernels.mxfp8 import grouped as _grouped
from kohakuwullm_amd.kernels.mxfp8 import quantize as _quantize

_FP8 = torch.float8_e4m3fn
_B = _quantize.BLOCK_SCALE
Tensor = torch.Tensor


@torch.library.custom_op("kohakuwullm_amd::quantize_mx", mutates_args=())
def quantize_mx(x: Tensor) -> tuple[Tensor, Tensor]:
    return _quantize.quantize_mx(x)


@quantize_mx.register_fake
def _(x):
    m, k = x.shape
    return x.new_empty((m, k), dtype=_FP8), x.new_empty((m, k // _B), dtype=torch.uint8)


@torch.library.custom_op("kohakuwullm_amd::quantize_mx_cols", mutates_args=())
def quantize_mx_cols(x: Tensor) -> tuple[Tensor, Tensor]:
    return _quantize.quantize_mx_cols(x)


@quantize_mx_cols.register_fake
def _(x):
    m, k = x.shape
    return x.new_empty((k, m), dtype=_FP8), x.new_empty((k, m // _B), dtype=torch.uint8)


@torch.library.custom_op("kohakuwullm_amd::quantize_mx_dual", mutates_args=())
def quantize_mx_dual(x: Tensor) -> tuple[Tensor, Tensor, Tensor, Tensor]:
    return _quantize.quantize_mx_dual(x)


@quantize_mx_dual.register_fake
def _(x):
    m, k = x.shape
    return (x.new_empty((m, k), dtype=_FP8), x.new_empty((m, k // _B), dtype=torch.uint8),
            x.new_empty((k, m), dtype=_FP8), x.new_empty((k, m // _B), dtype=torch.uint8))


@torch.library.custom_op("kohakuwullm_amd::mxfp8_matmul_pq", mutates_args=())
def mxfp8_matmul_pq(aq: Tensor, a_scale: Tensor, bq: Tensor, b_scale: Tensor,
                    out_dtype: torch.dtype = torch.bfloat16) -> Tensor:
    return _quantize.mxfp8_matmul_pq(aq, a_scale, bq, b_scale, out_dtype)


@mxfp8_matmul_pq.register_fake
def _(aq, a_scale, bq, b_scale, out_dtype=torch.bfloat16):
    return aq.new_empty((aq.shape[0], bq.shape[0]), dtype=out_dtype)


@torch.library.custom_op("kohakuwullm_amd::swiglu_mx", mutates_args=())
def swiglu_mx(gate: Tensor, up: Tensor) -> tuple[Tensor, Tensor]:
    return _fused_act.swiglu_mx(gate, up)


@swiglu_mx.register_fake
def _(gate, up):
    m, k = gate.shape
    return gate.new_empty((m, k), dtype=_FP8), gate.new_empty((m, k // _B), dtype=torch.uint8)


@torch.library.custom_op("kohakuwullm_amd::rms_norm_mx", mutates_args=())
def rms_norm_mx(x: Tensor, weight: Tensor, eps: float = 1e-6) -> tuple[Tensor, Tensor, Tensor]:
    out, q, s = _rms_norm_mx(x.detach(), weight.detach(), eps)
    return out, q, s


@rms_norm_mx.register_fake
def _(x, weight, eps=1e-6):
    k = x.shape[-1]
    return (torch.empty_like(x), x.new_empty(x.shape, dtype=_FP8),
            x.new_empty((*x.shape[:-1], k // _B), dtype=torch.uint8))


@torch.library.custom_op("kohakuwullm_amd::grouped_mxfp8_gemm", mutates_args=())
def grouped_mxfp8_gemm(xq: Tensor, x_scale: Tensor, wq: Tensor, w_scale: Tensor, offsets: Tensor,
                       index: Tensor | None = None, out_dtype: torch.dtype = torch.bfloat16) -> Tensor:
    return _grouped.grouped_mxfp8_gemm(xq, x_scale, wq, w_scale, offsets, index, out_dtype)


@grouped_mxfp8_gemm.register_fake
def _(xq, x_scale, wq, w_scale, offsets, index=None, out_dtype=torch.bfloat16):
    rows = xq.shape[0] if index is None else index.shape[0]
    return xq.new_empty((rows, wq.shape[1]), dtype=out_dtype)


@torch.library.custom_op("kohakuwullm_amd::expert_sort", mutates_args=())
def expert_sort(flat_expert: Tensor, counts: Tensor, top_k: int, num_experts: int) -> tuple[Tensor, Tensor, Tensor, Tensor]:
    return _dispatch.expert_sort(flat_expert, counts, top_k, num_experts)


@expert_sort.register_fake
def _(flat_expert, counts, top_k, num_experts):
    n = flat_expert.shape[0]
    i32 = torch.int32
    return (counts.new_empty((num_experts + 1,), dtype=i32), counts.new_empty((n,), dtype=i32),
            counts.new_empty((n,), dtype=i32), counts.new_empty((1,), dtype=i32))


@torch.library.custom_op("kohakuwullm_amd::combine_routed", mutates_args=())
def combine_routed(rows: Tensor, weight: Tensor, order: Tensor, token_of: Tensor, num_tokens: int) -> Tensor:
    return _dispatch.combine_routed(rows.detach(), weight.detach(), order, token_of, num_tokens)


@combine_routed.register_fake
def _(rows, weight, order, token_of, num_tokens):
    return rows.new_empty((num_tokens, rows.shape[1]))


__all__ = ["combine_routed", "expert_sort", "grouped_mxfp8_gemm", "mxfp8_matmul_pq", "quantize_mx", "quantize_mx_cols",
           "quantize_mx_dual", "rms_norm_mx", "swiglu_mx"]
