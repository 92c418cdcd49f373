"""Routed-expert feed-forward whose experts run on the MXFP8 kernels.

Host-side counterpart of the MXFP8 hooks of the reference's ``MoEMLP``
(``src/kohakuwullm/models/components/moe.py:336-392,451-508``): the stacked expert parameters
``w_in (E, 2H, dim)`` / ``w_out (E, dim, H)``, the ``mxfp8_matmul`` / ``enable_mxfp8``
declaration protocol, ``refresh_quantized_weight`` installed on the instance, the cache drop
on ``_apply``, and the two routed paths (``mxfp8_expert_path`` ``"fused"`` | ``"unfused"``).
The router is plain PyTorch; the dispatch (``expert_counts``, ``expert_sort``: ``offsets``,
``order``, ``token_of`` in the format of ``src/kohakuwullm/kernels/moe/moe_dispatch.py:223-282``)
and the combine of the unfused path run on the HIP kernels of ``kernels/moe/moe_dispatch.py``.
"""

from __future__ import annotations

import torch
import torch.nn as nn

from kohakuwullm_amd.kernels.moe.moe_dispatch import expert_counts, expert_sort
from kohakuwullm_amd.kernels.mxfp8.linear import compute_dtype
from kohakuwullm_amd.kernels.mxfp8.moe import (
    MXFP8ExpertWeights,
    mxfp8_moe_experts,
    mxfp8_moe_experts_reference,
    mxfp8_moe_experts_unfused,
)
from kohakuwullm_amd.kernels.mxfp8.quantize import BLOCK_SCALE
from kohakuwullm_amd.models.mxfp8_swap import Matmul
from kohakuwullm_amd.registry import MOE


class TopKRouter(nn.Module):
    """Softmax top-k token -> expert assignment (kept in 16/32-bit: a router's logit scale is the gate sharpness)."""

    def __init__(self, dim: int, num_experts: int, top_k: int, norm_topk_prob: bool = True) -> None:
        super().__init__()
        self.num_experts, self.top_k, self.norm_topk_prob = num_experts, top_k, norm_topk_prob
        self.weight = nn.Parameter(torch.empty(num_experts, dim))
        nn.init.normal_(self.weight, std=dim**-0.5)

    def route(self, x: torch.Tensor):
        scores = (x.float() @ self.weight.float().T).softmax(-1)
        topk_weight, topk_idx = scores.topk(self.top_k, dim=-1)
        if self.norm_topk_prob:
            topk_weight = topk_weight / topk_weight.sum(-1, keepdim=True)
        return topk_idx, topk_weight, expert_counts(topk_idx.reshape(-1), self.num_experts)


@MOE.register("moe")
class MoEMLP(nn.Module):
    """Top-k routed SwiGLU experts.  ``enable_mxfp8()`` (called by ``swap_mxfp8``) moves them to MXFP8."""

    def __init__(self, dim: int, hidden: int, num_experts: int, top_k: int, mxfp8_expert_path: str = "fused",
                 dtype=torch.bfloat16) -> None:
        super().__init__()
        self.dim, self.hidden, self.num_experts, self.top_k = dim, hidden, num_experts, top_k
        self.router = TopKRouter(dim, num_experts, top_k)
        self.w_in = nn.Parameter(torch.empty(num_experts, 2 * hidden, dim, dtype=dtype))
        self.w_out = nn.Parameter(torch.empty(num_experts, dim, hidden, dtype=dtype))
        nn.init.normal_(self.w_in, std=dim**-0.5)
        nn.init.normal_(self.w_out, std=(hidden * 2) ** -0.5)
        self._routed = self._routed_eager
        self._packed: MXFP8ExpertWeights | None = None
        self.mxfp8_expert_path = mxfp8_expert_path

    def mxfp8_matmul(self) -> dict[str, Matmul]:
        refusal = self._mxfp8_refusal()
        return {
            "w_in": Matmul(self.w_in[0].numel() * self.top_k, refusal),
            "w_out": Matmul(self.w_out[0].numel() * self.top_k, refusal),
            "router.weight": Matmul(self.router.weight.numel(), "a router's logit scale is the gate sharpness", never=True),
        }

    def _mxfp8_refusal(self) -> str | None:
        for name, value in (("dim", self.dim), ("hidden", self.hidden)):
            if value % BLOCK_SCALE:
                return (f"{name}={value} is not a multiple of {BLOCK_SCALE}; it is a contraction axis shared "
                        "with an activation cast")
        return None

    def enable_mxfp8(self) -> None:
        if self.mxfp8_expert_path == "fused":
            self._routed = self._routed_mxfp8
        elif self.mxfp8_expert_path == "unfused":
            self._routed = self._routed_mxfp8_unfused
        else:
            raise ValueError(f"unknown mxfp8_expert_path {self.mxfp8_expert_path!r}; expected 'fused' or 'unfused'")
        self.refresh_quantized_weight = self._refresh_mxfp8

    @torch.no_grad()
    def _refresh_mxfp8(self) -> None:
        """Requantize the four fp8 expert copies.  Call after every optimizer step."""
        if self._packed is None:
            self._packed = MXFP8ExpertWeights(self.w_in, self.w_out)
        else:
            self._packed.refresh(self.w_in, self.w_out)

    def mxfp8_refresh_plan(self):
        """The expert stacks as two matrices for ``refresh_mxfp8_weights``' single launch (``None``: refresh alone)."""
        if self._routed == self._routed_eager:
            return None
        return MXFP8ExpertWeights.plan(self.w_in, self.w_out)

    def mxfp8_install(self, copies) -> None:
        if self._packed is None:
            self._packed = MXFP8ExpertWeights()
        self._packed.install(copies, self.num_experts)

    def _apply(self, *args, **kwargs):
        self._packed = None
        return super()._apply(*args, **kwargs)

    def _routed_eager(self, flat, topk_weight, order, token_of, offsets):
        x = flat.to(compute_dtype(flat))
        return mxfp8_moe_experts_reference(x, self.w_in.to(x.dtype), self.w_out.to(x.dtype),
                                           topk_weight.reshape(-1).to(x.dtype), token_of, order,
                                           offsets[: self.num_experts + 1])

    def _routed_mxfp8(self, flat, topk_weight, order, token_of, offsets):
        if self._packed is None:
            self._refresh_mxfp8()
        x = flat.to(compute_dtype(flat))
        return mxfp8_moe_experts(x, self.w_in, self.w_out, topk_weight.reshape(-1), token_of, order,
                                 offsets[: self.num_experts + 1], self._packed)

    def _routed_mxfp8_unfused(self, flat, topk_weight, order, token_of, offsets):
        if self._packed is None:
            self._refresh_mxfp8()
        x = flat.to(compute_dtype(flat))
        return mxfp8_moe_experts_unfused(x, self.w_in, self.w_out, topk_weight.reshape(-1), token_of, order,
                                         offsets[: self.num_experts + 1], self._packed)

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        shape = x.shape
        flat = x.reshape(-1, shape[-1])
        topk_idx, topk_weight, counts = self.router.route(flat)
        offsets, order, token_of, _ = expert_sort(topk_idx.reshape(-1), counts, topk_idx.shape[-1], self.num_experts)
        return self._routed(flat, topk_weight, order, token_of, offsets).reshape(shape)
