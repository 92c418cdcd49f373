"""Sparse feed-forward ``shared(x) + sum_k w_k * expert_k(x)`` whose routed experts run on the MXFP8 kernels.

Drop-in for the reference's ``MoEMLP`` (``src/kohakuwullm/models/components/moe.py:252-523``):
registered as ``"moe"`` in the ``MLP`` registry, the same constructor keywords
(``dim, ratio, hidden, multiple_of, num_experts, top_k, num_shared, bias, router, router_dim,
dense_fallback, expert_path, **router_kwargs``), the same parameters (``w_in (E, 2H, dim)``,
``w_out (E, dim, H)``, ``router.weight``, ``shared.*``), the ``mxfp8_matmul`` /
``enable_mxfp8`` declaration protocol, ``refresh_quantized_weight`` installed on the instance,
the cache drop on ``_apply``, ``forward(x, route_on=None)``, ``router_losses`` and
``emits_router_loss``.  ``TopKRouter`` is registered as ``"topk"`` in ``ROUTER`` with the
reference's keywords (``components/moe.py:49-248``).

What runs where.  The MXFP8 routed paths (``mxfp8_expert_path`` ``"fused"`` | ``"unfused"``), the
dispatch (``expert_counts``, ``expert_sort``) and the combine run on this package's HIP kernels.
The router's scores and top-k, and the 16-bit routed path a layer uses before ``enable_mxfp8``
(the reference's bf16 Triton kernels, which are not part of the MXFP8 path), are plain PyTorch
here: ``expert_path`` ``"fused"`` and ``"eager"`` name the same PyTorch composition.
"""

from __future__ import annotations

import torch
import torch.nn as nn
import torch.nn.functional as F

from kohakuwullm_amd.kernels.moe.moe_dispatch import combine_routed, expert_counts, expert_sort
from kohakuwullm_amd.kernels.mxfp8.linear import compute_dtype
from kohakuwullm_amd.kernels.mxfp8.moe import (
    MXFP8ExpertWeights,
    mxfp8_moe_experts,
    mxfp8_moe_experts_unfused,
)
from kohakuwullm_amd.kernels.mxfp8.quantize import BLOCK_SCALE
from kohakuwullm_amd.models.mlp import GLUMLP, resolve_hidden
from kohakuwullm_amd.models.mxfp8_swap import Matmul
from kohakuwullm_amd.registry import MLP, ROUTER, build

SCORE_FUNCS = {
    "sigmoid": torch.sigmoid,
    "softmax": lambda logits: logits.softmax(-1),
    "sqrtsoftplus": lambda logits: F.softplus(logits).sqrt(),
}


def _histogram(flat_idx: torch.Tensor, num_buckets: int) -> torch.Tensor:
    """Rows per bucket without a host sync: the HIP kernel on the GPU, a scatter-add elsewhere."""
    if flat_idx.is_cuda:
        return expert_counts(flat_idx, num_buckets)
    counts = torch.zeros(num_buckets, dtype=torch.int32, device=flat_idx.device)
    return counts.scatter_add_(0, flat_idx, torch.ones_like(flat_idx, dtype=torch.int32))


@ROUTER.register("topk")
class TopKRouter(nn.Module):
    """Token -> expert assignment (``components/moe.py:49-248``), evaluated in fp32 with PyTorch ops.

    Scores are ``score_func(x W^T)``; selection adds the balancing bias (a buffer moved by
    :meth:`update_bias`, never by a gradient) and may be limited to the strongest ``topk_groups``
    of ``n_groups`` expert groups; gate weights are the unbiased scores of the selected experts,
    optionally renormalized, times ``routed_scaling_factor``.  ``fused`` is accepted for
    configuration compatibility: there is one implementation here.
    """

    def __init__(self, dim: int, num_experts: int, top_k: int = 8, score_func: str = "sigmoid",
                 norm_topk_prob: bool = True, routed_scaling_factor: float = 1.0, bias_update_rate: float = 1e-3,
                 n_groups: int = 1, topk_groups: int = 1, aux_loss_weight: float = 0.0, z_loss_weight: float = 0.0,
                 fused: bool = True) -> None:
        super().__init__()
        if num_experts % n_groups:
            raise ValueError(f"num_experts {num_experts} not divisible by n_groups {n_groups}")
        if score_func not in SCORE_FUNCS:
            raise ValueError(f"unknown score_func {score_func!r}")
        self.num_experts, self.top_k = num_experts, top_k
        self.score_func, self.norm_topk_prob = score_func, norm_topk_prob
        self.routed_scaling_factor, self.bias_update_rate = routed_scaling_factor, bias_update_rate
        self.n_groups, self.topk_groups = n_groups, topk_groups
        self.aux_loss_weight, self.z_loss_weight = aux_loss_weight, z_loss_weight
        self.reduce_load, self.load_group = True, None
        self.use_fused = False
        self.emits_loss = aux_loss_weight > 0.0 or z_loss_weight > 0.0
        self.weight = nn.Parameter(torch.empty(num_experts, dim))
        nn.init.normal_(self.weight, std=dim**-0.5)
        if bias_update_rate > 0:
            self.register_buffer("expert_bias", torch.zeros(num_experts))
            self.register_buffer("load_accum", torch.zeros(num_experts))
        else:
            self.expert_bias = self.load_accum = None
        self.aux_loss: torch.Tensor | None = None
        self.z_loss: torch.Tensor | None = None

    def forward(self, x: torch.Tensor):
        """``x (T, D)`` -> ``(topk_idx, topk_weight)``."""
        return self.route(x)[:2]

    def route(self, x: torch.Tensor):
        """``(topk_idx (T, k), topk_weight (T, k) in x.dtype, counts (E,) int32)``."""
        logits = F.linear(x.float(), self.weight.float())
        scores = SCORE_FUNCS[self.score_func](logits)
        choose_by = scores if self.expert_bias is None else scores + self.expert_bias
        if self.n_groups > 1:
            # a group's strength is the sum of its two best scores; only the strongest groups stay eligible
            per_group = choose_by.view(scores.shape[0], self.n_groups, -1)
            strength = per_group.topk(min(2, per_group.shape[-1]), dim=-1).values.sum(-1)
            allowed = torch.zeros_like(strength, dtype=torch.bool)
            allowed.scatter_(1, strength.topk(self.topk_groups, dim=-1).indices, True)
            choose_by = per_group.masked_fill(~allowed.unsqueeze(-1), float("-inf")).reshape_as(scores)
        topk_idx = choose_by.topk(self.top_k, dim=-1).indices
        topk_weight = scores.gather(1, topk_idx)
        if self.norm_topk_prob and self.top_k > 1:
            topk_weight = topk_weight / topk_weight.sum(-1, keepdim=True).clamp_min(1e-9)
        topk_weight = topk_weight * self.routed_scaling_factor
        counts = _histogram(topk_idx.reshape(-1), self.num_experts)
        self.z_loss = self.z_loss_weight * logits.logsumexp(-1).pow(2).mean() if self.z_loss_weight > 0 else None
        if self.aux_loss_weight > 0:
            # Switch-Transformer balance term E * sum_i f_i P_i
            share = counts.float() / (scores.shape[0] * self.top_k)
            self.aux_loss = self.aux_loss_weight * self.num_experts * (share * scores.mean(0)).sum()
        else:
            self.aux_loss = None
        if self.training and self.load_accum is not None:
            self.load_accum += counts
        return topk_idx, topk_weight.to(x.dtype), counts

    @torch.no_grad()
    def update_bias(self) -> torch.Tensor | None:
        """Once per optimizer step: move the selection bias towards the underloaded experts, clear the counter.

        Returns ``(max/mean, min/mean, experts without rows)`` of this step's load as one device tensor, or
        ``None`` when balancing is off or nothing was routed.  One GPU: there is no load to reduce over ranks.
        """
        if self.load_accum is None or not bool(self.load_accum.sum()):
            return None
        mean = self.load_accum.mean()
        self.expert_bias += self.bias_update_rate * torch.sign(mean - self.load_accum)
        unit = mean.clamp_min(1e-9)
        stats = torch.stack((self.load_accum.max() / unit, self.load_accum.min() / unit,
                             (self.load_accum == 0).sum().to(unit.dtype)))
        self.load_accum.zero_()
        return stats


@MLP.register("moe")
class MoEMLP(nn.Module):
    """Shared experts + top-k routed SwiGLU experts; ``enable_mxfp8()`` (``swap_mxfp8`` calls it) moves the routed ones to MXFP8.

    Args (``components/moe.py:270-285``): ``ratio`` / ``hidden`` / ``multiple_of`` size ONE routed expert;
    ``num_shared`` always-on experts form one ``GLUMLP`` of ``hidden * num_shared``; ``router`` is a spec for
    the ``ROUTER`` registry and receives ``router_kwargs``; ``router_dim`` is the width the router reads;
    ``dense_fallback`` is the per-expert loop (reads ``offsets`` on the host; refused by the MXFP8 swap);
    ``expert_path`` names the 16-bit routed path (``"fused"`` | ``"eager"``).
    """

    def __init__(self, dim: int, ratio: float = 4.0, hidden: int | None = None, multiple_of: int = 128,
                 num_experts: int = 64, top_k: int = 8, num_shared: int = 1, bias: bool = False, router="topk",
                 router_dim: int | None = None, dense_fallback: bool = False, expert_path: str = "fused",
                 **router_kwargs) -> None:
        super().__init__()
        if expert_path not in ("fused", "eager"):
            raise ValueError(f"unknown expert_path {expert_path!r}; expected 'fused' or 'eager'")
        self.dim, self.num_experts, self.top_k = dim, num_experts, top_k
        self.hidden = resolve_hidden(dim, ratio, hidden, multiple_of, glu=True)
        self.dense_fallback = dense_fallback
        self.router = build(router, ROUTER, dim=router_dim or dim, num_experts=num_experts, top_k=top_k, **router_kwargs)
        # a router with a sentinel slot (rows that no expert computes) sorts into one bucket more
        self.num_buckets = getattr(self.router, "num_buckets", num_experts)
        self._has_sentinel = self.num_buckets != num_experts
        self.w_in = nn.Parameter(torch.empty(num_experts, 2 * self.hidden, dim))
        self.w_out = nn.Parameter(torch.empty(num_experts, dim, self.hidden))
        nn.init.normal_(self.w_in, std=dim**-0.5)
        nn.init.normal_(self.w_out, std=(self.hidden * 2) ** -0.5)
        self.num_shared = num_shared
        self.shared = GLUMLP(dim, hidden=self.hidden * num_shared, bias=bias, multiple_of=1) if num_shared > 0 else None
        self.expert_path = expert_path
        self._routed = self._routed_16bit
        self._packed: MXFP8ExpertWeights | None = None
        self.mxfp8_expert_path = "fused"  # which MXFP8 path enable_mxfp8 installs: "fused" | "unfused"

    # ---- MXFP8 declaration protocol (models/mxfp8_protocol.py) ----

    def mxfp8_matmul(self) -> dict[str, Matmul]:
        refusal = self._mxfp8_refusal()
        return {
            "w_in": Matmul(self.w_in[0].numel() * self.top_k, refusal),
            "w_out": Matmul(self.w_out[0].numel() * self.top_k, refusal),
            "router.weight": Matmul(self.router.weight.numel(), "a router's logit scale is the gate sharpness", never=True),
        }

    def _mxfp8_refusal(self) -> str | None:
        if self.dense_fallback:
            return "dense_fallback=True is the eager test reference, not an fp8 path"
        for name, value in (("dim", self.dim), ("hidden", self.hidden)):
            if value % BLOCK_SCALE:
                return (f"{name}={value} is not a multiple of {BLOCK_SCALE}; it is a contraction axis shared "
                        "with an activation cast")
        return None

    def enable_mxfp8(self) -> None:
        paths = {"fused": self._routed_mxfp8, "unfused": self._routed_mxfp8_unfused}
        if self.mxfp8_expert_path not in paths:
            raise ValueError(f"unknown mxfp8_expert_path {self.mxfp8_expert_path!r}; expected 'fused' or 'unfused'")
        self._routed = paths[self.mxfp8_expert_path]
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
        if self._routed == self._routed_16bit:
            return None
        return MXFP8ExpertWeights.plan(self.w_in, self.w_out)

    def mxfp8_install(self, copies) -> None:
        if self._packed is None:
            self._packed = MXFP8ExpertWeights()
        self._packed.install(copies, self.num_experts)

    def _apply(self, *args, **kwargs):
        """Any device or dtype transform drops the fp8 expert copies."""
        self._packed = None
        return super()._apply(*args, **kwargs)

    def active_parameters(self) -> int:
        """Parameters one token touches (what its FLOPs follow)."""
        touched = (self.w_in[0].numel() + self.w_out[0].numel()) * self.top_k + self.router.weight.numel()
        if self.shared is not None:
            touched += sum(p.numel() for p in self.shared.parameters())
        return touched

    # ---- routed paths: (flat, topk_weight, order, token_of, offsets) -> (T, dim) ----

    def _valid_rows(self, offsets):
        """One-element view holding the number of rows that belong to real experts (the rest sit in the sentinel bucket)."""
        return offsets[self.num_experts : self.num_experts + 1]

    def _routed_16bit(self, flat, topk_weight, order, token_of, offsets):
        """The 16-bit control arm: gather, per-expert SwiGLU in the compute dtype, gated combine."""
        x = flat.to(compute_dtype(flat))
        rows = x.index_select(0, token_of.long())
        bounds = offsets[: self.num_experts + 1].tolist()  # host read: this arm is not the fast path
        w_in, w_out = self.w_in.to(x.dtype), self.w_out.to(x.dtype)
        pieces = []
        for e in range(self.num_experts):
            block = rows[bounds[e] : bounds[e + 1]]
            gate, value = (block @ w_in[e].T).chunk(2, dim=-1)
            pieces.append((F.silu(gate) * value) @ w_out[e].T)
        real = bounds[-1]
        out_sorted = torch.cat(pieces + [rows.new_zeros(rows.shape[0] - real, self.dim)], dim=0)
        weight = topk_weight.reshape(-1).to(x.dtype)
        if x.is_cuda and x.dtype in (torch.bfloat16, torch.float16, torch.float32):
            return combine_routed(out_sorted, weight, order, token_of, flat.shape[0], self._valid_rows(offsets))
        scaled = out_sorted[:real] * weight.index_select(0, order[:real].long()).unsqueeze(-1)
        return x.new_zeros(flat.shape[0], self.dim).index_add_(0, token_of[:real].long(), scaled)

    def _routed_mxfp8(self, flat, topk_weight, order, token_of, offsets):
        if self._packed is None:
            self._refresh_mxfp8()
        x = flat.to(compute_dtype(flat))  # compute dtype follows autocast; the activation may arrive fp32
        return mxfp8_moe_experts(x, self.w_in, self.w_out, topk_weight.reshape(-1), token_of, order,
                                 offsets[: self.num_experts + 1], self._packed)

    def _routed_mxfp8_unfused(self, flat, topk_weight, order, token_of, offsets):
        if self._packed is None:
            self._refresh_mxfp8()
        x = flat.to(compute_dtype(flat))
        return mxfp8_moe_experts_unfused(x, self.w_in, self.w_out, topk_weight.reshape(-1), token_of, order,
                                         offsets[: self.num_experts + 1], self._packed,
                                         self._valid_rows(offsets) if self._has_sentinel else None)

    def forward(self, x: torch.Tensor, route_on: torch.Tensor | None = None) -> torch.Tensor:
        shape = x.shape
        flat = x.reshape(-1, shape[-1])
        seen_by_router = flat if route_on is None else route_on.reshape(-1, route_on.shape[-1])
        topk_idx, topk_weight, counts = self.router.route(seen_by_router)
        # slot width from the tensor, not top_k: a router may pad it
        offsets, order, token_of, _ = expert_sort(topk_idx.reshape(-1), counts, topk_idx.shape[-1], self.num_buckets)
        out = self._routed(flat, topk_weight, order, token_of, offsets)
        if self.shared is not None:
            out = out + self.shared(flat)  # dtype by promotion, as the reference's forward (components/moe.py:395-449)
        return out.reshape(shape)

    def router_losses(self) -> torch.Tensor | None:
        """Sum of the router's auxiliary terms of the last forward, or ``None``."""
        terms = [t for t in (self.router.aux_loss, self.router.z_loss) if t is not None]
        return sum(terms) if terms else None

    @property
    def emits_router_loss(self) -> bool:
        return bool(getattr(self.router, "emits_loss", False))
