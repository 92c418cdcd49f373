"""Feed-forward and attention-projection containers the MXFP8 swap operates on.

``GLUMLP``/``SwiGLU`` keep the attribute names and constructor of the reference's
``src/kohakuwullm/models/components/mlp.py:37-80`` (``w_in`` | ``gate_proj``+``up_proj``,
``w_out``), and ``AttentionProjections`` the four names of
``models/components/attention.py:61-66`` (``q_proj, k_proj, v_proj, o_proj``), so
``swap_mxfp8`` finds the same layers.  They are last-dim ops and serve packed ``(T, D)``
and padded ``(B, S, D)`` hidden states unchanged.
"""

from __future__ import annotations

import torch
import torch.nn as nn
import torch.nn.functional as F

from kohakuwullm_amd.kernels.mxfp8.mlp import mxfp8_swiglu_mlp
from kohakuwullm_amd.kernels.mxfp8.quantize import quantize_mx, quantize_mx_cols
from kohakuwullm_amd.models.mxfp8_swap import Matmul
from kohakuwullm_amd.registry import MLP


def resolve_hidden(dim: int, ratio: float, hidden: int | None = None, multiple_of: int = 128, glu: bool = True) -> int:
    """Feed-forward width rounded up to ``multiple_of``; GLU layers take the usual 2/3 correction."""
    if hidden is not None:
        return hidden
    width = dim * ratio * (2 / 3) if glu else dim * ratio
    return multiple_of * ((int(width) + multiple_of - 1) // multiple_of)


class GLUMLP(nn.Module):
    """``w_out(act(gate) * value)`` with gate and value in one ``w_in`` (default) or split."""

    act = staticmethod(F.silu)

    def __init__(self, dim: int, ratio: float = 4.0, hidden: int | None = None, multiple_of: int = 128,
                 bias: bool = False, fused_gate: bool = True) -> None:
        super().__init__()
        self.hidden = resolve_hidden(dim, ratio, hidden, multiple_of, glu=True)
        self.fused_gate = fused_gate
        if fused_gate:
            self.w_in = nn.Linear(dim, 2 * self.hidden, bias=bias)
        else:
            self.gate_proj = nn.Linear(dim, self.hidden, bias=bias)
            self.up_proj = nn.Linear(dim, self.hidden, bias=bias)
        self.w_out = nn.Linear(self.hidden, dim, bias=bias)

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        if self.fused_gate:
            gate, value = self.w_in(x).chunk(2, dim=-1)
        else:
            gate, value = self.gate_proj(x), self.up_proj(x)
        return self.w_out(self.act(gate) * value)


@MLP.register("swiglu")
class SwiGLU(GLUMLP):
    """SwiGLU feed-forward; ``swap_mxfp8`` turns its projections into ``MXFP8Linear``."""


@MLP.register("swiglu_mxfp8")
class MXFP8SwiGLU(nn.Module):
    """SwiGLU feed-forward whose whole forward/backward is the fused MXFP8 graph.

    Holds ``w_in (2H, dim)`` and ``w_out (dim, H)`` as bare parameters and declares them
    through the ``mxfp8_matmul`` / ``enable_mxfp8`` protocol.  The quantized copies are
    plain attributes, refreshed by ``refresh_quantized_weight()`` after each optimizer step.
    """

    def __init__(self, dim: int, ratio: float = 4.0, hidden: int | None = None, multiple_of: int = 128,
                 dtype=torch.bfloat16) -> None:
        super().__init__()
        self.dim = dim
        self.hidden = resolve_hidden(dim, ratio, hidden, multiple_of, glu=True)
        self.w_in = nn.Parameter(torch.empty(2 * self.hidden, dim, dtype=dtype))
        self.w_out = nn.Parameter(torch.empty(dim, self.hidden, dtype=dtype))
        nn.init.normal_(self.w_in, std=dim**-0.5)
        nn.init.normal_(self.w_out, std=self.hidden**-0.5)
        self._packed = None

    def mxfp8_matmul(self) -> dict[str, Matmul]:
        refusal = None
        if self.dim % 32 or self.hidden % 32:
            refusal = f"dim={self.dim} / hidden={self.hidden} must be multiples of 32"
        return {
            "w_in": Matmul(2 * self.hidden * self.dim, refusal),
            "w_out": Matmul(self.hidden * self.dim, refusal),
        }

    def enable_mxfp8(self) -> None:
        self.refresh_quantized_weight()

    @torch.no_grad()
    def refresh_quantized_weight(self) -> None:
        self._packed = (
            quantize_mx(self.w_in),
            quantize_mx_cols(self.w_in),
            quantize_mx(self.w_out),
            quantize_mx_cols(self.w_out),
        )

    def mxfp8_refresh_plan(self) -> list[torch.Tensor] | None:
        """Both matrices as dual (row + column axis) quantizations, for ``refresh_mxfp8_weights``' single launch."""
        if self.dim % 32 or self.hidden % 32 or not self.w_in.is_cuda:
            return None
        return [self.w_in.detach(), self.w_out.detach()]

    def mxfp8_install(self, copies) -> None:
        (q1, s1, qt1, st1), (q2, s2, qt2, st2) = copies
        self._packed = ((q1, s1), (qt1, st1), (q2, s2), (qt2, st2))

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        if self._packed is None:
            self.refresh_quantized_weight()
        return mxfp8_swiglu_mlp(x, self.w_in, self.w_out, self._packed)

    def _apply(self, *args, **kwargs):
        self._packed = None
        return super()._apply(*args, **kwargs)


class AttentionProjections(nn.Module):
    """The four projections of a GQA attention block, without the attention core.

    ``project`` gives ``q (…, heads, hd)``, ``k, v (…, kv_heads, hd)``; ``merge`` applies
    ``o_proj`` to the flattened heads.
    """

    def __init__(self, dim: int, num_heads: int, num_kv_heads: int | None = None, head_dim: int | None = None,
                 bias: bool = False) -> None:
        super().__init__()
        self.num_heads = num_heads
        self.num_kv_heads = num_kv_heads or num_heads
        self.head_dim = head_dim or dim // num_heads
        self.q_proj = nn.Linear(dim, self.num_heads * self.head_dim, bias=bias)
        self.k_proj = nn.Linear(dim, self.num_kv_heads * self.head_dim, bias=bias)
        self.v_proj = nn.Linear(dim, self.num_kv_heads * self.head_dim, bias=bias)
        self.o_proj = nn.Linear(self.num_heads * self.head_dim, dim, bias=bias)

    def project(self, x: torch.Tensor):
        lead = x.shape[:-1]
        q = self.q_proj(x).view(*lead, self.num_heads, self.head_dim)
        k = self.k_proj(x).view(*lead, self.num_kv_heads, self.head_dim)
        v = self.v_proj(x).view(*lead, self.num_kv_heads, self.head_dim)
        return q, k, v

    def merge(self, heads: torch.Tensor) -> torch.Tensor:
        return self.o_proj(heads.reshape(*heads.shape[:-2], self.num_heads * self.head_dim))
