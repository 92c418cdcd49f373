"""Replace a built model's projections with MXFP8 linears, in place, and account for it.

Behaviour follows ``src/kohakuwullm/models/mxfp8_swap.py`` of the reference
(``swap_mxfp8`` :301-328, ``refresh_mxfp8_weights`` :331-343, ``SwapReport`` :41-103,
refusal rule :106-113): ``nn.Linear`` children with the projection attribute names are
replaced by ``linear_cls(in_features, out_features, dtype=weight.dtype)`` with the weight
copied; modules that declare bare-parameter matmuls through ``mxfp8_matmul()`` are
converted with ``enable_mxfp8()``; anything matmul-shaped that nobody claimed blocks.

Where the reference selects parents by class, this swap selects by the attribute names
alone, so it works on the reference's module classes and on this package's without
importing either.  ``kohakuwullm_amd.MXFP8Linear`` is equally valid as the ``linear_cls``
argument of the reference's own ``swap_mxfp8``.
"""

from __future__ import annotations

from dataclasses import dataclass, field

import torch
import torch.nn as nn

from kohakuwullm_amd.kernels.mxfp8.linear import MXFP8Linear
from kohakuwullm_amd.kernels.mxfp8.quantize import quantize_mx_dual_batch

# Declaration protocol for matmul a module holds as bare parameters: the attribute names
# `swap_mxfp8` looks up, and what `mxfp8_matmul()` returns per tensor.  Field for field the
# reference's protocol (src/kohakuwullm/models/mxfp8_protocol.py:9-27), so a module written
# against either package is discovered by either swap.
DECLARE = "mxfp8_matmul"
CONVERT = "enable_mxfp8"


@dataclass(frozen=True)
class Matmul:
    mac_per_token: int  # multiply-accumulates one token spends against this tensor
    refusal: str | None = None  # why fp8 must not take it, or None
    never: bool = False  # the refusal follows from the tensor's job, not from this model's shapes

ATTN_PROJECTIONS = ("q_proj", "k_proj", "v_proj", "o_proj")
MLP_PROJECTIONS = ("w_in", "gate_proj", "up_proj", "w_out", "fc1", "fc2")
LATENT_PROJECTIONS = ("down", "up")
PROJECTION_NAMES = ATTN_PROJECTIONS + MLP_PROJECTIONS + LATENT_PROJECTIONS

BUCKETS = ("fp8", "skipped", "unreached", "never")


@dataclass
class SwapReport:
    """What the surgery converted, refused and could not reach, with a per-token MAC census."""

    swapped: list[str] = field(default_factory=list)
    modules: list[str] = field(default_factory=list)
    skipped: list[tuple[str, str]] = field(default_factory=list)
    unreached: list[tuple[str, str]] = field(default_factory=list)
    by_design: list[str] = field(default_factory=list)
    unaccounted: list[str] = field(default_factory=list)
    out_of_scope: list[str] = field(default_factory=list)
    mac: dict[str, int] = field(default_factory=lambda: dict.fromkeys(BUCKETS, 0))

    @property
    def blocking(self) -> bool:
        return bool(self.skipped or self.unreached or self.unaccounted)

    @property
    def total_mac(self) -> int:
        return sum(self.mac.values())

    def share(self, bucket: str) -> float:
        total = self.total_mac
        return self.mac[bucket] / total if total else 0.0

    def summary(self) -> str:
        lines = [
            f"MXFP8: {len(self.swapped)} tensor(s) in fp8 over {len(self.modules)} module(s), "
            f"{self.share('fp8'):.1%} of {self.total_mac / 1e6:.1f}M per-token MAC"
        ]
        for label, entries in (("SKIPPED", self.skipped), ("UNREACHED", self.unreached)):
            lines += [f"  {label} {name}: {reason}" for name, reason in entries]
        if self.unaccounted:
            lines.append(f"  UNACCOUNTED: {', '.join(self.unaccounted)}")
        if self.by_design:
            lines.append(f"  bf16 by design: {len(self.by_design)} tensor(s), {self.share('never'):.1%} of per-token MAC")
        return "\n".join(lines)


def _reject(module: nn.Linear) -> str | None:
    if module.bias is not None:
        return "has a bias; MXFP8Linear is bias-free"
    if module.in_features % 128:
        return f"in_features={module.in_features} is not a multiple of 128"
    return None


def _qualify(prefix: str, name: str) -> str:
    return f"{prefix}.{name}" if prefix else name


def _in_scope(qualified: str, scope) -> bool:
    return scope is None or any(part in qualified for part in scope)


def _swap_children(parent, prefix, linear_cls, report, accounted, scope) -> None:
    for name in PROJECTION_NAMES:
        child = getattr(parent, name, None)
        if not isinstance(child, (nn.Linear, linear_cls)):
            continue
        qualified = _qualify(prefix, name)
        mac = child.in_features * child.out_features
        accounted.add(id(child.weight))
        if isinstance(child, linear_cls):  # a second swap over the same model
            report.swapped.append(qualified)
            report.modules.append(qualified)
            report.mac["fp8"] += mac
            continue
        if not _in_scope(qualified, scope):
            report.out_of_scope.append(qualified)
            report.mac["never"] += mac
            continue
        reason = _reject(child)
        if reason is not None:
            report.skipped.append((qualified, reason))
            report.mac["skipped"] += mac
            continue
        replacement = linear_cls(child.in_features, child.out_features, dtype=child.weight.dtype)
        with torch.no_grad():
            replacement.weight.copy_(child.weight)
        replacement.to(child.weight.device)
        setattr(parent, name, replacement)
        accounted.add(id(replacement.weight))
        report.swapped.append(qualified)
        report.modules.append(qualified)
        report.mac["fp8"] += mac


def _resolve_attr(module: nn.Module, path: str):
    obj = module
    for part in path.split("."):
        obj = getattr(obj, part)
    return obj


def _visit_declared(parent, prefix, report, accounted, convert_declared, scope) -> None:
    declared: dict[str, Matmul] = {}
    if isinstance(parent, nn.Embedding):
        declared["weight"] = Matmul(0, "an embedding is a gather, not a GEMM", never=True)
    declare = getattr(parent, DECLARE, None)
    if declare is not None:
        declared.update(declare())
    if not declared:
        return
    for name in declared:
        accounted.add(id(_resolve_attr(parent, name)))
    for name, entry in declared.items():
        if entry.never:
            report.by_design.append(_qualify(prefix, name))
            report.mac["never"] += entry.mac_per_token
    live = {n: e for n, e in declared.items() if not e.never}
    if not _in_scope(prefix, scope):
        for name, entry in live.items():
            report.out_of_scope.append(_qualify(prefix, name))
            report.mac["never"] += entry.mac_per_token
        return
    blocked = {n: e for n, e in live.items() if e.refusal is not None}
    eligible = {n: e for n, e in live.items() if e.refusal is None}
    if blocked:
        for name, entry in blocked.items():
            report.skipped.append((_qualify(prefix, name), entry.refusal))
            report.mac["skipped"] += entry.mac_per_token
        for name, entry in eligible.items():
            report.skipped.append((_qualify(prefix, name), f"a sibling tensor in {prefix or '<root>'} is refused"))
            report.mac["skipped"] += entry.mac_per_token
        return
    if not eligible:
        return
    convert = getattr(parent, CONVERT, None) if convert_declared else None
    if convert is None:
        why = (f"{type(parent).__name__} declares it fp8-eligible but has no {CONVERT}()" if convert_declared
               else "the caller passed convert_declared=False")
        for name, entry in eligible.items():
            report.unreached.append((_qualify(prefix, name), why))
            report.mac["unreached"] += entry.mac_per_token
        return
    convert()
    report.modules.append(prefix)
    for name, entry in eligible.items():
        report.swapped.append(_qualify(prefix, name))
        report.mac["fp8"] += entry.mac_per_token


def swap_mxfp8(model: nn.Module, linear_cls: type = MXFP8Linear, convert_declared: bool = True,
               scope: tuple[str, ...] | None = None) -> SwapReport:
    """Convert every reachable matmul of ``model`` to MXFP8, in place; weights are copied."""
    report = SwapReport()
    accounted: set[int] = set()
    for prefix, parent in list(model.named_modules()):
        if isinstance(parent, linear_cls):
            continue
        _swap_children(parent, prefix, linear_cls, report, accounted, scope)
        _visit_declared(parent, prefix, report, accounted, convert_declared, scope)
    for name, param in model.named_parameters():
        if param.dim() >= 2 and id(param) not in accounted:
            report.unaccounted.append(f"{name}{tuple(param.shape)}")
    return report


def refresh_mxfp8_weights(model: nn.Module) -> int:
    """Requantize every MXFP8 weight cache; call after every optimizer step.  Returns the module count.

    Same contract as the reference (``src/kohakuwullm/models/mxfp8_swap.py:331-343``); the modules
    that describe their cache as dual quantizations of whole matrices (``mxfp8_refresh_plan`` /
    ``mxfp8_install``) are served together, one launch per 24 matrices instead of two launches
    and four allocations per matrix, the others through their own ``refresh_quantized_weight``.
    """
    count = 0
    planned: dict[tuple, list] = {}
    for module in model.modules():
        refresh = getattr(module, "refresh_quantized_weight", None)
        if not callable(refresh):
            continue
        count += 1
        plan_of = getattr(module, "mxfp8_refresh_plan", None)
        plan = plan_of() if callable(plan_of) else None
        if not plan:
            refresh()
            continue
        planned.setdefault((plan[0].device, plan[0].dtype), []).append((module, plan))
    for group in planned.values():
        with torch.no_grad():
            copies = quantize_mx_dual_batch([x for _, plan in group for x in plan])
        at = 0
        for module, plan in group:
            module.mxfp8_install(copies[at : at + len(plan)])
            at += len(plan)
    return count
