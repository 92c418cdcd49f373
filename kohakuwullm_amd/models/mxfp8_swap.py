"""Replace a built model's projections with MXFP8 linears, in place, and account for it.

Behaviour follows ``src/kohakuwullm/models/mxfp8_swap.py`` of the reference
(``swap_mxfp8`` :301-328, ``refresh_mxfp8_weights`` :331-343, ``SwapReport`` :41-103,
refusal rule :106-113): ``nn.Linear`` children with the projection attribute names are
replaced by ``linear_cls(in_features, out_features, dtype=weight.dtype)`` with the weight
copied; modules that declare bare-parameter matmuls through ``mxfp8_matmul()`` are
converted with ``enable_mxfp8()``; anything matmul-shaped that nobody claimed blocks.

Where the reference selects parents by class, this swap selects by the attribute names
alone, so it works on the reference's module classes and on this package's without
importing either -- and converts an ``nn.Linear`` called ``up``, ``fc1``, ... under ANY parent,
which the reference would leave alone; pass ``scope`` to keep it to the blocks that are meant.  ``kohakuwullm_amd.MXFP8Linear`` is equally valid as the ``linear_cls``
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
    """What the surgery converted, refused and could not reach, with a per-token MAC census.

    Field names and meaning are the reference's (``mxfp8_swap.py:41-103``): ``swapped`` names tensors,
    ``modules`` the modules that hold an fp8 cache (what ``refresh_mxfp8_weights`` counts); ``skipped``,
    ``unreached`` and ``unaccounted`` block a run, ``by_design`` and ``out_of_scope`` do not.
    """

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
        return any((self.skipped, self.unreached, self.unaccounted))

    @property
    def total_mac(self) -> int:
        return sum(self.mac.values())

    def share(self, bucket: str) -> float:
        return self.mac[bucket] / self.total_mac if self.total_mac else 0.0

    def summary(self) -> str:
        """A few lines for a log: the fp8 share first, then every finding that blocks, then what stays 16-bit on purpose."""
        out = [f"MXFP8 swap: {len(self.swapped)} tensors / {len(self.modules)} modules now fp8 = "
               f"{self.share('fp8'):.1%} of {self.total_mac / 1e6:.1f}M MAC per token"]
        findings = [("skipped", name, why) for name, why in self.skipped]
        findings += [("unreached", name, why) for name, why in self.unreached]
        findings += [("unaccounted", name, "a matmul-shaped parameter nobody declared") for name in self.unaccounted]
        out += [f"  BLOCKING [{kind}] {name}: {why}" for kind, name, why in findings]
        for bucket in ("skipped", "unreached"):
            if self.mac[bucket]:
                out.append(f"  {bucket}: {self.mac[bucket] / 1e6:.1f}M MAC per token ({self.share(bucket):.1%})")
        kept = len(self.by_design) + len(self.out_of_scope)
        if kept:
            out.append(f"  16-bit on purpose: {len(self.by_design)} by design, {len(self.out_of_scope)} out of scope "
                       f"({self.share('never'):.1%} of MAC)")
        return "\n".join(out)


def _reject(module: nn.Linear) -> str | None:
    """Why ``MXFP8Linear`` cannot stand in for this layer (the reference's two rules and wording, ``mxfp8_swap.py:106-113``)."""
    if module.bias is not None:
        return "has a bias; MXFP8Linear is bias-free"
    if module.in_features % 128:
        return f"in_features={module.in_features} is not a multiple of 128"
    return None


class _Census:
    """The report under construction plus the set of parameters somebody has answered for."""

    def __init__(self, scope) -> None:
        self.report = SwapReport()
        self.scope = scope
        self._claimed: set[int] = set()

    def claim(self, tensor) -> None:
        self._claimed.add(id(tensor))

    def claimed(self, tensor) -> bool:
        return id(tensor) in self._claimed

    def wanted(self, qualified: str) -> bool:
        return self.scope is None or any(part in qualified for part in self.scope)

    def book(self, outcome: str, name: str, mac: int, why: str | None = None) -> None:
        """Enter one tensor under one of: fp8, skipped, unreached, by_design, out_of_scope."""
        r = self.report
        if outcome == "fp8":
            r.swapped.append(name)
        elif outcome == "skipped":
            r.skipped.append((name, why))
        elif outcome == "unreached":
            r.unreached.append((name, why))
        elif outcome == "by_design":
            r.by_design.append(name)
        else:
            r.out_of_scope.append(name)
        r.mac[outcome if outcome in BUCKETS else "never"] += mac


def _join(prefix: str, name: str) -> str:
    return f"{prefix}.{name}" if prefix else name


def _convert_linears(parent: nn.Module, prefix: str, linear_cls: type, census: _Census) -> None:
    """The projection-named ``nn.Linear`` children of ``parent``: replace the ones ``linear_cls`` can stand in for."""
    for name, child in list(parent.named_children()):
        if name not in PROJECTION_NAMES or not isinstance(child, (nn.Linear, linear_cls)):
            continue
        where, mac = _join(prefix, name), child.in_features * child.out_features
        census.claim(child.weight)
        if isinstance(child, linear_cls):  # converted by an earlier swap of the same model
            outcome, why = "fp8", None
        elif not census.wanted(where):
            outcome, why = "out_of_scope", None
        else:
            why = _reject(child)
            outcome = "skipped" if why else "fp8"
        if outcome == "fp8" and not isinstance(child, linear_cls):
            stand_in = linear_cls(child.in_features, child.out_features, dtype=child.weight.dtype)
            with torch.no_grad():
                stand_in.weight.copy_(child.weight)  # the A/B arms must start from identical weights
            setattr(parent, name, stand_in.to(child.weight.device))
            census.claim(stand_in.weight)
        census.book(outcome, where, mac, why)
        if outcome == "fp8":
            census.report.modules.append(where)


def _declarations(parent: nn.Module) -> dict[str, Matmul]:
    """What ``parent`` says about the matmuls it holds as bare parameters (an embedding speaks for itself)."""
    said: dict[str, Matmul] = {}
    if isinstance(parent, nn.Embedding):
        said["weight"] = Matmul(0, "an embedding is a gather, not a GEMM", never=True)
    # The LM head (src/kohakuwullm/models/mxfp8_swap.py:133-139 names its class; here: a module whose class is called
    # LMHead and that holds a bare (vocab, dim) ``projection``) stays 16-bit by design.
    projection = getattr(parent, "projection", None)
    if type(parent).__name__ == "LMHead" and isinstance(projection, nn.Parameter) and projection.dim() == 2:
        vocab, dim = projection.shape
        said["projection"] = Matmul(vocab * dim, "the head contracts over the vocabulary", never=True)
    declare = getattr(parent, DECLARE, None)
    if callable(declare):
        said.update(declare())
    return said


def _convert_declared(parent: nn.Module, prefix: str, census: _Census, convert_declared: bool) -> None:
    """Account for the tensors ``parent`` declares; convert them when all that may go to fp8 can."""
    said = _declarations(parent)
    open_cases: list[tuple[str, Matmul]] = []
    for name, entry in said.items():
        tensor = parent
        for part in name.split("."):  # a declaration may name a child's tensor ("router.weight")
            tensor = getattr(tensor, part)
        census.claim(tensor)
        if entry.never:
            census.book("by_design", _join(prefix, name), entry.mac_per_token)
        else:
            open_cases.append((_join(prefix, name), entry))
    if not open_cases:
        return
    if not census.wanted(prefix):
        ruling = lambda entry: ("out_of_scope", None)  # noqa: E731
    elif any(entry.refusal for _, entry in open_cases):
        # one refused tensor keeps the whole module in 16 bits; its siblings point at it
        sibling = f"a sibling tensor in {prefix or '<root>'} is refused"
        ruling = lambda entry: ("skipped", entry.refusal or sibling)  # noqa: E731
    elif not convert_declared:
        ruling = lambda entry: ("unreached", "the caller passed convert_declared=False")  # noqa: E731
    elif not callable(getattr(parent, CONVERT, None)):
        missing = f"{type(parent).__name__} declares it fp8-eligible but has no {CONVERT}()"
        ruling = lambda entry: ("unreached", missing)  # noqa: E731
    else:
        getattr(parent, CONVERT)()
        census.report.modules.append(prefix)
        ruling = lambda entry: ("fp8", None)  # noqa: E731
    for where, entry in open_cases:
        outcome, why = ruling(entry)
        census.book(outcome, where, entry.mac_per_token, why)


def swap_mxfp8(model: nn.Module, linear_cls: type = MXFP8Linear, convert_declared: bool = True,
               scope: tuple[str, ...] | None = None) -> SwapReport:
    """Convert every reachable matmul of ``model`` to MXFP8, in place; weights are copied.

    ``scope``: substrings of qualified names to restrict the conversion to (the rest is reported as
    ``out_of_scope`` and does not block).  ``convert_declared=False`` leaves declared bare-parameter
    matmuls alone and reports them ``unreached``.  Signature and outcomes as ``mxfp8_swap.py:301-328``.
    """
    census = _Census(scope)
    for prefix, parent in list(model.named_modules()):
        if isinstance(parent, linear_cls):
            continue
        _convert_linears(parent, prefix, linear_cls, census)
        _convert_declared(parent, prefix, census, convert_declared)
    census.report.unaccounted += [f"{name}{tuple(p.shape)}" for name, p in model.named_parameters()
                                  if p.dim() >= 2 and not census.claimed(p)]
    return census.report


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
