"""Expert-sort indices for the routed experts and the gated combine, on the HIP kernels.

Counterpart of ``src/kohakuwullm/kernels/moe/moe_dispatch.py`` (``expert_sort`` :223-261,
``combine_routed`` / ``_Combine`` :134-200) and of ``expert_counts``
(``src/kohakuwullm/models/components/moe.py:38-46``); same names, arguments and return values.

Differences from the reference, on purpose: the tensors must live on the GPU (a CPU tensor
raises: there is no second implementation to fall back to); the order inside an expert is the
input order (a stable sort) and the combine adds a token's rows in sorted-position order with
one writer per element, so both give the bits of the reference's own sort-based forms
(``expert_sort_reference`` :264-282, ``combine_routed_reference`` :203-220) on every run, where
the reference's device path depends on the order in which atomics land.  ``combine_routed``
needs ``order`` to be a permutation of the pair indices ``token * slots + slot`` with
``token_of = order // slots`` -- what ``expert_sort`` returns -- or a part of one (pairs that
were routed nowhere add nothing).
"""

from __future__ import annotations

import torch

from kohakuwullm_amd import _lib

_INDEX = {torch.int32: 4, torch.int64: 8}
_ROWS = (torch.bfloat16, torch.float16, torch.float32)


def _index_tensor(t: torch.Tensor, name: str) -> torch.Tensor:
    _lib.require_gpu(t, name)
    if t.dtype not in _INDEX:
        raise ValueError(f"{name}.dtype={t.dtype} is not int32 or int64")
    if t.dim() != 1:
        raise ValueError(f"{name} must be flat, got shape {tuple(t.shape)}")
    return t.contiguous()


def expert_counts(flat_idx: torch.Tensor, num_buckets: int) -> torch.Tensor:
    """``(num_buckets,)`` int32 rows per bucket, from a flat ``(T * slots,)`` index.  No host sync."""
    flat_idx = _index_tensor(flat_idx, "flat_idx")
    counts = torch.empty(num_buckets, dtype=torch.int32, device=flat_idx.device)
    n = flat_idx.numel()
    _lib.invoke("mx_expert_counts", n * flat_idx.element_size(), flat_idx,
                flat_idx.data_ptr(), _INDEX[flat_idx.dtype], n, num_buckets, counts.data_ptr())
    return counts


def expert_sort(flat_expert: torch.Tensor, counts: torch.Tensor, top_k: int, num_experts: int):
    """Group ``(token, slot)`` pairs by expert using their known histogram.

    Args:
        flat_expert: ``(T * top_k,)`` expert id per pair (int32 or int64).
        counts: ``(E,)`` int32 rows per expert, as returned by the router / ``expert_counts``.
        top_k: slots per token, used to recover the token from a pair index.
        num_experts: E (buckets, a sentinel bucket included when the router has one).

    Returns:
        ``(offsets, order, token_of, max_rows)``, all int32 on the device: ``offsets (E + 1,)``
        for the grouped GEMM, ``order`` sorted position -> pair index, ``token_of`` sorted
        position -> token index, ``max_rows`` a one-element diagnostic (largest count).
    """
    flat_expert = _index_tensor(flat_expert, "flat_expert")
    _lib.require_gpu(counts, "counts")
    if counts.dtype != torch.int32 or counts.shape != (num_experts,):
        raise ValueError(f"counts must be int32 of shape ({num_experts},), got {counts.dtype} {tuple(counts.shape)}")
    if top_k <= 0:
        raise ValueError(f"top_k={top_k} must be positive")
    n, device = flat_expert.numel(), flat_expert.device
    counts = counts.contiguous()
    offsets = torch.empty(num_experts + 1, dtype=torch.int32, device=device)
    order = torch.empty(n, dtype=torch.int32, device=device)
    token_of = torch.empty(n, dtype=torch.int32, device=device)
    max_rows = torch.empty(1, dtype=torch.int32, device=device)
    need = _lib.load().mx_expert_sort_workspace(n, num_experts)
    if need < 0:
        raise ValueError(f"expert_sort: {n} pairs in {num_experts} buckets is out of range")
    workspace = torch.empty(need, dtype=torch.int32, device=device)
    _lib.invoke("mx_expert_sort", n * (flat_expert.element_size() + 8), flat_expert,
                flat_expert.data_ptr(), _INDEX[flat_expert.dtype], n, counts.data_ptr(), top_k, num_experts,
                offsets.data_ptr(), order.data_ptr(), token_of.data_ptr(), max_rows.data_ptr(),
                workspace.data_ptr(), need)
    return offsets, order, token_of, max_rows


def expert_sort_into(flat_expert: torch.Tensor, counts: torch.Tensor, top_k: int, num_experts: int,
                     offsets: torch.Tensor, order: torch.Tensor, token_of: torch.Tensor) -> None:
    """:func:`expert_sort` into tensors the caller already holds, through the library entry point that allocates nothing.

    For loops whose buffers were sized once and that must not allocate per call (neither here nor in the
    library): ``offsets (E + 1,)``, ``order (n,)``, ``token_of (n,)`` int32 are overwritten; the scratch is a
    fixed 4 MiB array inside the library (requests beyond it raise; none with 256 buckets or fewer does).
    The results are those of :func:`expert_sort`, bit for bit.  Calls on one GPU share the scratch: issue them
    on one stream, or serialise them.
    """
    flat_expert = _index_tensor(flat_expert, "flat_expert")
    n = flat_expert.numel()
    for t, shape, name in ((counts, (num_experts,), "counts"), (offsets, (num_experts + 1,), "offsets"), (order, (n,), "order"),
                           (token_of, (n,), "token_of")):
        _lib.require_gpu(t, name)
        if t.dtype != torch.int32 or tuple(t.shape) != shape or not t.is_contiguous():
            raise ValueError(f"{name} must be a contiguous int32 tensor of shape {shape}, got {t.dtype} {tuple(t.shape)}")
    if top_k <= 0:
        raise ValueError(f"top_k={top_k} must be positive")
    _lib.invoke("mx_expert_sort_static", n * (flat_expert.element_size() + 8), flat_expert,
                flat_expert.data_ptr(), _INDEX[flat_expert.dtype], n, counts.data_ptr(), top_k, num_experts,
                offsets.data_ptr(), order.data_ptr(), token_of.data_ptr(), None)


def _valid_ptr(valid_rows, device) -> int:
    if valid_rows is None:
        return 0
    if valid_rows.device != device or valid_rows.dtype != torch.int32 or valid_rows.numel() != 1:
        raise ValueError("valid_rows must be a one-element int32 tensor on the rows' device")
    return valid_rows.data_ptr()


class _Combine(torch.autograd.Function):
    @staticmethod
    def forward(ctx, rows, weight, order, token_of, num_tokens, valid_rows):
        n, dim = rows.shape
        pairs = weight.numel()
        out = torch.empty(num_tokens, dim, dtype=rows.dtype, device=rows.device)
        inv = torch.empty(pairs, dtype=torch.int32, device=rows.device)
        _lib.invoke("mx_combine_routed", rows.element_size() * dim * (n + num_tokens), rows,
                    rows.data_ptr(), _lib.MX_DTYPE[rows.dtype], rows.stride(0), weight.data_ptr(),
                    _lib.MX_DTYPE[weight.dtype], order.data_ptr(), _valid_ptr(valid_rows, rows.device), inv.data_ptr(),
                    n, dim, num_tokens, pairs // num_tokens, out.data_ptr(), out.stride(0))
        ctx.save_for_backward(rows, weight, order, token_of, valid_rows)
        return out

    @staticmethod
    def backward(ctx, grad_out):
        rows, weight, order, token_of, valid_rows = ctx.saved_tensors
        n, dim = rows.shape
        grad_out = grad_out.contiguous()
        grad_rows = torch.empty_like(rows)
        grad_weight = torch.empty(weight.numel(), dtype=torch.float32, device=rows.device)
        _lib.invoke("mx_combine_routed_backward", rows.element_size() * dim * (2 * n + grad_out.shape[0]), rows,
                    grad_out.data_ptr(), grad_out.stride(0), rows.data_ptr(), rows.stride(0), _lib.MX_DTYPE[rows.dtype],
                    weight.data_ptr(), _lib.MX_DTYPE[weight.dtype], order.data_ptr(), token_of.data_ptr(),
                    _valid_ptr(valid_rows, rows.device), n, dim, grad_out.shape[0], weight.numel(),
                    grad_rows.data_ptr(), grad_rows.stride(0), grad_weight.data_ptr())
        return grad_rows, grad_weight.to(weight.dtype), None, None, None, None


def combine_routed(rows: torch.Tensor, weight: torch.Tensor, order: torch.Tensor, token_of: torch.Tensor,
                   num_tokens: int, valid_rows: torch.Tensor | None = None) -> torch.Tensor:
    """Scale each routed row by its gate weight and sum it back onto its token.

    Args:
        rows: ``(T * top_k, D)`` expert outputs in sorted order.
        weight: ``(T * top_k,)`` gate weights, indexed by pair index; its length fixes ``top_k``.
        order: sorted position -> pair index.
        token_of: sorted position -> token index.
        num_tokens: T, the row count of the returned tensor.
        valid_rows: one-element device tensor; sorted positions at or past it are skipped as
            uncomputed.  ``None`` means every row is valid.  Never read on the host.
    """
    if rows.shape[0] != order.numel():
        raise ValueError(f"rows {rows.shape[0]} != order {order.numel()}")
    _lib.require_gpu(rows, "rows")
    if rows.dim() != 2 or rows.dtype not in _ROWS:
        raise ValueError(f"rows must be 2-D bf16 / fp16 / fp32, got {rows.dtype} {tuple(rows.shape)}")
    if weight.dtype not in _ROWS or weight.device != rows.device:
        raise ValueError(f"weight must be bf16 / fp16 / fp32 on {rows.device}, got {weight.dtype} on {weight.device}")
    if num_tokens <= 0 or weight.numel() % num_tokens or rows.shape[0] > weight.numel():
        raise ValueError(f"{weight.numel()} gate weights are not a whole number of slots for {num_tokens} tokens, "
                         f"or fewer than the {rows.shape[0]} routed rows")
    for name, t in (("order", order), ("token_of", token_of)):
        if t.dtype != torch.int32 or t.device != rows.device or t.numel() != rows.shape[0]:
            raise ValueError(f"{name} must be int32 of {rows.shape[0]} entries on {rows.device}")
    return _Combine.apply(rows.contiguous(), weight.contiguous().reshape(-1), order.contiguous(), token_of.contiguous(),
                          num_tokens, valid_rows)
