"""Expert dispatch on the GPU against the oracle, through the C ABI: the histogram, the stable
grouping by expert and the gated combine are index / byte work and must match bit for bit; the
per-pair gate gradient is an fp32 dot product and is held to 1e-5 relative."""

import pytest
import torch

from conftest import SEED

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def _picks(tokens, top_k, experts, seed=SEED, skew=1.5, dtype=torch.int64):
    g = torch.Generator().manual_seed(seed)
    logits = torch.randn(tokens, experts, generator=g) - skew * torch.arange(experts).float().sqrt()
    return logits.topk(top_k, dim=-1).indices.reshape(-1).to(dtype)


@pytest.mark.parametrize("dtype", [torch.int64, torch.int32])
@pytest.mark.parametrize("n,buckets", [(0, 4), (1, 1), (1000, 3), (98304, 64), (98304, 65), (300001, 8192)])
def test_expert_counts(oracle, n, buckets, dtype):
    from kohakuwullm_amd.kernels.moe import expert_counts

    g = torch.Generator().manual_seed(SEED)
    flat = torch.randint(0, buckets, (n,), generator=g).to(dtype)
    counts = expert_counts(flat.to(DEV), buckets)
    assert counts.dtype == torch.int32 and torch.equal(counts.cpu(), oracle.expert_counts(flat, buckets))


def test_expert_counts_skips_out_of_range_and_rejects_bad_input():
    from kohakuwullm_amd import _lib
    from kohakuwullm_amd.kernels.moe import expert_counts

    flat = torch.tensor([0, 5, -1, 2, 7, 2], device=DEV)
    assert expert_counts(flat, 4).tolist() == [1, 0, 2, 0]
    with pytest.raises(ValueError):
        expert_counts(flat.float(), 4)
    with pytest.raises(_lib.MXFP8LibraryError):
        expert_counts(flat.cpu(), 4)
    with pytest.raises(_lib.MXFP8LibraryError):
        expert_counts(flat, 10000)


@pytest.mark.parametrize("tokens,top_k,experts", [
    (1, 1, 1), (7, 2, 3), (43, 3, 5), (96, 6, 64), (16384, 6, 64), (16384, 6, 65), (4096, 8, 1024), (300000, 6, 128),
])
@pytest.mark.parametrize("dtype", [torch.int64, torch.int32])
def test_expert_sort_is_the_stable_sort(oracle, tokens, top_k, experts, dtype):
    from kohakuwullm_amd.kernels.moe import expert_counts, expert_sort

    flat = _picks(tokens, min(top_k, experts), experts, dtype=dtype)
    slots = flat.numel() // tokens
    dev = flat.to(DEV)
    counts = expert_counts(dev, experts)
    offsets, order, token_of, max_rows = expert_sort(dev, counts, slots, experts)
    ref_offsets, ref_order, ref_token = oracle.expert_sort(flat, experts, slots)
    assert torch.equal(offsets.cpu(), ref_offsets)
    assert torch.equal(order.cpu(), ref_order)
    assert torch.equal(token_of.cpu(), ref_token)
    assert max_rows.item() == int(counts.max())
    again = expert_sort(dev, counts, slots, experts)
    assert torch.equal(again[1], order) and torch.equal(again[2], token_of)


def test_expert_sort_edge_cases(oracle):
    from kohakuwullm_amd.kernels.moe import expert_sort

    # no pairs at all
    counts = torch.zeros(4, dtype=torch.int32, device=DEV)
    offsets, order, token_of, max_rows = expert_sort(torch.zeros(0, dtype=torch.int64, device=DEV), counts, 2, 4)
    assert offsets.tolist() == [0] * 5 and order.numel() == 0 and token_of.numel() == 0 and max_rows.item() == 0
    # every pair on one expert, the others empty (leading, interior and trailing empties)
    flat = torch.full((5000,), 2, dtype=torch.int64)
    counts = torch.tensor([0, 0, 5000, 0], dtype=torch.int32, device=DEV)
    offsets, order, token_of, _ = expert_sort(flat.to(DEV), counts, 5, 4)
    assert offsets.tolist() == [0, 0, 0, 5000, 5000] and torch.equal(order.cpu(), torch.arange(5000, dtype=torch.int32))
    assert torch.equal(token_of.cpu(), torch.arange(5000, dtype=torch.int32) // 5)
    # a sentinel bucket: picks of the padding slots land past the last real expert
    flat = torch.tensor([3, 0, 3, 1, 0, 3], dtype=torch.int64)
    counts = torch.tensor([2, 1, 0, 3], dtype=torch.int32, device=DEV)
    offsets, order, token_of, _ = expert_sort(flat.to(DEV), counts, 2, 4)
    assert offsets.tolist() == [0, 2, 3, 3, 6] and order.tolist() == [1, 4, 3, 0, 2, 5] and token_of.tolist() == [0, 2, 1, 0, 1, 2]
    # a histogram that overstates the picks points past the end: those positions are dropped, not written
    flat = _picks(512, 2, 8)
    counts = (oracle.expert_counts(flat, 8) * 3).to(DEV)
    offsets, order, token_of, _ = expert_sort(flat.to(DEV), counts, 2, 8)
    torch.cuda.synchronize()
    assert offsets.tolist() == [0] + counts.cpu().cumsum(0).tolist()
    with pytest.raises(ValueError):
        expert_sort(flat.to(DEV), counts[:4], 2, 8)
    with pytest.raises(ValueError):
        expert_sort(flat.to(DEV), counts.long(), 2, 8)


def _combine_case(tokens, top_k, experts, dim, dtype, wdtype, seed=SEED):
    g = torch.Generator().manual_seed(seed + 1)
    flat = _picks(tokens, top_k, experts, seed)
    order = torch.argsort(flat, stable=True).to(torch.int32)
    token_of = (order // top_k).to(torch.int32)
    rows = torch.randn(tokens * top_k, dim, generator=g).to(dtype)
    weight = torch.rand(tokens * top_k, generator=g).add(0.25).to(wdtype)
    grad_out = torch.randn(tokens, dim, generator=g).to(dtype)
    return rows, weight, order, token_of, grad_out


@pytest.mark.parametrize("dtype,wdtype", [
    (torch.bfloat16, torch.bfloat16), (torch.bfloat16, torch.float32), (torch.float16, torch.float16),
    (torch.float16, torch.float32), (torch.float32, torch.float32),
])
@pytest.mark.parametrize("tokens,top_k,experts,dim", [(1, 1, 1, 8), (10, 4, 6, 16), (333, 6, 64, 1024), (2048, 2, 8, 520)])
def test_combine_routed_forward_backward(oracle, dtype, wdtype, tokens, top_k, experts, dim):
    from kohakuwullm_amd.kernels.moe import combine_routed

    rows, weight, order, token_of, grad_out = _combine_case(tokens, top_k, experts, dim, dtype, wdtype)
    n = tokens * top_k
    for valid in (None, n // 3):
        r = rows.to(DEV).requires_grad_(True)
        w = weight.to(DEV).requires_grad_(True)
        bound = None if valid is None else torch.tensor([valid], dtype=torch.int32, device=DEV)
        out = combine_routed(r, w, order.to(DEV), token_of.to(DEV), tokens, bound)
        assert torch.equal(out.cpu(), oracle.combine_routed(rows, weight, order, token_of, tokens, valid))
        out.backward(grad_out.to(DEV))
        ref_rows, ref_weight = oracle.combine_routed_grads(grad_out, rows, weight, order, token_of, valid)
        assert torch.equal(r.grad.cpu(), ref_rows)
        assert w.grad.dtype == wdtype
        # fp32 dot products of `dim` terms; a 16-bit gate gradient is that rounded once more
        tol = 1e-5 if wdtype == torch.float32 else (8e-3 if wdtype == torch.bfloat16 else 1e-3)
        assert oracle.rel_error(w.grad.cpu(), ref_weight) < tol
        if valid is not None:
            assert not w.grad.cpu()[order[valid:].long()].any()


def test_combine_routed_partial_routing(oracle):
    """Fewer sorted rows than pairs (some pairs were routed nowhere): they add nothing and get a zero gate gradient."""
    from kohakuwullm_amd.kernels.moe import combine_routed

    tokens, top_k, dim = 200, 4, 256
    rows, weight, order, token_of, grad_out = _combine_case(tokens, top_k, 12, dim, torch.bfloat16, torch.float32)
    for n in (0, 1, 517):
        r = rows[:n].to(DEV).requires_grad_(True)
        w = weight.to(DEV).requires_grad_(True)
        out = combine_routed(r, w, order[:n].to(DEV), token_of[:n].to(DEV), tokens)
        assert torch.equal(out.cpu(), oracle.combine_routed(rows[:n], weight, order[:n], token_of[:n], tokens))
        out.backward(grad_out.to(DEV))
        ref_rows, ref_weight = oracle.combine_routed_grads(grad_out, rows[:n], weight, order[:n], token_of[:n])
        assert torch.equal(r.grad.cpu(), ref_rows) and w.grad.shape == weight.shape
        assert torch.allclose(w.grad.cpu().double(), ref_weight, rtol=1e-4, atol=1e-4)
        assert not w.grad.cpu()[order[n:].long()].any()


def test_combine_routed_full_size_properties(oracle):
    """The routed-expert benchmark's shape (16384 tokens, top-6, 1024 wide): a sum, whatever the routing."""
    from kohakuwullm_amd.kernels.moe import combine_routed, expert_counts, expert_sort

    tokens, top_k, experts, dim = 16384, 6, 64, 1024
    flat = _picks(tokens, top_k, experts).to(DEV)
    _, order, token_of, _ = expert_sort(flat, expert_counts(flat, experts), top_k, experts)
    g = torch.Generator(device=DEV).manual_seed(SEED)
    rows = torch.randn(tokens * top_k, dim, device=DEV, generator=g).bfloat16()
    weight = torch.rand(tokens * top_k, device=DEV, generator=g).add(0.25)
    out = combine_routed(rows, weight, order, token_of, tokens)
    assert torch.equal(out, combine_routed(rows, weight, order, token_of, tokens))
    inv = torch.empty_like(order, dtype=torch.int64)
    inv[order.long()] = torch.arange(order.numel(), device=DEV)
    exact = (rows[inv].double() * weight.double()[:, None]).view(tokens, top_k, dim).sum(1)
    assert oracle.rel_error(out.cpu(), exact.cpu()) < 4e-3
    # linear in the gate: doubling every weight doubles every rounded product and every partial sum
    assert torch.equal(combine_routed(rows, weight * 2, order, token_of, tokens), out * 2)
    # a permutation of the slots of a token (another routing of the same rows) changes only rounding
    ones = torch.ones_like(weight)
    first = combine_routed(rows, ones, order, token_of, tokens)
    assert oracle.rel_error(first.cpu(), rows[inv].double().view(tokens, top_k, dim).sum(1).cpu()) < 4e-3


def test_combine_routed_rejects_bad_input():
    from kohakuwullm_amd import _lib
    from kohakuwullm_amd.kernels.moe import combine_routed

    rows = torch.zeros(12, 16, device=DEV, dtype=torch.bfloat16)
    weight = torch.ones(12, device=DEV)
    idx = torch.arange(12, device=DEV, dtype=torch.int32)
    with pytest.raises(ValueError):
        combine_routed(rows, weight, idx[:6], idx, 4)
    with pytest.raises(ValueError):
        combine_routed(rows, weight, idx, idx, 5)
    with pytest.raises(ValueError):
        combine_routed(rows, weight.double(), idx, idx, 4)
    with pytest.raises(ValueError):
        combine_routed(rows, weight, idx.long(), idx, 4)
    with pytest.raises(_lib.MXFP8LibraryError):
        combine_routed(rows.cpu(), weight.cpu(), idx.cpu(), idx.cpu(), 4)
    with pytest.raises(_lib.MXFP8LibraryError):
        combine_routed(rows[:, :12], weight, idx, idx // 3, 4)  # width not a multiple of 8
