"""Pins the oracle's expert dispatch (counts, sort, gated combine and its gradients) with checks
that do not restate its formulas: brute-force Python loops on small cases, the invariants of a
stable sort, torch's own ``index_add`` and autograd."""

import pytest
import torch

from conftest import SEED


def _routing(tokens, top_k, experts, seed=SEED, skew=1.5):
    g = torch.Generator().manual_seed(seed)
    logits = torch.randn(tokens, experts, generator=g) - skew * torch.arange(experts).float().sqrt()
    return logits.topk(top_k, dim=-1).indices.reshape(-1)


@pytest.mark.parametrize("tokens,top_k,experts", [(1, 1, 1), (7, 2, 3), (96, 6, 64), (500, 3, 17)])
def test_expert_sort_invariants_and_brute_force(oracle, tokens, top_k, experts):
    flat = _routing(tokens, top_k, experts)
    counts = oracle.expert_counts(flat, experts)
    offsets, order, token_of = oracle.expert_sort(flat, experts, top_k)
    # brute force: walk the experts, then the pairs in input order
    want_order, want_counts = [], []
    picks = flat.tolist()
    for e in range(experts):
        mine = [i for i, v in enumerate(picks) if v == e]
        want_counts.append(len(mine))
        want_order += mine
    assert counts.tolist() == want_counts and counts.dtype == torch.int32
    assert order.tolist() == want_order
    assert token_of.tolist() == [i // top_k for i in want_order]
    assert offsets.tolist() == [sum(want_counts[:e]) for e in range(experts + 1)]
    # invariants: a permutation, grouped by expert, input order kept inside an expert
    assert sorted(order.tolist()) == list(range(tokens * top_k))
    sorted_expert = flat[order.long()]
    assert (sorted_expert[1:] >= sorted_expert[:-1]).all()
    same = sorted_expert[1:] == sorted_expert[:-1]
    assert (order[1:][same] > order[:-1][same]).all()


def test_expert_counts_ignores_nothing_and_pads(oracle):
    flat = torch.tensor([3, 3, 0, 5, 3], dtype=torch.int64)
    assert oracle.expert_counts(flat, 8).tolist() == [1, 0, 0, 3, 0, 1, 0, 0]
    assert oracle.expert_counts(torch.zeros(0, dtype=torch.int64), 4).tolist() == [0, 0, 0, 0]


def _combine_case(tokens, top_k, experts, dim, dtype, seed=SEED):
    g = torch.Generator().manual_seed(seed + 1)
    flat = _routing(tokens, top_k, experts, seed)
    order = torch.argsort(flat, stable=True).to(torch.int32)
    token_of = (order // top_k).to(torch.int32)
    rows = torch.randn(tokens * top_k, dim, generator=g).to(dtype)
    weight = torch.rand(tokens * top_k, generator=g).add(0.25).to(dtype)
    return rows, weight, order, token_of


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
@pytest.mark.parametrize("valid", [None, 0, 11, 40])
def test_combine_matches_python_loop(oracle, dtype, valid):
    tokens, top_k, dim = 10, 4, 16
    rows, weight, order, token_of = _combine_case(tokens, top_k, 6, dim, dtype)
    got = oracle.combine_routed(rows, weight, order, token_of, tokens, valid)
    want = torch.zeros(tokens, dim, dtype=dtype)
    for p in range(tokens * top_k if valid is None else valid):
        t = int(token_of[p])
        for c in range(dim):
            scaled = torch.tensor(float(rows[p, c]) * float(weight[int(order[p])]), dtype=torch.float32).to(dtype)
            want[t, c] = (want[t, c].float() + scaled.float()).to(dtype)
    assert torch.equal(got, want)


def test_combine_fp32_matches_library_index_add(oracle):
    """The reference's own CPU form, ``zeros.index_add(0, token_of, rows * weight[order])``: in fp32 no
    rounding separates a 16-bit accumulator from a wider one, so the two must agree bit for bit."""
    tokens, top_k, dim = 64, 6, 96
    rows, weight, order, token_of = _combine_case(tokens, top_k, 16, dim, torch.float32)
    got = oracle.combine_routed(rows, weight, order, token_of, tokens)
    scaled = rows * weight.index_select(0, order.long()).reshape(-1, 1)
    want = torch.zeros(tokens, dim).index_add(0, token_of.long(), scaled)
    assert torch.equal(got, want)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_combine_16bit_is_a_chain_of_library_additions(oracle, dtype):
    """With 16-bit rows every addition rounds (the device kernel adds into a 16-bit ``out``,
    moe_dispatch.py:88-90): the same chain written with torch's own 16-bit ``mul`` and ``add``, row by
    row in sorted order.  torch's CPU ``index_add`` keeps a wider accumulator for 16-bit types, so it
    is the comparison only up to the rounding of top_k additions."""
    tokens, top_k, dim = 64, 6, 96
    rows, weight, order, token_of = _combine_case(tokens, top_k, 16, dim, dtype)
    got = oracle.combine_routed(rows, weight, order, token_of, tokens)
    want = torch.zeros(tokens, dim, dtype=dtype)
    for p in range(tokens * top_k):
        want[int(token_of[p])] += rows[p] * weight[int(order[p])]
    assert torch.equal(got, want)
    scaled = rows * weight.index_select(0, order.long()).reshape(-1, 1)
    wide = torch.zeros(tokens, dim, dtype=dtype).index_add(0, token_of.long(), scaled)
    exact = torch.zeros(tokens, dim, dtype=torch.float64).index_add(0, token_of.long(), rows.double() * weight.double()[order.long()][:, None])
    tol = 4e-3 if dtype == torch.bfloat16 else 6e-4
    assert oracle.rel_error(got, exact) < tol and oracle.rel_error(got, wide) < tol
    # a single routed row per token leaves nothing to accumulate: the rounded product itself
    one = oracle.combine_routed(rows[:tokens], weight[:tokens], torch.arange(tokens, dtype=torch.int32),
                                torch.arange(tokens, dtype=torch.int32), tokens)
    assert torch.equal(one, rows[:tokens] * weight[:tokens, None])


@pytest.mark.parametrize("valid", [None, 100])
def test_combine_grads_match_autograd(oracle, valid):
    tokens, top_k, dim = 32, 4, 48
    rows, weight, order, token_of = _combine_case(tokens, top_k, 8, dim, torch.bfloat16)
    g = torch.Generator().manual_seed(SEED + 2)
    grad_out = torch.randn(tokens, dim, generator=g).bfloat16()
    r = rows.double().requires_grad_(True)
    w = weight.double().requires_grad_(True)
    scaled = r * w[order.long()][:, None]
    if valid is not None:
        scaled = torch.where((torch.arange(rows.shape[0]) < valid)[:, None], scaled, torch.zeros_like(scaled))
    out = torch.zeros(tokens, dim, dtype=torch.float64).index_add(0, token_of.long(), scaled)
    out.backward(grad_out.double())
    grad_rows, grad_weight = oracle.combine_routed_grads(grad_out, rows, weight, order, token_of, valid)
    assert torch.allclose(grad_weight, w.grad, rtol=1e-12, atol=1e-12)
    # one product of two 16-bit numbers rounded once: the nearest bf16 of the fp64 gradient
    assert torch.equal(grad_rows, r.grad.to(torch.bfloat16))
