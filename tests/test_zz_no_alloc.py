"""The entry point that allocates nothing (``mx_expert_sort_static``) against the one that takes a caller workspace.

Two calls in a row on the same GPU, the second on a smaller input with another bucket count, so the fixed scratch
still holds the first call's contents when the second starts; results must equal ``mx_expert_sort``'s bit for bit
(integer index work).  A request beyond the fixed capacity is refused before anything is launched.
"""

import pytest
import torch

pytestmark = pytest.mark.gpu

DEV = "cuda:0"


def _both(lib, _lib, flat, buckets, top_k):
    """(offsets, order, token_of, max_rows) from the workspace entry point and from the static one, via the C ABI."""
    n = flat.numel()
    idx_bytes = flat.element_size()
    counts = torch.zeros(buckets, dtype=torch.int32, device=DEV)
    inside = (flat >= 0) & (flat < buckets)
    counts.scatter_add_(0, flat[inside].long(), torch.ones(int(inside.sum()), dtype=torch.int32, device=DEV))
    st = torch.cuda.current_stream().cuda_stream
    results = []
    for static in (False, True):
        offsets = torch.full((buckets + 1,), -7, dtype=torch.int32, device=DEV)
        order = torch.full((n,), -7, dtype=torch.int32, device=DEV)
        token_of = torch.full((n,), -7, dtype=torch.int32, device=DEV)
        max_rows = torch.full((1,), -7, dtype=torch.int32, device=DEV)
        common = (flat.data_ptr(), idx_bytes, n, counts.data_ptr(), top_k, buckets, offsets.data_ptr(), order.data_ptr(),
                  token_of.data_ptr(), max_rows.data_ptr())
        if static:
            _lib.check(lib.mx_expert_sort_static(*common, st), "mx_expert_sort_static")
        else:
            need = lib.mx_expert_sort_workspace(n, buckets)
            ws = torch.empty(need, dtype=torch.int32, device=DEV)
            _lib.check(lib.mx_expert_sort(*common, ws.data_ptr(), need, st), "mx_expert_sort")
        torch.cuda.synchronize()
        results.append((offsets, order, token_of, max_rows))
    return results


def test_static_scratch_sort_equals_workspace_sort(oracle):
    from kohakuwullm_amd import _lib
    from kohakuwullm_amd.kernels.moe import expert_sort, expert_sort_into

    lib = _lib.load()
    g = torch.Generator().manual_seed(20090220)
    # first call: the routing size of the routed-expert benchmark (98304 pairs, 64 experts), int64 picks
    big = torch.randint(0, 64, (98304,), generator=g).to(DEV)
    # second call, right behind it: fewer pairs, fewer buckets, int32 picks, some outside every bucket (dropped)
    small = torch.randint(-1, 8, (5003,), generator=g, dtype=torch.int32).to(DEV)
    for flat, buckets, top_k in ((big, 64, 6), (small, 7, 1), (torch.empty(0, dtype=torch.int64, device=DEV), 5, 2)):
        ref, got = _both(lib, _lib, flat, buckets, top_k)
        for name, a, b in zip(("offsets", "order", "token_of", "max_rows"), ref, got):
            assert torch.equal(a, b), (name, flat.numel(), buckets)
    # against the CPU oracle as well (stable argsort + cumsum), for the large case
    ref, got = _both(lib, _lib, big, 64, 6)
    off, order, token_of = oracle.expert_sort(big.cpu(), 64, 6)
    assert torch.equal(got[0].cpu(), off) and torch.equal(got[1].cpu(), order) and torch.equal(got[2].cpu(), token_of)
    # beyond the fixed array: refused, nothing launched, outputs untouched
    n, buckets = 1 << 20, 1024
    assert lib.mx_expert_sort_workspace(n, buckets) > (1 << 20)
    sentinel = torch.full((buckets + 1,), -7, dtype=torch.int32, device=DEV)
    flat = torch.zeros(n, dtype=torch.int32, device=DEV)
    rc = lib.mx_expert_sort_static(flat.data_ptr(), 4, n, sentinel.data_ptr(), 1, buckets, sentinel.data_ptr(), flat.data_ptr(),
                                   flat.data_ptr(), None, torch.cuda.current_stream().cuda_stream)
    assert rc == _lib.MX_ETOOBIG and b"scratch" in lib.mx_strerror(rc)
    torch.cuda.synchronize()
    assert bool((sentinel == -7).all())
    # the Python wrapper over it writes into the caller's tensors and agrees with expert_sort
    counts = torch.bincount(big, minlength=64).int()
    want = expert_sort(big, counts, 6, 64)
    offsets = torch.empty(65, dtype=torch.int32, device=DEV)
    order = torch.empty(98304, dtype=torch.int32, device=DEV)
    token_of = torch.empty_like(order)
    expert_sort_into(big, counts, 6, 64, offsets, order, token_of)
    assert torch.equal(offsets, want[0]) and torch.equal(order, want[1]) and torch.equal(token_of, want[2])
