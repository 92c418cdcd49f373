"""The once-per-step requantization of all weights: the batched dual quantizer against the oracle,
bit for bit, and ``refresh_mxfp8_weights`` against each module's own refresh."""

import pytest
import torch

from conftest import SEED

pytestmark = pytest.mark.gpu
DEV = "cuda:0"

SHAPES = [(32, 32), (96, 160), (128, 128), (160, 96), (4096, 1536), (64, 2048), (2048, 64), (416, 1056), (1536, 4096),
          (32, 4128), (256, 256)]


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
def test_dual_batch_matches_oracle(oracle, dtype):
    """More matrices than one launch takes (24), ragged sizes, edge tiles on both axes."""
    from kohakuwullm_amd.kernels.mxfp8 import quantize_mx_dual_batch

    g = torch.Generator().manual_seed(SEED)
    shapes = (SHAPES * 3)[:29]
    xs = [(torch.randn(m, k, generator=g) * 10.0 ** (j % 5 - 2)).to(dtype) for j, (m, k) in enumerate(shapes)]
    xs[3][0:32, 0:32] = 0.0  # an empty block on both axes
    got = quantize_mx_dual_batch([x.to(DEV) for x in xs])
    assert len(got) == len(xs)
    for x, (q, s, qt, st) in zip(xs, got):
        ref_q, ref_s = oracle.quantize_rows(x)
        ref_qt, ref_st = oracle.quantize_cols(x)
        assert torch.equal(q.view(torch.uint8).cpu(), ref_q) and torch.equal(s.cpu(), ref_s)
        assert torch.equal(qt.view(torch.uint8).cpu(), ref_qt) and torch.equal(st.cpu(), ref_st)
        assert q.is_contiguous() and qt.is_contiguous() and q.dtype == torch.float8_e4m3fn and st.dtype == torch.uint8


def test_dual_batch_views_inputs_and_errors():
    from kohakuwullm_amd import _lib
    from kohakuwullm_amd.kernels.mxfp8 import quantize_mx_dual, quantize_mx_dual_batch

    assert quantize_mx_dual_batch([]) == []
    g = torch.Generator(device=DEV).manual_seed(SEED)
    big = torch.randn(512, 640, device=DEV, generator=g).bfloat16()
    # a row-strided view (a slice of a wider matrix), a transposed view (copied first), an empty matrix
    views = [big[:, 128:384], big.t(), big[:0], big[64:192]]
    got = quantize_mx_dual_batch(views)
    for x, copies in zip(views, got):
        for a, b in zip(copies, quantize_mx_dual(x.contiguous())):
            assert torch.equal(a.view(torch.uint8), b.view(torch.uint8))
    with pytest.raises(ValueError):
        quantize_mx_dual_batch([big, big[:, :48]])
    with pytest.raises(ValueError):
        quantize_mx_dual_batch([big, big.half()])
    with pytest.raises(_lib.MXFP8LibraryError):
        quantize_mx_dual_batch([big.cpu()])


def test_refresh_mxfp8_weights_serves_all_modules_at_once():
    from kohakuwullm_amd import _lib
    from kohakuwullm_amd.kernels.mxfp8.linear import MXFP8Linear
    from kohakuwullm_amd.models.mlp import MXFP8SwiGLU
    from kohakuwullm_amd.models.moe import MoEMLP
    from kohakuwullm_amd.models.mxfp8_swap import refresh_mxfp8_weights, swap_mxfp8

    torch.manual_seed(0)

    class Block(torch.nn.Module):
        def __init__(self):
            super().__init__()
            self.proj = torch.nn.ModuleList(MXFP8Linear(256, n) for n in (256, 384, 100, 1024))  # 100: padded out_features
            self.ffn = MXFP8SwiGLU(256, hidden=512)
            self.moe = MoEMLP(256, hidden=128, num_experts=8, top_k=2, num_shared=0)
            self.moe_small = MoEMLP(256, hidden=96, num_experts=4, top_k=2, num_shared=0)  # 2H = 192 rows per expert: not one matrix, refreshes alone

    model = Block().to(DEV, torch.bfloat16)
    swap_mxfp8(model)
    model.ffn.enable_mxfp8()

    def caches():
        out = [t for lin in model.proj for t in lin._cache]
        out += [t for pair in model.ffn._packed for t in pair]
        for moe in (model.moe, model.moe_small):
            for name in ("in_fwd", "in_dgrad", "out_fwd", "out_dgrad"):
                out += list(getattr(moe._packed, name))
        return out

    # each module on its own
    for module in model.modules():
        if callable(getattr(module, "refresh_quantized_weight", None)):
            module.refresh_quantized_weight()
    alone = [t.clone() for t in caches()]
    with torch.no_grad():
        for p in model.parameters():
            p.mul_(1.5).add_(0.01)
    for module in model.modules():
        if callable(getattr(module, "refresh_quantized_weight", None)):
            module.refresh_quantized_weight()
    moved = [t.clone() for t in caches()]
    assert any(not torch.equal(a.view(torch.uint8), b.view(torch.uint8)) for a, b in zip(alone, moved))
    # all of them through refresh_mxfp8_weights: same bytes, same shapes and strides, few launches
    for lin in model.proj:
        lin._cache = None
    model.ffn._packed = None
    model.moe._packed = model.moe_small._packed = None
    _lib.TIMER = []
    assert refresh_mxfp8_weights(model) == 7
    calls, _lib.TIMER = [name for name, *_ in _lib.TIMER], None
    # one batch for the three plain linears, the feed-forward block and the large MoE; the padded
    # linear (rows + rows of the padded transpose) and the small MoE (per-expert column launches) go alone
    assert calls.count("mx_quantize_dual_batch") == 1
    assert len(calls) == 1 + 2 + 7
    for a, b in zip(moved, caches()):
        assert a.shape == b.shape and a.stride() == b.stride() and a.dtype == b.dtype
        assert torch.equal(a.view(torch.uint8), b.view(torch.uint8))
    # and the modules compute with what was installed
    x = torch.randn(64, 256, device=DEV, dtype=torch.bfloat16)
    for lin in model.proj:
        assert lin(x).shape == (64, lin.out_features)
    assert model.ffn(x).shape == x.shape and model.moe(x).shape == x.shape
