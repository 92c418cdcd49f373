"""The vendor (cuBLAS SWIZZLE_32_4_4) scale layout as an exchange format.

Byte permutations are compared bit for bit with the CPU oracle, which is itself pinned against the
documented view/permute chain of the reference (tests/test_oracle_quantize.py).
"""

import pytest
import torch

from conftest import SEED

pytestmark = pytest.mark.gpu

DEV = "cuda:0"
F8 = torch.float8_e4m3fn


@pytest.mark.parametrize("rows,cols", [(300, 10), (128, 4), (1, 1), (4096, 16), (129, 5), (1000, 48)])
def test_swizzle_and_back(oracle, rows, cols):
    from kohakuwullm_amd.kernels.mxfp8.interop import expected_swizzled_numel, swizzle_mx_scales, unswizzle_mx_scales

    g = torch.Generator().manual_seed(SEED)
    s = torch.randint(1, 255, (rows, cols), dtype=torch.uint8, generator=g)
    got = swizzle_mx_scales(s.to(DEV))
    assert got.numel() == expected_swizzled_numel(rows, cols * 32) and got.dtype == torch.uint8
    assert torch.equal(got.cpu(), oracle.swizzle_32_4_4(s))
    assert torch.equal(unswizzle_mx_scales(got, rows, cols * 32).cpu(), s)
    # a row-strided view (a slice of a wider scale matrix) is read in place
    wide = torch.randint(1, 255, (rows, cols + 3), dtype=torch.uint8, generator=g)
    assert torch.equal(swizzle_mx_scales(wide.to(DEV)[:, :cols]).cpu(), oracle.swizzle_32_4_4(wide[:, :cols].contiguous()))


def test_quantize_mx_vendor(oracle):
    from kohakuwullm_amd.kernels.mxfp8 import quantize_mx, quantize_mx_vendor

    g = torch.Generator().manual_seed(SEED)
    x = torch.randn(300, 640, generator=g).bfloat16()
    q, sv = quantize_mx_vendor(x.to(DEV))
    rq, rs = oracle.quantize_rows(x)
    assert q.dtype == F8 and torch.equal(q.view(torch.uint8).cpu(), rq)
    assert sv.dtype == getattr(torch, "float8_e8m0fnu", torch.uint8) and sv.dim() == 1
    assert torch.equal(sv.view(torch.uint8).cpu(), oracle.swizzle_32_4_4(rs))
    # a transposed view is quantized along its own last axis without a copy
    xt = torch.randn(640, 384, generator=g).bfloat16()
    qt, svt = quantize_mx_vendor(xt.to(DEV).t())
    rq2, rs2 = oracle.quantize_rows(xt.t().contiguous())
    assert torch.equal(qt.view(torch.uint8).cpu(), rq2) and torch.equal(svt.view(torch.uint8).cpu(), oracle.swizzle_32_4_4(rs2))
    assert torch.equal(quantize_mx(xt.to(DEV).t())[0], qt)
    with pytest.raises(ValueError):
        quantize_mx_vendor(torch.zeros(8, 96, device=DEV, dtype=torch.bfloat16))


def test_vendor_matmul_routes(oracle):
    from kohakuwullm_amd.kernels.mxfp8 import mxfp8_matmul_pq
    from kohakuwullm_amd.kernels.mxfp8.interop import (
        as_vendor_scales,
        mxfp8_mm_swizzled,
        vendor_mxfp8_matmul,
        vendor_mxfp8_matmul_swizzled,
    )

    g = torch.Generator().manual_seed(SEED)
    a = torch.randn(300, 512, generator=g).bfloat16()
    b = (torch.randn(200, 512, generator=g) * 0.02).bfloat16()
    aq, as_ = oracle.quantize_rows(a)
    bq, bs = oracle.quantize_rows(b)
    ref = oracle.gemm_nt(aq, as_, bq, bs)
    daq, das, dbq, dbs = aq.to(DEV).view(F8), as_.to(DEV), bq.to(DEV).view(F8), bs.to(DEV)
    base = mxfp8_matmul_pq(daq, das, dbq, dbs)
    for out in (
        vendor_mxfp8_matmul(daq, das, dbq, dbs),
        vendor_mxfp8_matmul_swizzled(daq, as_vendor_scales(das), dbq, as_vendor_scales(dbs)),
        mxfp8_mm_swizzled(daq, as_vendor_scales(das), dbq, as_vendor_scales(dbs)),
        torch.ops.kohakuwullm_amd.mxfp8_mm_swizzled(daq, as_vendor_scales(das), dbq, as_vendor_scales(dbs), torch.bfloat16),
    ):
        assert torch.equal(out, base)  # the same GEMM on the same natural scales
    assert oracle.rel_error(base.cpu(), ref) < 1e-2
    out32 = mxfp8_mm_swizzled(daq, as_vendor_scales(das), dbq, as_vendor_scales(dbs), torch.float32)
    assert out32.dtype == torch.float32 and oracle.rel_error(out32.cpu(), ref) < 1e-4
    with pytest.raises(ValueError):
        vendor_mxfp8_matmul_swizzled(daq, as_vendor_scales(das)[:-4], dbq, as_vendor_scales(dbs))


def test_mm_swizzled_fake_shape():
    """The registered fake gives tracing its output shape and dtype without touching data."""
    from torch._subclasses.fake_tensor import FakeTensorMode

    from kohakuwullm_amd.kernels.mxfp8.interop import expected_swizzled_numel, mxfp8_mm_swizzled

    with FakeTensorMode():
        aq = torch.empty(256, 512, dtype=F8, device=DEV)
        bq = torch.empty(384, 512, dtype=F8, device=DEV)
        sa = torch.empty(expected_swizzled_numel(256, 512), dtype=torch.uint8, device=DEV)
        sb = torch.empty(expected_swizzled_numel(384, 512), dtype=torch.uint8, device=DEV)
        out = mxfp8_mm_swizzled(aq, sa, bq, sb, torch.float16)
        assert out.shape == (256, 384) and out.dtype == torch.float16


def test_expert_combine_direct(oracle):
    """The gather-combine against index_add in fp64, with dropped pairs and an empty expert; bit-reproducible."""
    from kohakuwullm_amd.kernels.mxfp8.moe import combine_sorted_rows

    g = torch.Generator().manual_seed(SEED)
    tokens, top_k, n, e = 96, 3, 256, 5
    pairs = tokens * top_k
    expert = torch.randint(0, e + 1, (pairs,), generator=g)  # expert id e = dropped (sentinel bucket)
    expert[expert == 2] = 3  # expert 2 stays empty
    order = torch.argsort(expert, stable=True).int()
    counts = torch.bincount(expert, minlength=e + 1)[:e]
    offsets = torch.zeros(e + 1, dtype=torch.int32)
    offsets[1:] = counts.cumsum(0)
    m_real = int(offsets[-1])
    y = torch.randn(pairs, n, generator=g).bfloat16()
    y[m_real:] = float("nan")  # rows of the sentinel bucket must never be read
    gate = (torch.rand(pairs, generator=g) + 0.5).bfloat16()
    ref = torch.zeros(tokens, n, dtype=torch.float64)
    idx = order[:m_real].long()
    ref.index_add_(0, idx // top_k, y[:m_real].double() * gate[idx].double()[:, None])
    for gt, want in ((gate, ref), (None, torch.zeros(tokens, n, dtype=torch.float64).index_add_(0, idx // top_k, y[:m_real].double()))):
        outs = [combine_sorted_rows(y.to(DEV), order.to(DEV), offsets.to(DEV), e, None if gt is None else gt.to(DEV), tokens, top_k)
                for _ in range(2)]
        assert torch.equal(outs[0], outs[1]) and outs[0].dtype == torch.bfloat16
        assert oracle.rel_error(outs[0].cpu(), want) < 4e-3  # one bf16 rounding of an fp32 sum
        # the pair -> position table of one call serves a later call for the same routing
        gd = None if gt is None else gt.to(DEV)
        out_a, pos = combine_sorted_rows(y.to(DEV), order.to(DEV), offsets.to(DEV), e, gd, tokens, top_k, return_positions=True)
        out_b = combine_sorted_rows(y.to(DEV), None, offsets.to(DEV), e, gd, tokens, top_k, positions=pos)
        assert torch.equal(out_a, outs[0]) and torch.equal(out_b, outs[0])
        inv = pos.cpu()
        assert torch.equal(inv[order[:m_real].long()], torch.arange(m_real, dtype=torch.int32))
        assert (inv[order[m_real:].long()] == -1).all()
