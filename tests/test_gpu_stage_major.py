"""The stage-major code layout (128-column panels, each holding every row): the quantizers write
the same bytes as in the row-major layout, only elsewhere, and the GEMM reads them to the same
result, bit for bit."""

import pytest
import torch

from conftest import SEED

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
F8 = torch.float8_e4m3fn


def _u8(t):
    return t.view(torch.uint8)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
@pytest.mark.parametrize("m,k", [(128, 32), (256, 160), (1024, 1536), (384, 4128)])
def test_quantize_dual_stage_major_holds_the_same_codes(dtype, m, k):
    from kohakuwullm_amd.kernels.mxfp8.quantize import quantize_mx_dual, rows_of_stage_major

    g = torch.Generator(device=DEV).manual_seed(SEED)
    x = (torch.randn(m, k, device=DEV, generator=g) * 3.0).to(dtype)
    q, s, qt, st = quantize_mx_dual(x)
    q2, s2, qt2, st2 = quantize_mx_dual(x, stage_major_t=True)
    assert qt2.shape == (m // 128, k, 128) and qt2.is_contiguous()
    assert torch.equal(_u8(q), _u8(q2)) and torch.equal(s, s2) and torch.equal(st, st2)
    assert torch.equal(_u8(rows_of_stage_major(qt2)), _u8(qt))
    with pytest.raises(ValueError):
        quantize_mx_dual(x[:96], stage_major_t=True)


@pytest.mark.parametrize("m,h", [(128, 128), (256, 384), (1024, 1024)])
def test_swiglu_duals_stage_major_hold_the_same_codes(m, h):
    from kohakuwullm_amd.kernels.mxfp8.mlp import swiglu_bwd_mx_dual, swiglu_mx_dual
    from kohakuwullm_amd.kernels.mxfp8.quantize import rows_of_stage_major

    g = torch.Generator(device=DEV).manual_seed(SEED)
    gu = (torch.randn(m, 2 * h, device=DEV, generator=g) * 1.5).bfloat16()
    dh = (torch.randn(m, h, device=DEV, generator=g) * 1e-2).bfloat16()
    q, s, qt, st = swiglu_mx_dual(gu)
    q2, s2, qt2, st2 = swiglu_mx_dual(gu, stage_major_t=True)
    assert qt2.shape == (m // 128, h, 128)
    assert torch.equal(_u8(q), _u8(q2)) and torch.equal(s, s2) and torch.equal(st, st2)
    assert torch.equal(_u8(rows_of_stage_major(qt2)), _u8(qt))
    pq, ps, ptq, pts = swiglu_bwd_mx_dual(dh, gu)
    pq2, ps2, ptq2, pts2 = swiglu_bwd_mx_dual(dh, gu, stage_major=True)
    assert pq2.shape == (2 * h // 128, m, 128) and ptq2.shape == (m // 128, 2 * h, 128)
    assert torch.equal(ps, ps2) and torch.equal(pts, pts2)
    assert torch.equal(_u8(rows_of_stage_major(pq2)), _u8(pq))
    assert torch.equal(_u8(rows_of_stage_major(ptq2)), _u8(ptq))
    if h % 128 == 0 and m > 128:
        with pytest.raises(ValueError):
            swiglu_bwd_mx_dual(dh[:, :96].contiguous(), gu[:, : 2 * 96].contiguous(), stage_major=True)


def _to_stage_major(codes):
    rows, cols = codes.shape
    return codes.view(rows, cols // 128, 128).permute(1, 0, 2).contiguous()


@pytest.mark.parametrize("m,n,k", [(256, 256, 256), (300, 520, 1024), (1024, 1536, 16384), (8192, 1536, 2048), (96, 4096, 8192)])
def test_gemm_reads_stage_major_operands_to_the_same_bits(m, n, k):
    """Row-major and stage-major operands give identical outputs: same kernel, same order of additions
    (whole tiles, the even K split of a partial round, and the K slices of a shared launch)."""
    from kohakuwullm_amd.kernels.mxfp8.quantize import mxfp8_matmul_pq_batch

    g = torch.Generator(device=DEV).manual_seed(SEED)
    aq = torch.randint(0, 127, (m, k), device=DEV, dtype=torch.uint8, generator=g).view(F8)
    bq = torch.randint(0, 127, (n, k), device=DEV, dtype=torch.uint8, generator=g).view(F8)
    a_s = torch.randint(118, 130, (m, k // 32), device=DEV, dtype=torch.uint8, generator=g)
    b_s = torch.randint(118, 130, (n, k // 32), device=DEV, dtype=torch.uint8, generator=g)
    (ref,) = mxfp8_matmul_pq_batch([(aq, a_s, bq, b_s)])
    a3, b3 = _to_stage_major(aq), _to_stage_major(bq)
    for a, b in ((a3, bq), (aq, b3), (a3, b3)):
        (out,) = mxfp8_matmul_pq_batch([(a, a_s, b, b_s)])
        assert torch.equal(out, ref)
    # several products in one call, layouts mixed: the plan (XCD shares, K slices) depends on the shapes
    # only, so the same call with row-major operands adds in the same order
    outs = mxfp8_matmul_pq_batch([(a3, a_s, b3, b_s), (aq, a_s, bq, b_s), (a3, a_s, bq, b_s)], torch.float32)
    refs = mxfp8_matmul_pq_batch([(aq, a_s, bq, b_s)] * 3, torch.float32)
    for out, ref32 in zip(outs, refs):
        assert torch.equal(out, ref32)


def test_mlp_backward_uses_stage_major_operands_and_matches_the_row_major_path(monkeypatch):
    from kohakuwullm_amd.kernels.mxfp8 import mlp
    from kohakuwullm_amd.kernels.mxfp8.quantize import quantize_mx, quantize_mx_cols

    g = torch.Generator(device=DEV).manual_seed(SEED)
    tokens, dim, hidden = 512, 256, 384
    x = torch.randn(tokens, dim, device=DEV, generator=g).bfloat16()
    w_in = (torch.randn(2 * hidden, dim, device=DEV, generator=g) * 0.05).bfloat16()
    w_out = (torch.randn(dim, hidden, device=DEV, generator=g) * 0.05).bfloat16()
    dy = (torch.randn(tokens, dim, device=DEV, generator=g) * 1e-2).bfloat16()
    packed = (quantize_mx(w_in), quantize_mx_cols(w_in), quantize_mx(w_out), quantize_mx_cols(w_out))

    def run():
        xs, wi, wo = (t.clone().requires_grad_(True) for t in (x, w_in, w_out))
        y = mlp.mxfp8_swiglu_mlp(xs, wi, wo, packed)
        y.backward(dy)
        return y.detach(), xs.grad, wi.grad, wo.grad

    seen = []
    real = mlp.swiglu_bwd_mx_dual
    monkeypatch.setattr(mlp, "swiglu_bwd_mx_dual", lambda dh, gu, stage_major=False: (seen.append(stage_major), real(dh, gu, stage_major))[1])
    with_panels = run()
    assert seen == [True]
    monkeypatch.setattr(mlp, "stage_major_ok", lambda cols: False)
    row_major = run()
    assert seen == [True, False]
    for a, b in zip(with_panels, row_major):
        assert torch.equal(a, b)
