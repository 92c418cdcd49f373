"""RMSNorm -> MXFP8 producer on the GPU against the oracle, through the C ABI.

The arithmetic after the (fp64, order-insensitive) sum of squares is the same sequence of fp32
operations on both sides, so rstd, the 16-bit output, the codes and the scale bytes are expected
to be identical; the assertions allow a row to differ only where its rstd differs, which takes
an fp64 rounding difference that lands exactly on an fp32 rounding boundary.
"""

import pytest
import torch

from conftest import SEED

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
F8 = torch.float8_e4m3fn


def _inputs(m, k, dtype, wdtype, seed=SEED):
    g = torch.Generator().manual_seed(seed)
    x = (torch.randn(m, k, generator=g) * 3.0).to(dtype)
    if m > 2:
        x[1] = 0.0  # a zero row
        x[2] *= 2.0**-60  # a tiny row: eps dominates
    w = None if wdtype is None else (1.0 + 0.1 * torch.randn(k, generator=g)).to(wdtype)
    return x, w


def _compare(oracle, x, w, eps, out, rstd, q, s):
    ref_out, ref_rstd, ref_q, ref_s = oracle.rms_norm_mx(x, w, eps)
    rows_ok = rstd.cpu() == ref_rstd
    assert rows_ok.float().mean().item() >= 1.0 - 1e-4, "rstd differs on more rows than fp64 summation order explains"
    assert torch.allclose(rstd.cpu(), ref_rstd, rtol=2e-7, atol=0)
    if out is not None:
        assert torch.equal(out.cpu()[rows_ok], ref_out[rows_ok])
        assert oracle.rel_error(out.cpu(), ref_out) < 1e-3
    if q is not None:
        assert torch.equal(q.view(torch.uint8).cpu()[rows_ok], ref_q[rows_ok])
        assert torch.equal(s.cpu()[rows_ok], ref_s[rows_ok])
    return rows_ok


SHAPES = [(1, 32), (5, 64), (37, 96), (64, 512), (130, 1536), (33, 2048), (9, 2560), (17, 4096), (6, 5120), (3, 16416)]


@pytest.mark.parametrize("m,k", SHAPES)
@pytest.mark.parametrize("dtype,wdtype", [(torch.bfloat16, torch.bfloat16), (torch.float16, torch.float32), (torch.bfloat16, None)])
def test_rms_norm_mx_matches_oracle(oracle, m, k, dtype, wdtype):
    from kohakuwullm_amd.kernels.elementwise import rms_norm_mx

    x, w = _inputs(m, k, dtype, wdtype)
    out, q, s = rms_norm_mx(x.to(DEV), None if w is None else w.to(DEV), 1e-6)
    assert out.shape == x.shape and out.dtype == dtype and q.dtype == F8 and q.shape == (m, k) and s.shape == (m, k // 32)
    # rstd is not returned by the reference's API either: read it through the plain launcher
    from kohakuwullm_amd.kernels.elementwise.rmsnorm import launch_rmsnorm

    rstd = torch.empty(m, device=DEV, dtype=torch.float32)
    launch_rmsnorm(x.to(DEV), None if w is None else w.to(DEV), 1e-6, None, rstd, torch.empty_like(q), torch.empty_like(s))
    _compare(oracle, x, w, 1e-6, out, rstd, q, s)


def test_outputs_are_independent_and_pitched_rows_work(oracle):
    """Each of out / rstd / (q, s) alone gives what it gives together; row pitches larger than K are honoured."""
    from kohakuwullm_amd.kernels.elementwise.rmsnorm import launch_rmsnorm
    from kohakuwullm_amd.kernels.mxfp8.fused_act import rmsnorm_mx

    m, k = 45, 1536
    x, w = _inputs(m, k, torch.bfloat16, torch.bfloat16, SEED + 5)
    wide = torch.zeros(m, k + 64, dtype=torch.bfloat16)
    wide[:, :k] = x
    xd, wd = wide.to(DEV)[:, :k], w.to(DEV)
    out = torch.full((m, k + 8), 7.0, device=DEV, dtype=torch.bfloat16)
    q = torch.zeros(m, k + 32, device=DEV, dtype=F8)
    s = torch.zeros(m, k // 32 + 3, device=DEV, dtype=torch.uint8)  # a pitch that is not a multiple of 4: byte stores
    rstd = torch.zeros(m, device=DEV)
    launch_rmsnorm(xd, wd, 1e-5, out[:, :k], rstd, q[:, :k], s[:, : k // 32])
    ok = _compare(oracle, x, w, 1e-5, out[:, :k], rstd, q[:, :k], s[:, : k // 32])
    assert ok.all()
    assert (out[:, k:] == 7.0).all() and not q.view(torch.uint8)[:, k:].any() and not s[:, k // 32 :].any()
    out2 = torch.empty(m, k, device=DEV, dtype=torch.bfloat16)
    launch_rmsnorm(xd, wd, 1e-5, out2, None, None, None)
    assert torch.equal(out2, out[:, :k])
    q2, s2 = rmsnorm_mx(x.to(DEV), wd, 1e-5)
    assert torch.equal(q2.view(torch.uint8), q[:, :k].view(torch.uint8)) and torch.equal(s2, s[:, : k // 32])


def test_vendor_layout_and_errors(oracle):
    from kohakuwullm_amd.kernels.elementwise import rms_norm, rms_norm_mx, rms_norm_mx_vendor

    m, k = 200, 256
    x, w = _inputs(m, k, torch.bfloat16, torch.bfloat16, SEED + 6)
    out, q, s = rms_norm_mx(x.to(DEV), w.to(DEV))
    out_v, q_v, s_v = rms_norm_mx_vendor(x.to(DEV), w.to(DEV))
    assert torch.equal(out, out_v) and torch.equal(q.view(torch.uint8), q_v.view(torch.uint8))
    assert torch.equal(s_v.view(torch.uint8).cpu(), oracle.swizzle_32_4_4(s.cpu()))
    assert torch.equal(rms_norm(x.to(DEV), w.to(DEV)), out)
    with pytest.raises(ValueError):
        rms_norm_mx(x.to(DEV)[:, :40].contiguous(), w.to(DEV)[:40].contiguous())  # K % 32
    with pytest.raises(ValueError):
        rms_norm_mx_vendor(x.to(DEV)[:, :96].contiguous(), w.to(DEV)[:96].contiguous())  # K % 128
    with pytest.raises(Exception):
        rms_norm(x, w)  # CPU tensors: no CPU route
    with pytest.raises(ValueError):
        rms_norm(x.to(DEV), w.to(DEV)[:-1])


@pytest.mark.parametrize("m,k,wdtype", [(300, 1536, torch.bfloat16), (7, 96, torch.float32), (2100, 2048, None), (64, 4096, torch.bfloat16)])
def test_backward_matches_autograd_oracle(oracle, m, k, wdtype):
    from kohakuwullm_amd.kernels.elementwise import rms_norm_mx

    x, w = _inputs(m, k, torch.bfloat16, wdtype, SEED + 8)
    g = torch.Generator().manual_seed(SEED + 9)
    dout = torch.randn(m, k, generator=g).bfloat16()
    xd = x.to(DEV).requires_grad_(True)
    wd = None if w is None else w.to(DEV).requires_grad_(True)
    out, q, s = rms_norm_mx(xd, wd, 1e-6)
    assert not q.requires_grad and not s.requires_grad
    out.backward(dout.to(DEV))
    ref_dx, ref_dw = oracle.rms_norm_grads(x, w, dout, 1e-6)
    # row 2 is scaled by 2^-60: its dx is huge (rstd ~ 1e3 relative to x ~ 1e-18) but finite; compare per row
    got = xd.grad.cpu().double()
    num = (got - ref_dx).norm(dim=1)
    den = ref_dx.norm(dim=1).clamp_min(1e-30)
    assert (num / den).max().item() < 1e-2  # bf16 outputs of fp32 arithmetic
    if w is not None:
        assert wd.grad.dtype == wdtype
        assert oracle.rel_error(wd.grad.cpu(), ref_dw) < 1e-2


@pytest.mark.parametrize("m,k", [(32, 32), (64, 96), (160, 1536), (256, 2048), (384, 4096), (96, 5120)])
@pytest.mark.parametrize("dtype,wdtype", [(torch.bfloat16, torch.bfloat16), (torch.float16, torch.float32), (torch.bfloat16, None)])
def test_rmsnorm_mx_dual_matches_oracle(oracle, m, k, dtype, wdtype):
    """Both operands of the linear layer behind the norm from one call: the row-axis pair is the oracle's
    rms_norm_mx, the token-axis pair the oracle's column quantizer on the same fp32 normalized values (formed with
    the oracle's rstd in the kernel's order: (x * rstd) * w, one fp32 rounding per product); the stage-major layout
    holds the same bytes.  Rows whose rstd differs from the oracle's (an fp64 rounding on an fp32 boundary) are
    excluded from the bit comparison as in the row-axis test; none is expected."""
    from kohakuwullm_amd.kernels.mxfp8.fused_act import rmsnorm_mx, rmsnorm_mx_dual

    x, w = _inputs(m, k, dtype, wdtype)
    xd, wd = x.to(DEV), None if w is None else w.to(DEV)
    q, s, qt, st, rstd = rmsnorm_mx_dual(xd, wd, 1e-6)
    assert q.shape == (m, k) and s.shape == (m, k // 32) and qt.shape == (k, m) and st.shape == (k, m // 32)
    rows_ok = _compare(oracle, x, w, 1e-6, None, rstd, q, s)
    assert bool(rows_ok.all())
    _, ref_rstd, _, _ = oracle.rms_norm_mx(x, w, 1e-6)
    y = x.float() * ref_rstd[:, None]
    if w is not None:
        y = y * w.float()
    ref_qt, ref_st = oracle.quantize_cols(y)
    assert torch.equal(qt.view(torch.uint8).cpu(), ref_qt) and torch.equal(st.cpu(), ref_st)
    # the same row-axis bytes as the single-axis producer
    q1, s1 = rmsnorm_mx(xd, wd, 1e-6)
    assert torch.equal(q.view(torch.uint8), q1.view(torch.uint8)) and torch.equal(s, s1)
    if m % 128 == 0 and m > 128:
        _, _, panels, st2, _ = rmsnorm_mx_dual(xd, wd, 1e-6, stage_major_t=True)
        assert panels.shape == (m // 128, k, 128) and torch.equal(st2, st)
        assert torch.equal(panels.view(torch.uint8).permute(1, 0, 2).reshape(k, m), qt.view(torch.uint8))


def test_rmsnorm_mx_dual_full_width_and_errors(oracle):
    """The hidden-state matrix of the attention configuration (32768 x 2048), against the device's own single-axis
    producer and column quantizer (bit-exact against the oracle themselves); refusals."""
    from kohakuwullm_amd.kernels.mxfp8.fused_act import rmsnorm_mx, rmsnorm_mx_dual
    from kohakuwullm_amd.kernels.mxfp8.quantize import quantize_mx_cols

    x, w = _inputs(32768, 2048, torch.bfloat16, torch.bfloat16)
    xd, wd = x.to(DEV), w.to(DEV)
    q, s, qt, st, rstd = rmsnorm_mx_dual(xd, wd, 1e-6)
    q1, s1 = rmsnorm_mx(xd, wd, 1e-6)
    assert torch.equal(q.view(torch.uint8), q1.view(torch.uint8)) and torch.equal(s, s1)
    y = (xd.float() * rstd[:, None]) * wd.float()
    qt1, st1 = quantize_mx_cols(y)
    assert torch.equal(qt.view(torch.uint8), qt1.view(torch.uint8)) and torch.equal(st, st1)
    with pytest.raises(ValueError):
        rmsnorm_mx_dual(xd[:33], wd)  # tokens not a multiple of 32
    with pytest.raises(ValueError):
        rmsnorm_mx_dual(xd[:128], wd, stage_major_t=True)  # one panel is not a stage-major matrix
    with pytest.raises(Exception):
        rmsnorm_mx_dual(x, w)  # CPU tensors: there is no CPU path
