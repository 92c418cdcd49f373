"""Pins the oracle's RMSNorm -> MXFP8 producer with checks that do not restate its formula:
torch's own ``rms_norm`` in fp64, closed forms, and the exact scale invariance of the norm."""

import pytest
import torch

from conftest import SEED


def _inputs(m, k, dtype, seed=SEED):
    g = torch.Generator().manual_seed(seed)
    x = (torch.randn(m, k, generator=g) * 3.0).to(dtype)
    w = (1.0 + 0.1 * torch.randn(k, generator=g)).to(dtype)
    return x, w


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("m,k", [(64, 32), (33, 1536), (8, 4096)])
def test_out_matches_library_rms_norm(oracle, m, k, dtype):
    x, w = _inputs(m, k, dtype)
    out, rstd, q, s = oracle.rms_norm_mx(x, w, 1e-6)
    ref = torch.nn.functional.rms_norm(x.double(), (k,), w.double(), 1e-6)
    # the fp32 chain is within a few fp32 ulps of the fp64 value, so rounding to 16 bits agrees
    # except on rounding ties: at most one unit in the last place, almost everywhere none
    ref16 = ref.to(dtype)
    same = (out == ref16).float().mean().item()
    assert same > 0.999
    ulp = torch.finfo(dtype).eps
    assert ((out.double() - ref).abs() <= ulp * ref.abs() + 1e-30).all()
    ref_rstd = 1.0 / torch.sqrt(x.double().square().mean(dim=1) + 1e-6)
    assert torch.allclose(rstd.double(), ref_rstd, rtol=3e-7, atol=0)
    # the codes are those of the fp32 row: dequantized they sit within e4m3 rounding of it
    deq = oracle.dequant(q, s)
    assert oracle.rel_error(deq, ref) < 0.04
    assert ((deq - ref).abs() <= 0.0625 * ref.abs().view(m, k // 32, 32).amax(-1, keepdim=True).expand(m, k // 32, 32).reshape(m, k) + 1e-30).all()


def test_closed_forms(oracle):
    k = 64
    w = torch.linspace(0.5, 2.0, k).bfloat16()
    # a constant row c normalizes to sign(c) * w (eps negligible), whatever c
    for c in (1.0, -4.0, 0.0078125, 1024.0):
        x = torch.full((3, k), c).bfloat16()
        out, rstd, q, s = oracle.rms_norm_mx(x, w, 0.0)
        assert rstd[0].item() == pytest.approx(1.0 / abs(c), rel=1e-6)
        want = w.float() if c > 0 else -w.float()
        assert torch.equal(out.float(), want.expand(3, k))
        q2, s2 = oracle.quantize_rows(want.expand(3, k).contiguous())
        assert torch.equal(q, q2) and torch.equal(s, s2)
    # a zero row: rstd = 1/sqrt(eps), y = 0, the empty-block byte
    out, rstd, q, s = oracle.rms_norm_mx(torch.zeros(2, k).bfloat16(), w, 1e-6)
    assert rstd[0].item() == pytest.approx(1000.0, rel=1e-6)
    assert not out.any() and not q.any() and (s == 19).all()
    # unit basis row: mean = 1/K, y = sqrt(K) * w[j] at j
    x = torch.zeros(1, k).bfloat16()
    x[0, 5] = 1.0
    out, rstd, q, s = oracle.rms_norm_mx(x, None, 0.0)
    assert rstd[0].item() == 8.0 and out[0, 5].item() == 8.0 and out.float().sum().item() == 8.0


def test_power_of_two_scale_invariance(oracle):
    """With eps = 0 the norm of 2^j x equals the norm of x bit for bit: every step scales exactly."""
    x, w = _inputs(40, 512, torch.bfloat16, SEED + 1)
    base = oracle.rms_norm_mx(x, w, 0.0)
    for j in (-20, -3, 7, 30):
        got = oracle.rms_norm_mx((x.float() * 2.0**j).bfloat16(), w, 0.0)
        assert torch.equal(got[0], base[0]) and torch.equal(got[2], base[2]) and torch.equal(got[3], base[3])
        assert torch.equal(got[1] * 2.0**j, base[1])


def test_grads_match_hand_formula(oracle):
    """The autograd oracle against the closed form dx = (dy - xhat mean(dy xhat)) rstd, dw = sum(dout xhat)."""
    x, w = _inputs(17, 96, torch.bfloat16, SEED + 2)
    g = torch.Generator().manual_seed(SEED + 3)
    dout = torch.randn(17, 96, generator=g).bfloat16()
    dx, dw = oracle.rms_norm_grads(x, w, dout, 1e-6)
    xd, wd, dd = x.double(), w.double(), dout.double()
    rstd = 1.0 / torch.sqrt(xd.square().mean(1, keepdim=True) + 1e-6)
    xhat = xd * rstd
    dy = dd * wd
    want_dx = (dy - xhat * (dy * xhat).mean(1, keepdim=True)) * rstd
    assert torch.allclose(dx, want_dx, rtol=1e-10, atol=1e-12)
    assert torch.allclose(dw, (dd * xhat).sum(0), rtol=1e-10, atol=1e-12)
