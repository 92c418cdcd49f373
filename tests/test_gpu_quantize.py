"""Parity of the HIP quantizers with the CPU oracle: bit-exact codes and scales.

Calls go through the C ABI (ctypes -> libmxfp8_hip.so).  Inputs are drawn on a CPU
generator and copied to the device so both sides see the same bits.
"""

import pytest
import torch

from conftest import SEED

from mx_checks import assert_codes_equal_up_to_ties  # noqa: E402

pytestmark = pytest.mark.gpu

DEV = "cuda:0"


def _mx():
    from kohakuwullm_amd.kernels import mxfp8

    return mxfp8


def _rand(shape, dtype, scale=1.0, seed=SEED):
    g = torch.Generator().manual_seed(seed)
    return (torch.randn(*shape, generator=g) * scale).to(dtype)


def _eq(got, ref, what):
    got = got.view(torch.uint8).cpu()
    if not torch.equal(got, ref):
        bad = (got != ref).nonzero()
        raise AssertionError(f"{what}: {bad.shape[0]} mismatches, first at {bad[0].tolist()}: got {got[tuple(bad[0])]} ref {ref[tuple(bad[0])]}")


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
@pytest.mark.parametrize("shape", [(1, 32), (3, 96), (8, 1024), (257, 160), (96, 4096), (1000, 512)])
def test_rows_bit_exact(oracle, dtype, shape):
    x = _rand(shape, dtype, 1.0)
    q, s = _mx().quantize_mx(x.to(DEV))
    qr, sr = oracle.quantize_rows(x)
    assert q.dtype == torch.float8_e4m3fn and s.dtype == torch.uint8
    _eq(s, sr, "scales")
    _eq(q, qr, "codes")


@pytest.mark.parametrize("scale", [0.02, 1e-2, 1e-2 * 2.0**-20, 300.0, 1e30])
def test_rows_scales_of_magnitude(oracle, scale):
    x = _rand((64, 512), torch.bfloat16, scale)
    q, s = _mx().quantize_mx(x.to(DEV))
    qr, sr = oracle.quantize_rows(x)
    _eq(s, sr, "scales")
    _eq(q, qr, "codes")


def test_rows_every_bf16_value(oracle):
    """Each finite bf16 value as the amax of a block, with every other finite bf16 value beside it."""
    bits = torch.arange(0, 1 << 16, dtype=torch.int32).to(torch.int16).view(torch.bfloat16)
    finite = bits[torch.isfinite(bits.float())]
    n = finite.numel()  # 65280
    g = torch.Generator().manual_seed(SEED)
    # block = [amax candidate, 31 random finite values]; 2040 rows x 32 blocks
    x = finite[torch.randint(0, n, (n, 32), generator=g)]
    x[:, 0] = finite
    x = x.reshape(-1, 1024).contiguous()
    q, s = _mx().quantize_mx(x.to(DEV))
    qr, sr = oracle.quantize_rows(x)
    _eq(s, sr, "scales")
    _eq(q, qr, "codes")


def test_rows_edge_blocks(oracle):
    x = _rand((16, 256), torch.bfloat16)
    x[0, :32] = 0.0
    x[1, 32:64] = 1e-35
    x[2, 64] = 3.0e38
    x[2, 65] = -3.0e38
    x[3, :32] = 0.0
    x[3, 5] = -448.0 * 8
    x[4, 96:128] = -0.0
    x[5, 128:160] = 2.0**-133  # bf16 subnormal
    q, s = _mx().quantize_mx(x.to(DEV))
    qr, sr = oracle.quantize_rows(x)
    _eq(s, sr, "scales")
    _eq(q, qr, "codes")
    assert s[0, 0] == 19 and s[2, 2] == 247 and s[3, 0] == 130


def test_rows_strided_views(oracle):
    base = _rand((320, 384), torch.bfloat16, 2.0)
    dev = base.to(DEV)
    # row-pitch view
    q, s = _mx().quantize_mx(dev[:, 64:320])
    qr, sr = oracle.quantize_rows(base[:, 64:320])
    _eq(s, sr, "pitch scales")
    _eq(q, qr, "pitch codes")
    # transposed view: no copy, column kernel underneath
    q, s = _mx().quantize_mx(dev.t())
    qr, sr = oracle.quantize_rows(base.t())
    _eq(s, sr, "transposed scales")
    _eq(q, qr, "transposed codes")
    # doubly strided view: generic kernel
    q, s = _mx().quantize_mx(dev[::2, ::2][:, :160])
    qr, sr = oracle.quantize_rows(base[::2, ::2][:, :160])
    _eq(s, sr, "generic scales")
    _eq(q, qr, "generic codes")


def test_rows_errors():
    mx = _mx()
    with pytest.raises(ValueError):
        mx.quantize_mx(torch.zeros(4, 48, dtype=torch.bfloat16, device=DEV))
    with pytest.raises(ValueError):
        mx.quantize_mx_cols(torch.zeros(48, 64, dtype=torch.bfloat16, device=DEV))
    q, s = mx.quantize_mx(torch.zeros(0, 64, dtype=torch.bfloat16, device=DEV))
    assert q.shape == (0, 64) and s.shape == (0, 2)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
@pytest.mark.parametrize("shape", [(32, 8), (64, 128), (160, 136), (128, 1000), (1024, 384), (96, 2048)])
def test_cols_bit_exact(oracle, dtype, shape):
    x = _rand(shape, dtype, 1.5)
    qt, st = _mx().quantize_mx_cols(x.to(DEV))
    qr, sr = oracle.quantize_cols(x)
    assert qt.shape == (shape[1], shape[0]) and st.shape == (shape[1], shape[0] // 32)
    _eq(st, sr, "scales")
    _eq(qt, qr, "codes")


def test_cols_unaligned_falls_back(oracle):
    x = _rand((64, 100), torch.bfloat16)  # K % 8 != 0 -> generic path
    qt, st = _mx().quantize_mx_cols(x.to(DEV))
    qr, sr = oracle.quantize_cols(x)
    _eq(st, sr, "scales")
    _eq(qt, qr, "codes")


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("shape", [(32, 32), (128, 128), (160, 96), (512, 1536), (96, 4096)])
def test_dual_bit_exact(oracle, dtype, shape):
    x = _rand(shape, dtype, 0.7)
    q, s, qt, st = _mx().quantize_mx_dual(x.to(DEV))
    qr, sr = oracle.quantize_rows(x)
    qtr, str_ = oracle.quantize_cols(x)
    _eq(s, sr, "row scales")
    _eq(q, qr, "row codes")
    _eq(st, str_, "col scales")
    _eq(qt, qtr, "col codes")


def test_swiglu_mx(oracle):
    from kohakuwullm_amd.kernels.mxfp8.fused_act import swiglu_mx

    g = _rand((200, 512), torch.bfloat16, 2.0, seed=3)
    u = _rand((200, 512), torch.bfloat16, 1.0, seed=4)
    q, s = swiglu_mx(g.to(DEV), u.to(DEV))
    qr, sr = oracle.swiglu_quantize_rows(g, u)
    q, s = q.view(torch.uint8).cpu(), s.cpu()
    act = g.float() * torch.sigmoid(g.float()) * u.float()
    # the device sigmoid uses the hardware exp/rcp: a value a few fp32 ulp away can fall on the other side of
    # a rounding boundary.  Only such ties may differ, and few of them.
    n_q, n_s = assert_codes_equal_up_to_ties(oracle, q, s, act, what="swiglu_mx")
    assert n_s < 1e-3 * s.numel() and n_q < 5e-3 * q.numel()
    assert (s != sr).sum() <= n_s + 1 and (q != qr).float().mean() < 5e-3  # the C oracle's libm agrees with torch's to the same ties
    assert oracle.rel_error(oracle.dequant(q, s), act) < 0.04
    # chunked halves of one projection, as GLUMLP produces them
    both = torch.cat([g, u], dim=1).to(DEV)
    gh, uh = both.chunk(2, dim=-1)
    q2, s2 = swiglu_mx(gh, uh)
    assert torch.equal(q2.view(torch.uint8).cpu(), q) and torch.equal(s2.cpu(), s)


def test_full_size_properties(oracle):
    """The 546M-dense activation shape: invariants that need no CPU pass over the whole tensor."""
    mx = _mx()
    g = torch.Generator().manual_seed(SEED)
    x = torch.randn(16384, 1536, generator=g).bfloat16()
    dev = x.to(DEV)
    q, s, qt, st = mx.quantize_mx_dual(dev)
    q1, s1 = mx.quantize_mx(dev)
    qt1, st1 = mx.quantize_mx_cols(dev)
    assert torch.equal(q.view(torch.uint8), q1.view(torch.uint8)) and torch.equal(s, s1)
    assert torch.equal(qt.view(torch.uint8), qt1.view(torch.uint8)) and torch.equal(st, st1)
    # columns == rows of the materialised transpose
    q2, s2 = mx.quantize_mx(dev.t().contiguous())
    assert torch.equal(qt.view(torch.uint8), q2.view(torch.uint8)) and torch.equal(st, s2)
    # a seeded row sample against the oracle
    rows = torch.randint(0, 16384, (64,), generator=g)
    qr, sr = oracle.quantize_rows(x[rows].contiguous())
    _eq(q[rows.to(DEV)], qr, "sampled codes")
    _eq(s[rows.to(DEV)], sr, "sampled scales")
    # block amax lands in the top binade of its scale
    deq = q.float().reshape(16384, -1, 32).abs().amax(-1)
    assert (deq <= 448).all() and (deq >= 224).all()


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
@pytest.mark.parametrize("t,h,d", [(1, 1, 32), (77, 3, 64), (500, 16, 128), (33, 5, 96), (4096, 4, 128)])
def test_quantize_heads_matches_oracle(oracle, dtype, t, h, d):
    from kohakuwullm_amd.kernels.mxfp8.attention_quant import column_mean, quantize_heads

    g = torch.Generator().manual_seed(SEED)
    x = (torch.randn(t, h, d, generator=g) * 3.0 + 0.5).to(dtype)
    if t > 2:
        x[1] = 0.0
    mu = torch.randn(h, d, generator=g)
    for shift in (None, mu):
        q, s = quantize_heads(x.to(DEV), None if shift is None else shift.to(DEV))
        ref_q, ref_s = oracle.quantize_heads(x, shift)
        assert q.shape == (t, h, d) and s.shape == (t, h, d // 32) and q.dtype == torch.float8_e4m3fn
        assert torch.equal(q.view(torch.uint8).cpu(), ref_q) and torch.equal(s.cpu(), ref_s)
    assert torch.allclose(column_mean(x.to(DEV)).cpu(), x.float().mean(0), atol=1e-5) and column_mean(x.to(DEV)).dtype == torch.float32


def test_quantize_heads_reads_projection_slices_in_place_and_checks_input(oracle):
    """q / k of a fused (T, (Hq + 2 Hkv) D) projection output, quantized where they lie; odd layouts are copied."""
    from kohakuwullm_amd import _lib
    from kohakuwullm_amd.kernels.mxfp8.attention_quant import quantize_heads

    g = torch.Generator().manual_seed(SEED)
    t, hq, hkv, d = 300, 16, 4, 128
    qkv = torch.randn(t, (hq + 2 * hkv) * d, generator=g).bfloat16()
    dev = qkv.to(DEV)
    parts = {"q": (0, hq), "k": (hq * d, hkv)}
    for lo, heads in parts.values():
        view = dev[:, lo : lo + heads * d].view(t, heads, d)
        assert not view.is_contiguous()
        _lib.TIMER = []
        q, s = quantize_heads(view)
        calls, _lib.TIMER = _lib.TIMER, None
        assert [c[0] for c in calls] == ["mx_quantize_heads"]
        ref_q, ref_s = oracle.quantize_heads(qkv[:, lo : lo + heads * d].reshape(t, heads, d))
        assert torch.equal(q.view(torch.uint8).cpu(), ref_q) and torch.equal(s.cpu(), ref_s)
    # (H, T, D) storage seen as (T, H, D): unit stride along D, heads far apart
    xt = torch.randn(hkv, t, d, generator=g).bfloat16()
    q, s = quantize_heads(xt.to(DEV).permute(1, 0, 2))
    ref_q, ref_s = oracle.quantize_heads(xt.permute(1, 0, 2))
    assert torch.equal(q.view(torch.uint8).cpu(), ref_q) and torch.equal(s.cpu(), ref_s)
    # D not innermost: copied, same result
    xd = torch.randn(t, d, hkv, generator=g).bfloat16()
    q, s = quantize_heads(xd.to(DEV).permute(0, 2, 1))
    ref_q, ref_s = oracle.quantize_heads(xd.permute(0, 2, 1).contiguous())
    assert torch.equal(q.view(torch.uint8).cpu(), ref_q) and torch.equal(s.cpu(), ref_s)
    assert quantize_heads(dev[:0].view(0, 24, d))[0].shape == (0, 24, d)
    with pytest.raises(ValueError):
        quantize_heads(dev[:, : 4 * 48].view(t, 4, 48))
    with pytest.raises(ValueError):
        quantize_heads(dev[:, : 4 * d].view(t, 4, d), torch.zeros(4, d, device=DEV, dtype=torch.bfloat16))
    with pytest.raises(_lib.MXFP8LibraryError):
        quantize_heads(qkv[:, : 4 * d].view(t, 4, d))
