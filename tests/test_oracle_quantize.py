"""Pins the CPU oracle's quantizer before anything is compared against it.

The checks are independent of the oracle's own formulas: torch's CPU float8 cast,
torch/libm evaluations of the literal ``ceil(log2(amax/448))`` expression
(scripts/bench/moe/kernel_ladder.py:184-188 in the reference), known answers, and
invariants the format fixes.
"""

import math

import numpy as np
import pytest
import torch

from conftest import SEED


def _all_bf16():
    bits = torch.arange(0, 1 << 16, dtype=torch.int32).to(torch.int16)
    return bits.view(torch.bfloat16)


def _all_fp16():
    bits = torch.arange(0, 1 << 16, dtype=torch.int32).to(torch.int16)
    return bits.view(torch.float16)


def test_e4m3_decode_table_matches_torch(oracle):
    table = oracle.e4m3_decode_table()
    ref = torch.arange(256, dtype=torch.int32).to(torch.uint8).view(torch.float8_e4m3fn).float()
    finite = ~torch.isnan(ref)
    assert finite.sum() == 254
    assert torch.equal(table[finite], ref[finite])
    assert torch.isnan(table[~finite]).all()
    assert table[0x7E] == 448.0 and table[0x01] == 2.0**-9 and table[0x08] == 2.0**-6


@pytest.mark.parametrize("values", ["bf16", "fp16"])
def test_e4m3_encode_exhaustive_vs_torch(oracle, values):
    x = (_all_bf16() if values == "bf16" else _all_fp16()).float()
    x = x[torch.isfinite(x) & (x.abs() <= 448.0)]
    got = torch.tensor([oracle.lib().ora_e4m3_from_f32(float(v)) for v in x.tolist()], dtype=torch.uint8)
    ref = x.to(torch.float8_e4m3fn).view(torch.uint8)
    assert torch.equal(got, ref)


def test_e4m3_encode_fp32_ties_and_saturation(oracle):
    enc = oracle.lib().ora_e4m3_from_f32
    table = oracle.e4m3_decode_table()
    # every midpoint between neighbouring codes goes to the even code; just off goes to nearest
    for c in range(0, 0x7E):
        lo, hi = float(table[c]), float(table[c + 1])
        mid = (lo + hi) / 2
        even = c if c % 2 == 0 else c + 1
        assert enc(mid) == even, (c, mid)
        assert enc(float(np.nextafter(np.float32(mid), np.float32(0)))) == c
        assert enc(float(np.nextafter(np.float32(mid), np.float32(1e9)))) == c + 1
        assert enc(-mid) == (even | 0x80)
    assert enc(448.0) == 0x7E and enc(1e9) == 0x7E and enc(float("inf")) == 0x7E
    assert enc(-1e9) == 0xFE
    assert enc(float("nan")) & 0x7F == 0x7F
    assert enc(-0.0) == 0x80 and enc(0.0) == 0x00
    assert enc(-1e-40) == 0x80  # underflow keeps the sign, like torch's cast
    rnd = torch.randn(20000, generator=torch.Generator().manual_seed(SEED)) * 50
    rnd = rnd[rnd.abs() <= 448]
    got = torch.tensor([enc(float(v)) for v in rnd.tolist()], dtype=torch.uint8)
    assert torch.equal(got, rnd.to(torch.float8_e4m3fn).view(torch.uint8))


@pytest.mark.parametrize("values", ["bf16", "fp16"])
def test_scale_byte_closed_form_vs_literal(oracle, values):
    x = (_all_bf16() if values == "bf16" else _all_fp16()).float()
    x = x[torch.isfinite(x) & (x >= 0)]
    lib = oracle.lib()
    closed = torch.tensor([lib.ora_scale_byte(float(v)) for v in x.tolist()], dtype=torch.uint8)
    literal = torch.tensor([lib.ora_scale_byte_literal(float(v)) for v in x.tolist()], dtype=torch.uint8)
    assert torch.equal(closed, literal)
    # torch's own log2/ceil on the same values (the reference's pure-torch statement)
    e = torch.ceil(torch.log2(x.clamp_min(1e-30) / 448.0)).clamp_min(-127.0)
    assert torch.equal(closed, (e + 127.0).to(torch.uint8))
    assert closed.min() == 19
    assert closed.max() == (247 if values == "bf16" else 135)


def test_scale_byte_known_answers(oracle):
    sb = oracle.lib().ora_scale_byte
    assert sb(1.0) == 119
    assert sb(448.0) == 127
    assert sb(450.0) == 128
    assert sb(0.0) == 19
    assert sb(1e-35) == 19
    assert sb(3e38) == 247
    for j in range(-100, 100, 7):  # amax exactly 448 * 2^j is a tie: no round-up
        assert sb(448.0 * 2.0**j) == 127 + j
        assert sb(float(np.nextafter(np.float32(448.0 * 2.0**j), np.float32(np.inf)))) == 128 + j
        assert sb(float(torch.tensor(448.0 * 2.0**j).bfloat16()) * (1 + 2**-7)) == 128 + j


def _rand(shape, dtype, scale=1.0, seed=SEED):
    g = torch.Generator().manual_seed(seed)
    return (torch.randn(*shape, generator=g) * scale).to(dtype)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("scale", [1.0, 0.02, 1e-2, 300.0])
def test_quantize_rows_matches_torch_statement(oracle, dtype, scale):
    x = _rand((96, 256), dtype, scale)
    q, s = oracle.quantize_rows(x)
    qt, st = oracle.quantize_rows_torch(x)
    assert torch.equal(s, st)
    assert torch.equal(q, qt)


def test_quantize_rows_edge_blocks(oracle):
    x = _rand((8, 128), torch.bfloat16)
    x[0, :32] = 0.0  # all-zero block -> byte 19, codes 0
    x[1, 32:64] = 1e-35  # below the 1e-30 clamp
    x[2, 64] = 3.0e38
    x[3, :32] = 0.0
    x[3, 5] = -448.0 * 2.0**3  # tie: no round-up, code -448
    x[4, 96:128] = -0.0
    q, s = oracle.quantize_rows(x)
    assert s[0, 0] == 19 and (q[0, :32] == 0).all()
    assert s[1, 1] == 19 and (q[1, 32:64] == 2).all()  # 1e-35 * 2^108 = 3.2e-3 -> 2 * 2^-9
    assert s[2, 2] == 247
    assert s[3, 0] == 130 and q[3, 5] == 0xFE
    assert s[4, 3] == 19 and (q[4, 96:128] == 0x80).all()
    qt, st = oracle.quantize_rows_torch(x)
    assert torch.equal(s, st) and torch.equal(q, qt)
    with pytest.raises(ValueError):
        oracle.quantize_rows(x[:, :48])


def test_quantize_invariants(oracle):
    x = _rand((128, 192), torch.bfloat16, 3.0)
    q, s = oracle.quantize_rows(x)
    # top binade: the block amax lands in (224, 448] * 2^e
    deq = oracle.dequant(q, s)
    blocks = deq.reshape(128, -1, 32).abs().amax(-1)
    top = torch.exp2(s.double() - 127.0) * 448.0
    assert (blocks <= top).all() and (blocks > top / 2 * 0.93).all()
    # the gather commutes with the quantizer
    idx = torch.randperm(128, generator=torch.Generator().manual_seed(1))[:40]
    qg, sg = oracle.quantize_rows(x[idx].contiguous())
    assert torch.equal(qg, q[idx]) and torch.equal(sg, s[idx])
    # zero padding never changes the real codes
    xp = torch.nn.functional.pad(x, (0, 64))
    qp, sp = oracle.quantize_rows(xp)
    assert torch.equal(qp[:, :192], q) and torch.equal(sp[:, :6], s)
    assert (sp[:, 6:] == 19).all() and (qp[:, 192:] == 0).all()
    # strided input: the transposed view quantizes like its contiguous copy
    qs, ss = oracle.quantize_rows(x.t())
    qc, sc = oracle.quantize_rows(x.t().contiguous())
    assert torch.equal(qs, qc) and torch.equal(ss, sc)
    # column axis == row axis of the transpose
    qT, sT = oracle.quantize_cols(x)
    assert torch.equal(qT, qc) and torch.equal(sT, sc)
    # relative error of a randn tensor is the e4m3 figure (~2^-4 worst, ~2.6e-2 rms)
    assert 0.015 < oracle.rel_error(deq, x) < 0.04


def test_swiglu_quantize_matches_composition(oracle):
    g = _rand((64, 128), torch.bfloat16, 2.0, seed=3)
    u = _rand((64, 128), torch.bfloat16, 1.0, seed=4)
    q, s = oracle.swiglu_quantize_rows(g, u)
    act = g.float() * torch.sigmoid(g.float()) * u.float()
    q2, s2 = oracle.quantize_rows(act)
    # expf vs torch.sigmoid may differ by an ulp in fp32, which can flip a rounding
    assert (s != s2).float().mean() < 1e-3
    assert (q != q2).float().mean() < 2e-3
    assert oracle.rel_error(oracle.dequant(q, s), act) < 0.04


def test_swizzle_matches_permute_formula(oracle):
    s = torch.randint(0, 255, (300, 10), dtype=torch.uint8, generator=torch.Generator().manual_seed(5))
    got = oracle.swizzle_32_4_4(s)
    # brute force through the documented view/permute chain (interop.py:24-41)
    rt, ct = 3, 3
    padded = torch.zeros(rt * 128, ct * 4, dtype=torch.uint8)
    padded[:300, :10] = s
    tiles = padded.view(rt, 128, ct, 4).permute(0, 2, 1, 3)
    ref = tiles.reshape(-1, 4, 32, 4).transpose(1, 2).reshape(-1, 32, 16).flatten()
    assert torch.equal(got, ref)


def test_quantize_heads_against_torch_statement_and_invariants(oracle):
    """The attention-operand quantizer: blocks along D with an fp32 mean taken off first.  Pinned by
    the reference's own pure-torch quantizer formula on the shifted operand, by what a zero, an
    equal and an exactly representable shift must give, and by the flat row quantizer when mu is absent."""
    g = torch.Generator().manual_seed(SEED)
    t, h, d = 37, 3, 64
    x = (torch.randn(t, h, d, generator=g) * 2.0).bfloat16()
    mu = torch.randn(h, d, generator=g) * 0.5
    q, s = oracle.quantize_heads(x, mu)
    ref_q, ref_s = oracle.quantize_rows_torch((x.float() - mu[None]).reshape(t, h * d))
    assert torch.equal(q.reshape(t, h * d), ref_q) and torch.equal(s.reshape(t, -1), ref_s)
    q0, s0 = oracle.quantize_heads(x)
    flat_q, flat_s = oracle.quantize_rows(x.reshape(t, h * d))
    assert torch.equal(q0.reshape(t, -1), flat_q) and torch.equal(s0.reshape(t, -1), flat_s)
    qz, sz = oracle.quantize_heads(x, torch.zeros(h, d))
    assert torch.equal(qz, q0) and torch.equal(sz, s0)
    # an operand equal to its mean: every block empty (code 0, byte 19)
    same = mu.bfloat16().float()
    qe, se = oracle.quantize_heads(same[None].expand(t, h, d).bfloat16(), same)
    assert not qe.any() and (se == 19).all()
    # small integers shifted by an integer are exact in bf16: shifting operand and mean alike changes nothing
    xi = torch.randint(-8, 9, (t, h, d), generator=g).float()
    mi = torch.randint(-4, 5, (h, d), generator=g).float()
    a = oracle.quantize_heads(xi.bfloat16(), mi)
    b = oracle.quantize_heads((xi + 16.0).bfloat16(), mi + 16.0)
    assert torch.equal(a[0], b[0]) and torch.equal(a[1], b[1])
