"""The committed golden vectors against the CPU oracle and, on a GPU, against the HIP library.

``tests/golden/*.npz`` hold expected bytes worked out in exact rational arithmetic by
``tests/golden/make_vectors.py`` from the format's definitions alone (smallest power-of-two
scale with ``amax <= 448 * 2^e``, nearest e4m3fn code with ties to even, exact sums); neither
the oracle nor the library had a hand in them.  They restate what the reference's quantizer
computes (kernels/mxfp8/quantize.py:39-56, scripts/bench/moe/kernel_ladder.py:184-188).
"""

import os

import numpy as np
import pytest
import torch

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")
TILES = ("unit_bf16", "small_bf16", "large_bf16", "half_fp16")
DEV = "cuda:0"


def _load(name):
    return np.load(os.path.join(GOLDEN, name + ".npz"))


def _tensor(bits: np.ndarray, kind: str) -> torch.Tensor:
    dtype = torch.bfloat16 if kind == "bf16" else torch.float16
    return torch.from_numpy(bits.view(np.int16).copy()).view(dtype)


def _single_value_blocks():
    """One row of 32 per finite bf16 value: the value first, zeros behind it."""
    z = _load("bf16_single_value_blocks")
    x = torch.zeros(z["bits"].shape[0], 32, dtype=torch.bfloat16)
    x[:, 0] = _tensor(z["bits"], "bf16")
    return x, torch.from_numpy(z["scale_byte"]), torch.from_numpy(z["code"])


def _same(got: torch.Tensor, want: np.ndarray, what: str):
    got = got.view(torch.uint8).cpu()
    want = torch.from_numpy(want)
    if not torch.equal(got, want):
        bad = (got != want).nonzero()
        raise AssertionError(f"{what}: {bad.shape[0]} mismatches, first at {bad[0].tolist()}")


def test_fixture_known_answers():
    """The vectors themselves against the hand-worked examples of the format."""
    z = _load("bf16_single_value_blocks")
    table = {int(b): (int(s), int(c)) for b, s, c in zip(z["bits"], z["scale_byte"], z["code"])}
    assert table[0x3F80] == (119, 0x78)  # 1.0 -> 2^-8 * 256
    assert table[0x43E0] == (127, 0x7E)  # 448 -> 2^0 * 448
    assert table[0x43E1] == (128, 0x76)  # 450 -> 2^1 * 224 (225 ties to the even code)
    assert table[0x0000] == (19, 0x00) and table[0x8000] == (19, 0x80)
    assert table[0xBF80] == (119, 0xF8)
    assert int(z["scale_byte"].min()) == 19 and int(z["scale_byte"].max()) == 247


def test_oracle_single_value_blocks(oracle):
    x, byte, code = _single_value_blocks()
    q, s = oracle.quantize_rows(x)
    assert torch.equal(s[:, 0], byte)
    assert torch.equal(q[:, 0], code)
    assert not q[:, 1:].any()


@pytest.mark.parametrize("tile", TILES)
def test_oracle_tiles(oracle, tile):
    z = _load("quantized_tiles")
    x = _tensor(z[tile + "_bits"], tile.split("_")[1])
    q, s = oracle.quantize_rows(x)
    _same(q, z[tile + "_q"], "codes")
    _same(s, z[tile + "_s"], "scales")
    qt, st = oracle.quantize_cols(x)
    _same(qt, z[tile + "_qT"], "column-axis codes")
    _same(st, z[tile + "_sT"], "column-axis scales")
    qs, ss = oracle.quantize_rows_torch(x)
    _same(qs, z[tile + "_q"], "codes of the torch statement")
    _same(ss, z[tile + "_s"], "scales of the torch statement")


def test_oracle_gemm_exact(oracle):
    z = _load("gemm_nt_exact")
    ops = [torch.from_numpy(z[k]) for k in ("aq", "as", "bq", "bs")]
    want = torch.from_numpy(z["c"])
    # fp64 sums of 96 products that carry at most 8 significant bits each: a few ulp at most
    assert oracle.rel_error(oracle.gemm_nt(*ops), want) < 1e-14
    assert oracle.rel_error(oracle.gemm_nt_scalar(*ops), want) < 1e-14


@pytest.mark.gpu
def test_hip_single_value_blocks():
    from kohakuwullm_amd.kernels import mxfp8

    x, byte, code = _single_value_blocks()
    q, s = mxfp8.quantize_mx(x.to(DEV))
    q, s = q.view(torch.uint8).cpu(), s.cpu()
    assert torch.equal(s[:, 0], byte)
    assert torch.equal(q[:, 0], code)
    assert not q[:, 1:].any()


@pytest.mark.gpu
@pytest.mark.parametrize("tile", TILES)
def test_hip_tiles(tile):
    from kohakuwullm_amd.kernels import mxfp8

    z = _load("quantized_tiles")
    x = _tensor(z[tile + "_bits"], tile.split("_")[1]).to(DEV)
    q, s = mxfp8.quantize_mx(x)
    _same(q, z[tile + "_q"], "codes")
    _same(s, z[tile + "_s"], "scales")
    qt, st = mxfp8.quantize_mx_cols(x)
    _same(qt, z[tile + "_qT"], "column-axis codes")
    _same(st, z[tile + "_sT"], "column-axis scales")
    q2, s2, qt2, st2 = mxfp8.quantize_mx_dual(x)
    _same(q2, z[tile + "_q"], "dual codes")
    _same(s2, z[tile + "_s"], "dual scales")
    _same(qt2, z[tile + "_qT"], "dual column-axis codes")
    _same(st2, z[tile + "_sT"], "dual column-axis scales")


@pytest.mark.gpu
def test_hip_gemm_exact():
    """fp32 output within 1e-4, bf16 within 1e-2 (relative Frobenius) of the exact product."""
    from kohakuwullm_amd.kernels import mxfp8

    z = _load("gemm_nt_exact")
    aq, a_s, bq, b_s = (torch.from_numpy(z[k]).to(DEV) for k in ("aq", "as", "bq", "bs"))
    aq, bq = aq.view(torch.float8_e4m3fn), bq.view(torch.float8_e4m3fn)
    want = torch.from_numpy(z["c"])
    for dtype, bar in ((torch.float32, 1e-4), (torch.bfloat16, 1e-2)):
        got = mxfp8.mxfp8_matmul_pq(aq, a_s, bq, b_s, out_dtype=dtype).double().cpu()
        err = float((got - want).norm() / want.norm())
        assert err < bar, (dtype, err)
