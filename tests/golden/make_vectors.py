"""Writes the golden vectors in this directory from exact rational arithmetic.

Nothing here uses the CPU oracle, the HIP library, libm or a float8 cast: every
expected byte follows from the definitions with Python integers and ``Fraction``.

* UE8M0 scale byte of a block: the smallest integer e with ``amax <= 448 * 2^e``
  (that is ``ceil(log2(amax / 448))``), not below the value the ``1e-30`` clamp
  gives (-108), stored as ``e + 127`` (scripts/bench/moe/kernel_ladder.py:184-188
  in the reference).
* e4m3fn code of ``v / 2^e``: nearest point of the OCP e4m3fn grid, ties to the
  even code, sign kept.
* GEMM: ``sum_k a[m,k] * b[n,k]`` of the decoded operands, exact, rounded once to
  float64.

Run ``python tests/golden/make_vectors.py`` to rewrite the ``.npz`` files; the
tests read only the files.
"""

import os
from fractions import Fraction

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
BLOCK = 32
E4M3_MAX = 448
CLAMP_EXPONENT = -108  # ceil(log2(float32(1e-30) / 448))


def e4m3_grid() -> list[Fraction]:
    """Values of the non-negative e4m3fn codes 0x00..0x7E, in code order."""
    grid = []
    for code in range(0x7F):
        field, mant = code >> 3, code & 7
        if field == 0:
            grid.append(Fraction(mant, 8) * Fraction(1, 64))
        else:
            grid.append((1 + Fraction(mant, 8)) * Fraction(2) ** (field - 7))
    return grid


GRID = e4m3_grid()


def bf16_fraction(bits: int) -> Fraction:
    sign = -1 if bits & 0x8000 else 1
    field, mant = (bits >> 7) & 0xFF, bits & 0x7F
    assert field != 0xFF
    if field == 0:
        return sign * Fraction(mant, 128) * Fraction(2) ** -126
    return sign * (1 + Fraction(mant, 128)) * Fraction(2) ** (field - 127)


def fp16_fraction(bits: int) -> Fraction:
    sign = -1 if bits & 0x8000 else 1
    field, mant = (bits >> 10) & 0x1F, bits & 0x3FF
    assert field != 0x1F
    if field == 0:
        return sign * Fraction(mant, 1024) * Fraction(2) ** -14
    return sign * (1 + Fraction(mant, 1024)) * Fraction(2) ** (field - 15)


def scale_exponent(amax: Fraction) -> int:
    if amax == 0:
        return CLAMP_EXPONENT
    # smallest e with amax <= 448 * 2^e
    ratio = amax / E4M3_MAX
    e = ratio.numerator.bit_length() - ratio.denominator.bit_length()
    while Fraction(2) ** e < ratio:
        e += 1
    while Fraction(2) ** (e - 1) >= ratio:
        e -= 1
    return max(e, CLAMP_EXPONENT)


def e4m3_code(v: Fraction) -> int:
    sign = 0x80 if v < 0 else 0
    a = abs(v)
    if a >= GRID[-1]:
        return sign | 0x7E
    lo, hi = 0, len(GRID) - 1  # GRID[lo] <= a < GRID[hi]
    while hi - lo > 1:
        mid = (lo + hi) // 2
        if GRID[mid] <= a:
            lo = mid
        else:
            hi = mid
    below, above = a - GRID[lo], GRID[hi] - a
    if below < above:
        return sign | lo
    if above < below:
        return sign | hi
    return sign | (lo if lo % 2 == 0 else hi)


def quantize_block(values: list[Fraction], negative_zero: list[bool]) -> tuple[int, list[int]]:
    e = scale_exponent(max(abs(v) for v in values))
    step = Fraction(2) ** e
    codes = [(0x80 if nz else 0) if v == 0 else e4m3_code(v / step) for v, nz in zip(values, negative_zero)]
    return e + 127, codes


def quantize_rows(bits: np.ndarray, to_fraction) -> tuple[np.ndarray, np.ndarray]:
    m, k = bits.shape
    q = np.zeros((m, k), dtype=np.uint8)
    s = np.zeros((m, k // BLOCK), dtype=np.uint8)
    for i in range(m):
        for b in range(k // BLOCK):
            raw = [int(v) for v in bits[i, b * BLOCK : (b + 1) * BLOCK]]
            byte, codes = quantize_block([to_fraction(v) for v in raw], [v == 0x8000 for v in raw])
            s[i, b] = byte
            q[i, b * BLOCK : (b + 1) * BLOCK] = codes
    return q, s


def single_value_table() -> dict[str, np.ndarray]:
    """Each finite bf16 bit pattern alone in a block of zeros: its scale byte and its code."""
    bits, bytes_, codes = [], [], []
    for pattern in range(1 << 16):
        if (pattern >> 7) & 0xFF == 0xFF:
            continue
        v = bf16_fraction(pattern)
        byte, code = quantize_block([v], [pattern == 0x8000])
        bits.append(pattern)
        bytes_.append(byte)
        codes.append(code[0])
    return {
        "bits": np.array(bits, dtype=np.uint16),
        "scale_byte": np.array(bytes_, dtype=np.uint8),
        "code": np.array(codes, dtype=np.uint8),
    }


def seeded_tiles() -> dict[str, np.ndarray]:
    """64 x 128 tiles of normal draws at several magnitudes, quantized along rows and along columns."""
    rng = np.random.RandomState(20090220)
    out = {}
    for name, scale, kind in (("unit", 1.0, "bf16"), ("small", 0.01, "bf16"), ("large", 300.0, "bf16"), ("half", 2.0, "fp16")):
        x = (rng.standard_normal((64, 128)) * scale).astype(np.float32)
        if kind == "bf16":
            as_int = x.view(np.uint32).astype(np.uint64)
            rounded = (as_int + 0x7FFF + ((as_int >> 16) & 1)) >> 16  # round to nearest even
            bits, conv = rounded.astype(np.uint16), bf16_fraction
        else:
            bits, conv = x.astype(np.float16).view(np.uint16), fp16_fraction
        bits[0, :BLOCK] = 0  # an empty block
        bits[1, 40] = 0x8000  # a negative zero
        q, s = quantize_rows(bits, conv)
        qT, sT = quantize_rows(np.ascontiguousarray(bits.T), conv)
        out[f"{name}_{kind}_bits"] = bits
        out[f"{name}_{kind}_q"], out[f"{name}_{kind}_s"] = q, s
        out[f"{name}_{kind}_qT"], out[f"{name}_{kind}_sT"] = qT, sT
    return out


def decode(code: int, byte: int) -> Fraction:
    v = GRID[code & 0x7F] * Fraction(2) ** (byte - 127)
    return -v if code & 0x80 else v


def gemm_case() -> dict[str, np.ndarray]:
    """A 24 x 16 product over K = 96 of random codes and scale bytes, exact."""
    rng = np.random.RandomState(1902)
    m, n, k = 24, 16, 96
    aq = rng.randint(0, 256, (m, k)).astype(np.uint8)
    bq = rng.randint(0, 256, (n, k)).astype(np.uint8)
    aq[(aq & 0x7F) == 0x7F] = 0x38  # no NaN codes
    bq[(bq & 0x7F) == 0x7F] = 0xB8
    as_ = rng.randint(118, 136, (m, k // BLOCK)).astype(np.uint8)
    bs = rng.randint(118, 136, (n, k // BLOCK)).astype(np.uint8)
    a = [[decode(int(aq[i, j]), int(as_[i, j // BLOCK])) for j in range(k)] for i in range(m)]
    b = [[decode(int(bq[i, j]), int(bs[i, j // BLOCK])) for j in range(k)] for i in range(n)]
    c = np.array([[float(sum(x * y for x, y in zip(a[i], b[j]))) for j in range(n)] for i in range(m)], dtype=np.float64)
    return {"aq": aq, "as": as_, "bq": bq, "bs": bs, "c": c}


def main() -> None:
    np.savez_compressed(os.path.join(HERE, "bf16_single_value_blocks.npz"), **single_value_table())
    np.savez_compressed(os.path.join(HERE, "quantized_tiles.npz"), **seeded_tiles())
    np.savez_compressed(os.path.join(HERE, "gemm_nt_exact.npz"), **gemm_case())


if __name__ == "__main__":
    main()
