"""Checks shared by the parity tests.

``assert_codes_equal_up_to_ties``: a quantizer whose input goes through the hardware's
``exp``/``rcp`` (the SwiGLU kernels) cannot match a libm evaluation bit for bit: an fp32
value a few ulp away may fall on the other side of an e4m3 rounding boundary, or push a
block maximum across the threshold of its scale byte.  Those are the ONLY differences the
check lets through: every differing code must be the neighbouring code, with the oracle's
scaled value within ``ulps`` fp32 ulp of the boundary between the two; every differing scale
byte must differ by one, with the block maximum within ``ulps`` ulp of the threshold.
Anything else (a systematic one-code bias, a wrong scale) fails.
"""

import torch

BLOCK = 32


def _fp32_ulp(v: torch.Tensor) -> torch.Tensor:
    a = v.abs().float().clamp_min(torch.finfo(torch.float32).tiny)
    return (torch.nextafter(a, torch.full_like(a, float("inf"))) - a).double()


def assert_codes_equal_up_to_ties(oracle, q, s, values, ulps: int = 4, what: str = "", magnitude=None):
    """``q (R,K)``, ``s (R,K/32)``: device codes and scale bytes of ``values (R,K)`` (fp32, the oracle's
    evaluation of what the kernel quantizes), blocks along the last axis.  Returns the number of differing
    (codes, scale bytes), all of them shown to be rounding ties.

    ``magnitude`` (same shape, default ``|values|``): the size of the terms a value was formed from, where it is
    a difference of larger terms (SwiGLU's derivative crosses zero); the ulp is then taken there.
    """
    q = q.view(torch.uint8).cpu()
    s = s.cpu()
    values = values.float().contiguous()
    magnitude = values.abs() if magnitude is None else torch.maximum(magnitude.float().abs(), values.abs())
    rows, k = values.shape
    ref_q, ref_s = oracle.quantize_rows(values)
    bad_s = s != ref_s
    if bad_s.any():
        # the byte changes where amax / 448 crosses a power of two: amax = 1.75 * 2^j, mantissa field 0x600000
        amax = values.abs().view(rows, k // BLOCK, BLOCK).amax(-1)
        mant = amax.view(torch.int32) & 0x7FFFFF
        assert ((s.int() - ref_s.int()).abs()[bad_s] == 1).all(), f"{what}: a scale byte is off by more than one"
        # ulp of the block's largest value, in units of the ulp of the terms it was formed from
        at = values.abs().view(rows, k // BLOCK, BLOCK).argmax(-1, keepdim=True)
        mag = magnitude.view(rows, k // BLOCK, BLOCK).gather(-1, at).squeeze(-1)
        slack = ulps * (_fp32_ulp(mag) / _fp32_ulp(amax)).round().int()
        assert ((mant - 0x600000).abs()[bad_s] <= slack[bad_s]).all(), f"{what}: a scale byte differs away from its threshold"
    same_block = (~bad_s).repeat_interleave(BLOCK, dim=1)
    bad_q = (q != ref_q) & same_block
    if bad_q.any():
        got, ref = q[bad_q], ref_q[bad_q]
        mag_g, mag_r = (got & 0x7F).int(), (ref & 0x7F).int()
        assert ((mag_g - mag_r).abs() == 1).all(), f"{what}: a differing code is not the neighbouring code"
        sign_differs = ((got ^ ref) & 0x80) != 0
        assert (~sign_differs | (mag_g == 0) | (mag_r == 0)).all(), f"{what}: codes of opposite sign away from zero"
        table = oracle.e4m3_decode_table().double()
        scale = torch.exp2(ref_s.double() - 127.0).repeat_interleave(BLOCK, dim=1)[bad_q]
        boundary = (table[mag_g.long()] + table[mag_r.long()]) / 2 * scale  # between the two magnitudes
        v = values[bad_q]
        gap = (v.abs().double() - boundary).abs()
        unit = _fp32_ulp(magnitude[bad_q])
        assert (gap <= ulps * unit).all(), (
            f"{what}: a differing code whose value is {float((gap / unit).max()):.1f} ulp from the boundary"
        )
    return int(bad_q.sum()), int(bad_s.sum())
