"""Why the bf16 fast path may multiply by a reciprocal instead of dividing.

The reference computes bf16(x / s) for bf16 x and s (forward.py:471: the division
runs in fp32 and its result is rounded to bf16).  The kernels compute
bf16(fp32(x * r)) with r = rcp(s) accurate to 1 ulp of fp32.  Both round the same
way provided the exact quotient is never closer to a bf16 rounding boundary than
the error of x * r.  These tests establish that gap by brute force over every
pair of bf16 significands, and replay the two computations on them.
"""
from fractions import Fraction

import numpy as np
import torch


def test_quotients_of_bf16_significands_stay_clear_of_rounding_boundaries():
    # significands 1.m with 7 fraction bits = integers 128..255; the quotient
    # a / b lies in (0.5, 2).  bf16 rounding boundaries are the midpoints between
    # neighbouring 8-bit significands in the quotient's binade.
    worst = Fraction(1)
    for a in range(128, 256):
        for b in range(128, 256):
            q = Fraction(a, b)
            # scale q into [128, 256): boundaries are k + 1/2 for integer k
            scaled = q * 128 if q >= 1 else q * 256
            assert 128 <= scaled < 256
            k = scaled.numerator // scaled.denominator
            for boundary in (Fraction(2 * k - 1, 2), Fraction(2 * k + 1, 2)):
                gap = abs(scaled - boundary) / scaled
                assert gap != 0, (a, b)  # never a tie
                worst = min(worst, gap)
    # x * rcp(s) is off by at most 2^-23 (rcp) + 2^-24 (product rounding) relative
    assert worst > Fraction(1, 2 ** 17)
    assert worst > 8 * (Fraction(1, 2 ** 23) + Fraction(1, 2 ** 24))


def _bf16_values(exponents):
    sig = torch.arange(128, 256, dtype=torch.float32) / 128.0
    vals = torch.cat([sig * (2.0 ** e) for e in exponents])
    return torch.cat([vals, -vals]).to(torch.bfloat16)


def test_reciprocal_multiply_rounds_like_the_division_for_any_1ulp_reciprocal():
    x = _bf16_values([-9, -6, -1, 0, 3]).float()
    s = _bf16_values([-8, -7, 0, 5])[: 4 * 128].float()  # positive scales
    want = (x[:, None] / s[None, :]).to(torch.bfloat16)
    r = (1.0 / s).numpy()
    for nudge in (0, 1, -1):  # the correctly rounded reciprocal and both neighbours
        rr = torch.from_numpy((r.view(np.int32) + nudge).view(np.float32))
        got = (x[:, None] * rr[None, :]).to(torch.bfloat16)
        assert torch.equal(got.view(torch.int16), want.view(torch.int16)), nudge
