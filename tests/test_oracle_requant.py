"""Pins R1 (the ACT rescale-clamp, compiler/torq/Utils/Kernel.h:610-624) of the oracle.

Checks chosen so that a plausible mistake fails one of them: a missing rounding term,
rounding to even / away from zero instead of toward +inf, a logical instead of an
arithmetic shift, a zero point added before the shift, a clamp applied before the
zero point, 32-bit instead of 64-bit products.
"""
import json
import os
from fractions import Fraction

import numpy as np
import pytest

from oracle import oracle as orc

KAT = json.load(open(os.path.join(os.path.dirname(__file__), "golden", "kat.json")))
I32 = (-(1 << 31), (1 << 31) - 1)


def exact(acc, bias, scale, shift, zp, lo, hi):
    t1 = (acc + bias) * scale
    t3 = (Fraction(t1, 1 << shift) + Fraction(1, 2)).__floor__() if shift > 0 else t1
    return max(lo, min(hi, t3 + zp))


def test_identity_scale_is_power_of_two():
    for sh in (1, 7, 12, 30):
        for acc in (-1000, -1, 0, 1, 77, 12345):
            assert orc.act_rescale_clamp(acc, 0, 1 << sh, sh, 9, *I32) == acc + 9


@pytest.mark.parametrize("case", KAT["requant_ties"])
def test_ties_round_toward_plus_infinity(case):
    got = orc.act_rescale_clamp(case["acc"], case["bias"], case["scale"], case["shift"], case["zp"],
                                case["min"], case["max"])
    assert got == case["expected"]


def test_half_cases_explicit():
    # -2.5 -> -2, 2.5 -> 3, -0.5 -> 0, 0.5 -> 1
    assert orc.act_rescale_clamp(-5, 0, 1, 1, 0, *I32) == -2
    assert orc.act_rescale_clamp(5, 0, 1, 1, 0, *I32) == 3
    assert orc.act_rescale_clamp(-1, 0, 1, 1, 0, *I32) == 0
    assert orc.act_rescale_clamp(1, 0, 1, 1, 0, *I32) == 1


def test_brute_force_against_rationals():
    rng = np.random.default_rng(7)
    scales = [1, 3, 21399, (1 << 30), (1 << 31) - 1, 1515257681, -5, -(1 << 30)]
    shifts = [0, 1, 6, 12, 20, 31, 38, 47, 62]
    accs = list(range(-128, 128)) + [int(v) for v in rng.integers(-(1 << 26), 1 << 26, size=300)]
    for scale in scales:
        for sh in shifts:
            for acc in accs:
                bias = int(rng.integers(-(1 << 15), 1 << 15))
                zp = int(rng.integers(-128, 128))
                want = exact(acc, bias, scale, sh, zp, -128, 127)
                assert orc.act_rescale_clamp(acc, bias, scale, sh, zp, -128, 127) == want, (acc, bias, scale, sh, zp)


def test_needs_64_bit_product():
    # (2^26) * (2^31 - 1) overflows 32 and 56 bits; exact value known in closed form.
    acc, scale, sh = 1 << 26, (1 << 31) - 1, 40
    want = (acc * scale + (1 << 39)) >> 40
    assert orc.act_rescale_clamp(acc, 0, scale, sh, 0, *I32) == want
    assert orc.act_rescale_clamp(-acc, 0, scale, sh, 0, *I32) == (-acc * scale + (1 << 39)) >> 40


def test_monotone_and_clamped():
    prev = None
    for acc in range(-5000, 5000, 7):
        q = orc.act_rescale_clamp(acc, 11, 1234567, 24, -3, -128, 127)
        assert -128 <= q <= 127
        if prev is not None:
            assert q >= prev
        prev = q
    # clamp is applied after the zero point
    assert orc.act_rescale_clamp(100, 0, 1, 0, 100, -128, 127) == 127
    assert orc.act_rescale_clamp(-100, 0, 1, 0, -100, -128, 127) == -128
    assert orc.act_rescale_clamp(0, 0, 1, 0, 5, 5, 127) == 5


def test_zero_shift_has_no_rounding_term():
    assert orc.act_rescale_clamp(7, 1, 3, 0, 2, *I32) == (7 + 1) * 3 + 2
