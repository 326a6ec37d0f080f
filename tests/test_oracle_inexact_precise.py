"""The oracle's INEXACT_ROUND RESCALE in precise mode (reference_model/src/ops/type_conversion.cpp:326-346) pinned by
exact rational arithmetic: the scaled value x = v * multiplier * 2^-shift is truncated in plain precise mode; in
compliance mode it is first moved to ceil(x - bound) (normal pass) or floor(x + bound) (bounds pass), with
bound = 0.5 + (3 |x| + |x + output_zp|) * 2^-24.  The operands are chosen so that every double operation of the
reference is exact or far from a rounding boundary, so the exact rationals say what the doubles must give."""
import math
from fractions import Fraction

import numpy as np
import pytest

import oracle


def _exact(v, m, s, out_zp, mode):
    x = Fraction(int(v) * int(m), 1 << int(s))
    if mode == 1:
        return math.trunc(x)
    bound = Fraction(1, 2) + (3 * abs(x) + abs(x + out_zp)) * Fraction(1, 1 << 24)
    return math.ceil(x - bound) if mode == 2 else math.floor(x + bound)


def test_hand_picked_values_either_side_of_an_integer():
    """multiplier 2^30, shift 32: x = v / 4.  FP32 rounding to nearest, FP64 truncation and the two edges of the
    compliance bound all differ on these values, so a swapped branch, a dropped bound or a floor for a ceil shows."""
    v = np.array([7, 6, 8, -6, -7, 5, -5, 2, -2, 0], np.int32).reshape(1, -1)
    kw = dict(out_dtype=np.int32, rounding_mode=oracle.ROUND_INEXACT, per_channel=False)
    m, s = [1 << 30], [32]
    got = {mode: oracle.rescale(v, m, s, inexact_mode=mode, **kw) for mode in (0, 1, 2, 3)}
    assert all(st == oracle.VALID for _, st in got.values())
    #                     x:  1.75  1.5   2.0  -1.5  -1.75  1.25  -1.25  0.5  -0.5  0
    assert got[0][0].ravel().tolist() == [2, 2, 2, -2, -2, 1, -1, 0, 0, 0]      # rint, ties to even
    assert got[1][0].ravel().tolist() == [1, 1, 2, -1, -1, 1, -1, 0, 0, 0]      # truncation of the FP64 value
    assert got[2][0].ravel().tolist() == [2, 1, 2, -2, -2, 1, -1, 0, -1, 0]     # ceil(x - 0.5 - eps)
    assert got[3][0].ravel().tolist() == [2, 2, 2, -1, -2, 1, -1, 1, 0, 0]      # floor(x + 0.5 + eps)
    for mode in (1, 2, 3):
        assert got[mode][0].ravel().tolist() == [_exact(int(x), m[0], s[0], 0, mode) for x in v.ravel()]


@pytest.mark.parametrize("mode", [1, 2, 3])
@pytest.mark.parametrize("out_zp", [0, -100, 77])
def test_random_values_against_exact_rationals(mode, out_zp):
    """int8 -> int8 with an output zero point (it enters the bound): operands small enough for exact doubles; values
    whose moved result lies within 2^-20 of an integer are left out, the rest must agree with the rationals"""
    rng = np.random.default_rng(100 * mode + out_zp)
    v = rng.integers(-128, 128, (64, 16)).astype(np.int8)
    mult = rng.integers(1 << 20, 1 << 30, 16).astype(np.int32)
    shift = rng.integers(24, 31, 16).astype(np.int8)
    got, st = oracle.rescale(v, mult, shift, in_zp=3, out_zp=out_zp, out_dtype=np.int8, rounding_mode=oracle.ROUND_INEXACT,
                             inexact_mode=mode)
    assert st == oracle.VALID
    checked = 0
    for r in range(v.shape[0]):
        for c in range(16):
            x = Fraction((int(v[r, c]) - 3) * int(mult[c]), 1 << int(shift[c]))
            bound = Fraction(1, 2) + (3 * abs(x) + abs(x + out_zp)) * Fraction(1, 1 << 24)
            edge = x if mode == 1 else (x - bound if mode == 2 else x + bound)
            if abs(edge - round(edge)) < Fraction(1, 1 << 20):
                continue
            want = min(127, max(-128, _exact(int(v[r, c]) - 3, mult[c], shift[c], out_zp, mode) + out_zp))
            assert int(got[r, c]) == want, (r, c, float(x))
            checked += 1
    assert checked > 900


def test_the_default_is_fp32_maths_and_the_setting_does_not_leak():
    v = np.array([[7, -7]], np.int32)
    kw = dict(out_dtype=np.int32, rounding_mode=oracle.ROUND_INEXACT, per_channel=False)
    assert oracle.rescale(v, [1 << 30], [32], inexact_mode=1, **kw)[0].ravel().tolist() == [1, -1]
    assert oracle.rescale(v, [1 << 30], [32], **kw)[0].ravel().tolist() == [2, -2]
    # SINGLE / DOUBLE rounding never read the setting
    a = oracle.rescale(v, [1 << 30], [32], out_dtype=np.int32, rounding_mode=oracle.ROUND_SINGLE, per_channel=False)
    b = oracle.rescale(v, [1 << 30], [32], out_dtype=np.int32, rounding_mode=oracle.ROUND_SINGLE, per_channel=False, inexact_mode=3)
    assert np.array_equal(a[0], b[0])
