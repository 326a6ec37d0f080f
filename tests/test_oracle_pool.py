"""Pins for the oracle's AVG_POOL2D / MAX_POOL2D (CPU only): the reference's own unit-test vectors, exact
rational arithmetic for reciprocal_scale, and an independent numpy restatement over padded windows."""
from fractions import Fraction

import numpy as np
import pytest

import oracle

POOL_SHAPES = [  # n, ih, iw, c, kernel, stride, pad
    (1, 2, 2, 1, (2, 2), (2, 2), (0, 0, 0, 0)),
    (2, 8, 8, 4, (2, 2), (2, 2), (0, 0, 0, 0)),
    (1, 7, 9, 5, (3, 3), (2, 2), (1, 1, 1, 1)),
    (2, 10, 6, 16, (3, 2), (1, 2), (2, 1, 0, 0)),
    (1, 5, 5, 3, (5, 5), (1, 1), (0, 0, 0, 0)),        # global pooling
    (1, 12, 12, 8, (4, 4), (4, 4), (3, 1, 2, 2)),      # windows that hold a single image row
    (3, 9, 11, 7, (1, 1), (2, 2), (0, 0, 0, 0)),
]


def windows(x, kernel, stride, pad, fill):
    """[taps, N, OH, OW, C] gathered windows and the same-shaped validity mask, taps in (ky, kx) order"""
    n, ih, iw, c = x.shape
    oh, ow = oracle.pool_out_hw(ih, iw, kernel, stride, pad)
    xp = np.full((n, ih + pad[0] + pad[1], iw + pad[2] + pad[3], c), fill, x.dtype)
    ok = np.zeros(xp.shape, bool)
    xp[:, pad[0]:pad[0] + ih, pad[2]:pad[2] + iw] = x
    ok[:, pad[0]:pad[0] + ih, pad[2]:pad[2] + iw] = True
    taps, valid = [], []
    for ky in range(kernel[0]):
        for kx in range(kernel[1]):
            sl = (slice(None), slice(ky, ky + (oh - 1) * stride[0] + 1, stride[0]),
                  slice(kx, kx + (ow - 1) * stride[1] + 1, stride[1]))
            taps.append(xp[sl])
            valid.append(ok[sl])
    return np.stack(taps), np.stack(valid)


def test_avg_pool_reference_unit_vectors():
    """tensor_ops_tests.cpp:800-823 with the expectation of :552-564 worked out: the zero point is subtracted in
    int32, the sum is scaled by (2^30+1) >> 32 with a single rounding, out_zp added, clipped to int8."""
    x = np.array([126, -126, -128, 0], np.int8).reshape(1, 2, 2, 1)
    assert oracle.avg_pool2d(x, (2, 2), (2, 2), in_zp=4, out_zp=15).ravel().tolist() == [-21]
    x = np.array([126, 126, 127, 127], np.int8).reshape(1, 2, 2, 1)
    assert oracle.avg_pool2d(x, (2, 2), (2, 2), in_zp=-12, out_zp=-5).ravel().tolist() == [127]   # 139 - 5 clipped


def test_reciprocal_scale_exact():
    """quant_util.h:32-43: k = ceil(log2(count)), multiplier = floor(((2^30 + 1) << k) / count), shift = 30 + k,
    and the multiplier is a Q30 value in [2^30, 2^31)"""
    for count in range(1, 4097):
        k = (count - 1).bit_length()
        m, s = oracle.reciprocal_scale(count)
        assert (1 << k) // 2 < count <= (1 << k)
        assert m == int(Fraction(((1 << 30) + 1) << k, count)) and s == 30 + k
        assert (1 << 30) <= m < (1 << 31)


@pytest.mark.parametrize("shape", POOL_SHAPES)
@pytest.mark.parametrize("dtype,zps", [(np.int8, (0, 0)), (np.int8, (-7, 12)), (np.int8, (127, -128)), (np.int16, (0, 0))])
def test_avg_pool_int_against_numpy(shape, dtype, zps):
    n, ih, iw, c, kernel, stride, pad = shape
    rng = np.random.default_rng(ih * 31 + c)
    info = np.iinfo(dtype)
    x = rng.integers(info.min, info.max + 1, (n, ih, iw, c)).astype(dtype)
    taps, valid = windows(x.astype(np.int64), kernel, stride, pad, 0)
    acc = np.where(valid, taps - zps[0], 0).sum(0)
    count = valid.sum(0)
    want = np.empty(acc.shape, np.int64)
    for cnt in np.unique(count):
        k = int(cnt - 1).bit_length()
        m, s = (((1 << 30) + 1) << k) // int(cnt), 30 + k
        sel = count == cnt
        want[sel] = (acc[sel] * m + (1 << (s - 1))) >> s
    want = np.clip(want + zps[1], info.min, info.max).astype(dtype)
    assert np.array_equal(oracle.avg_pool2d(x, kernel, stride, pad, *zps), want)


@pytest.mark.parametrize("shape", POOL_SHAPES)
def test_avg_pool_float_sums_in_tap_order(shape):
    n, ih, iw, c, kernel, stride, pad = shape
    rng = np.random.default_rng(ih + c)
    x = rng.normal(0, 4, (n, ih, iw, c)).astype(np.float16).astype(np.float32)
    taps, valid = windows(x, kernel, stride, pad, 0)
    acc = np.zeros(taps.shape[1:], np.float32)
    for t, v in zip(taps, valid):
        acc = np.where(v, acc + t, acc)          # one fp32 rounding per tap, in (ky, kx) order
    want = acc / valid.sum(0).astype(np.float32)
    got = oracle.avg_pool2d(x, kernel, stride, pad)
    assert got.dtype == np.float32 and np.array_equal(got, want)


@pytest.mark.parametrize("shape", POOL_SHAPES)
@pytest.mark.parametrize("dtype", [np.int8, np.int16])
def test_max_pool_int_against_numpy(shape, dtype):
    n, ih, iw, c, kernel, stride, pad = shape
    rng = np.random.default_rng(iw + c)
    info = np.iinfo(dtype)
    x = rng.integers(info.min, info.max + 1, (n, ih, iw, c)).astype(dtype)
    taps, _ = windows(x, kernel, stride, pad, info.min)
    assert np.array_equal(oracle.max_pool2d(x, kernel, stride, pad), taps.max(0))


@pytest.mark.parametrize("shape", POOL_SHAPES)
def test_max_pool_float_nan_modes(shape):
    n, ih, iw, c, kernel, stride, pad = shape
    rng = np.random.default_rng(3 * iw + c)
    x = rng.normal(0, 4, (n, ih, iw, c)).astype(np.float32)
    x[rng.random(x.shape) < 0.1] = np.nan
    x[rng.random(x.shape) < 0.02] = -np.inf
    taps, valid = windows(x, kernel, stride, pad, 0)
    nan_in_window = (np.isnan(taps) & valid).any(0)
    all_nan = (np.isnan(taps) | ~valid).all(0)
    finite_max = np.where(np.isnan(taps) | ~valid, -np.inf, taps).max(0)
    # PROPAGATE: any NaN in the window gives NaN
    got = oracle.max_pool2d(x, kernel, stride, pad, nan_mode=1)
    assert np.array_equal(np.isnan(got), nan_in_window) and np.array_equal(got[~nan_in_window], finite_max[~nan_in_window])
    # IGNORE: NaNs are skipped; a window of nothing but NaNs gives NaN
    got = oracle.max_pool2d(x, kernel, stride, pad, nan_mode=2)
    assert np.array_equal(np.isnan(got), all_nan) and np.array_equal(got[~all_nan], finite_max[~all_nan])


def test_max_pool_of_lowest_values_and_padding():
    x = np.full((1, 3, 3, 2), -128, np.int8)
    assert np.all(oracle.max_pool2d(x, (3, 3), (1, 1), (2, 2, 2, 2)) == -128)
    xf = np.full((1, 3, 3, 2), -np.inf, np.float32)
    assert np.all(oracle.max_pool2d(xf, (3, 3), (1, 1), (2, 2, 2, 2)) == -np.inf)


@pytest.mark.parametrize("kernel,stride,pad,out_hw", [
    ((2, 2), (2, 2), (2, 0, 0, 0), None),        # pad >= kernel
    ((0, 2), (1, 1), (0, 0, 0, 0), (1, 1)),      # kernel < 1
    ((2, 2), (0, 1), (0, 0, 0, 0), (1, 1)),      # stride < 1
    ((2, 2), (1, 1), (-1, 0, 0, 0), (1, 1)),     # negative pad
    ((3, 3), (2, 2), (0, 0, 0, 0), (3, 3)),      # (8 - 3) % 2 != 0
    ((2, 2), (2, 2), (0, 0, 0, 0), (4, 5)),      # declared output does not match
])
def test_pool_attribute_errors(kernel, stride, pad, out_hw):
    """check_pool2d_attribute, tensor_ops.cpp:52-113"""
    x = np.zeros((1, 8, 8, 2), np.int8)
    for fn in (oracle.avg_pool2d, oracle.max_pool2d):
        with pytest.raises(oracle.OracleStatus):
            fn(x, kernel, stride, pad, out_hw=out_hw)


def test_avg_pool_zero_points_are_for_int8_only():
    """OpAvgPool2d::eval, tensor_ops.cpp:568-571: a zero point other than 0 with int16 or floating-point data is an error"""
    for x in (np.zeros((1, 4, 4, 2), np.int16), np.zeros((1, 4, 4, 2), np.float32)):
        for zps in ((5, 0), (0, -3)):
            with pytest.raises(oracle.OracleStatus):
                oracle.avg_pool2d(x, (2, 2), (2, 2), (0, 0, 0, 0), *zps)
    assert oracle.avg_pool2d(np.full((1, 4, 4, 2), 7, np.int8), (2, 2), (2, 2), (0, 0, 0, 0), 5, -3).tolist() == \
        np.full((1, 2, 2, 2), -1, np.int8).tolist()
