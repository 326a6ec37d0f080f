"""Pins of the oracle's CONV3D and TRANSPOSE_CONV2D: the literal operands of the reference's own unit tests
(reference_model/test/ref_model_tests/tensor_ops_tests.cpp:268-446 helpers, :622-766 cases) and independent
numpy restatements built from a different formulation than the oracle's loops."""
import numpy as np
import pytest

import oracle

# (inVals, weightVals, inZp, weightZp) of the "zero point avoids overflow" cases
ZP_CASES_2X2 = [
    ([126, -126, -120, 0], [2, 1, 4, -7], 4, 15),
    ([122, -7, -120, 121], [2, 1, 4, -7], -10, -5),
    ([3, -12, 5, 70], [-120, -12, 0, -7], 55, 15),
    ([-5, 65, -1, 32], [-2, 125, 4, -1], -10, -5),
]
ZP_CASES_2X2X2 = [
    ([127, -128, 126, -127, 125, -126, 124, -125], [2, -2, 1, -1, 3, -3, 4, -4], 4, 15),
    ([122, -7, -120, 121, 123, -8, -119, 120], [2, 1, 4, -7, 3, -2, 5, -6], -10, -5),
    ([3, -12, 5, 70, -10, 20, 15, 25], [-120, -12, 0, -7, -50, 10, -30, 5], 55, 15),
    ([-5, 65, -1, 32, 20, -10, -15, 5], [-2, 125, 4, -1, -20, 30, 60, 120], -10, -5),
]


@pytest.mark.parametrize("case", ZP_CASES_2X2)
def test_transpose_conv2d_reference_zero_point_cases(case):
    """tensor_ops_tests.cpp:268-348: 2x2 input, 2x2 kernel, stride 1, no out_pad -> 3x3; the expected value is
    the test's own full-correlation sum (the test indexes the input as inRow*IN_HEIGHT+inCol on a square)."""
    vals, wts, izp, wzp = case
    x = np.array(vals, np.int8).reshape(1, 2, 2, 1)
    w = np.array(wts, np.int8).reshape(1, 2, 2, 1)
    got = oracle.transpose_conv2d("i8", x, w, np.zeros(1, np.int32), in_zp=izp, w_zp=wzp)
    want = np.zeros((3, 3), np.int64)
    for orow in range(3):
        for ocol in range(3):
            for kr in range(2):
                for kc in range(2):
                    ir, ic = orow - kr, ocol - kc
                    if 0 <= ir < 2 and 0 <= ic < 2:
                        want[orow, ocol] += (vals[ir * 2 + ic] - izp) * (wts[kr * 2 + kc] - wzp)
    assert got.shape == (1, 3, 3, 1) and np.array_equal(got[0, :, :, 0], want)


@pytest.mark.parametrize("bias,want", [([-5], [5 * 3 + 9 * -7 - 5, 5 * -1 + 9 * 4 - 5]),
                                       ([-5, 14], [5 * 3 + 9 * -7 - 5, 5 * -1 + 9 * 4 + 14])])
def test_transpose_conv2d_reference_bias_broadcast(bias, want):
    """tensor_ops_tests.cpp:736-766: input {5, 9} over two channels, weights {3,-7,-1,4} as [2,1,1,2]."""
    x = np.array([5, 9], np.int8).reshape(1, 1, 1, 2)
    w = np.array([3, -7, -1, 4], np.int8).reshape(2, 1, 1, 2)
    got = oracle.transpose_conv2d("i8", x, w, np.array(bias, np.int32))
    assert got.reshape(-1).tolist() == want


@pytest.mark.parametrize("case", ZP_CASES_2X2X2)
def test_conv3d_reference_zero_point_cases(case):
    """tensor_ops_tests.cpp:395-446: 2x2x2 volume and kernel -> one output, sum((in-zp)*(w-zp))."""
    vals, wts, izp, wzp = case
    x = np.array(vals, np.int8).reshape(1, 2, 2, 2, 1)
    w = np.array(wts, np.int8).reshape(1, 2, 2, 2, 1)
    got = oracle.conv3d("i8", x, w, np.zeros(1, np.int32), in_zp=izp, w_zp=wzp)
    assert got.reshape(-1).tolist() == [sum((a - izp) * (b - wzp) for a, b in zip(vals, wts))]


def _tconv_numpy(x, w, bias, out_pad, stride, in_zp, w_zp):
    """Scatter formulation: every input pixel adds its (in - zp) x (w - zp) patch into the output at
    (iy*sy + ky + out_pad_top, ix*sx + kx + out_pad_left); the oracle gathers instead."""
    n, ih, iw, ic = x.shape
    oc, kh, kw, _ = w.shape
    oh = (ih - 1) * stride[0] + out_pad[0] + out_pad[1] + kh
    ow = (iw - 1) * stride[1] + out_pad[2] + out_pad[3] + kw
    out = np.zeros((n, oh, ow, oc), np.int64)
    xf, wf = x.astype(np.int64) - in_zp, w.astype(np.int64) - w_zp
    for iy in range(ih):
        for ix in range(iw):
            contrib = np.einsum("nc,ohwc->nhwo", xf[:, iy, ix, :], wf)    # [n, kh, kw, oc]
            for ky in range(kh):
                for kx in range(kw):
                    oy, ox = iy * stride[0] + ky + out_pad[0], ix * stride[1] + kx + out_pad[2]
                    if 0 <= oy < oh and 0 <= ox < ow:
                        out[:, oy, ox, :] += contrib[:, ky, kx, :]
    out += bias.astype(np.int64) if bias.shape[0] == oc else int(bias[0])
    return out.astype(np.int32)


TCONV_SHAPES = [  # n, ih, iw, ic, oc, kh, kw, out_pad, stride
    (1, 4, 5, 3, 2, 3, 3, (0, 0, 0, 0), (1, 1)),
    (2, 3, 4, 5, 7, 2, 3, (1, 0, 2, 1), (2, 3)),
    (1, 5, 5, 4, 4, 3, 3, (-1, -2, -1, 0), (2, 2)),
    (1, 2, 6, 8, 3, 4, 1, (0, 1, 0, 0), (3, 1)),
]


@pytest.mark.parametrize("shape", TCONV_SHAPES)
def test_transpose_conv2d_equals_scatter_formulation(shape):
    n, ih, iw, ic, oc, kh, kw, out_pad, stride = shape
    rng = np.random.default_rng(sum(shape[:7]))
    x = rng.integers(-128, 128, (n, ih, iw, ic)).astype(np.int8)
    w = rng.integers(-128, 128, (oc, kh, kw, ic)).astype(np.int8)
    for bias in (rng.integers(-9999, 9999, oc).astype(np.int32), np.array([77], np.int32)):
        got = oracle.transpose_conv2d("i8", x, w, bias, out_pad, stride, in_zp=-3, w_zp=9)
        assert np.array_equal(got, _tconv_numpy(x, w, bias, out_pad, stride, -3, 9))


def test_transpose_conv2d_shape_rules():
    x, w, b = np.zeros((1, 2, 2, 1), np.int8), np.zeros((1, 3, 3, 1), np.int8), np.zeros(1, np.int32)
    with pytest.raises(oracle.OracleStatus):     # out_pad <= -kernel (tensor_ops.cpp:2037-2041)
        oracle.transpose_conv2d("i8", x, w, b, out_pad=(-3, 0, 0, 0))
    with pytest.raises(oracle.OracleStatus):     # declared output shape mismatch (:2046-2053)
        oracle.transpose_conv2d("i8", x, w, b, out_hw=(5, 4))
    with pytest.raises(oracle.OracleStatus):
        oracle.transpose_conv2d("i8", x, w, b, stride=(0, 1))


def _conv3d_numpy(x, w, bias, pad, stride, dil, in_zp, w_zp):
    """Sum over the depth taps of 2-D convolutions (the 2-D oracle is pinned by its own tests)."""
    n, idp, ih, iw, ic = x.shape
    oc, kd, kh, kw, _ = w.shape
    od, oh, ow = oracle.conv3d_out_dhw((idp, ih, iw), (kd, kh, kw), pad, stride, dil)
    out = np.zeros((n, od, oh, ow, oc), np.int64)
    zero = np.zeros(1, np.int32)
    for o in range(od):
        for k in range(kd):
            d = o * stride[0] + k * dil[0] - pad[0]
            if 0 <= d < idp:
                out[:, o] += oracle.conv2d("i8", x[:, d], w[:, k], zero, pad[2:], stride[1:], dil[1:], in_zp, w_zp)
    out += bias.astype(np.int64) if bias.shape[0] == oc else int(bias[0])
    return out.astype(np.int32)


CONV3D_SHAPES = [  # n, id, ih, iw, ic, oc, kd, kh, kw, pad, stride, dilation
    (1, 4, 5, 5, 3, 4, 2, 3, 3, (0, 0, 1, 1, 1, 1), (1, 1, 1), (1, 1, 1)),
    (2, 5, 6, 4, 2, 3, 3, 2, 2, (1, 1, 0, 0, 1, 1), (2, 2, 1), (1, 1, 2)),
    (1, 3, 3, 3, 16, 5, 3, 1, 1, (2, 2, 0, 0, 0, 0), (1, 1, 1), (2, 1, 1)),
]


@pytest.mark.parametrize("shape", CONV3D_SHAPES)
def test_conv3d_equals_sum_of_2d_convolutions(shape):
    n, idp, ih, iw, ic, oc, kd, kh, kw, pad, stride, dil = shape
    rng = np.random.default_rng(sum(shape[:9]))
    x = rng.integers(-128, 128, (n, idp, ih, iw, ic)).astype(np.int8)
    w = rng.integers(-128, 128, (oc, kd, kh, kw, ic)).astype(np.int8)
    for bias in (rng.integers(-9999, 9999, oc).astype(np.int32), np.array([-5], np.int32)):
        got = oracle.conv3d("i8", x, w, bias, pad, stride, dil, in_zp=6, w_zp=-2)
        assert np.array_equal(got, _conv3d_numpy(x, w, bias, pad, stride, dil, 6, -2))


def test_conv3d_shape_rules():
    x, w, b = np.zeros((1, 4, 4, 4, 1), np.int8), np.zeros((1, 2, 2, 2, 1), np.int8), np.zeros(1, np.int32)
    with pytest.raises(oracle.OracleStatus):     # inexact division (tensor_ops.cpp:207-211)
        oracle.conv3d("i8", x, w, b, stride=(3, 1, 1), out_dhw=(1, 3, 3))
    with pytest.raises(oracle.OracleStatus):     # negative pad
        oracle.conv3d("i8", x, w, b, pad=(-1, 0, 0, 0, 0, 0), out_dhw=(2, 3, 3))


def test_fp_variants_agree_with_fp64_on_exact_inputs():
    """Small integers are exact in every float type: f32, f64 and the int path give the same numbers."""
    rng = np.random.default_rng(5)
    x = rng.integers(-8, 8, (1, 3, 4, 4, 3))
    w = rng.integers(-8, 8, (2, 2, 2, 2, 3))
    b = rng.integers(-8, 8, 2)
    want = oracle.conv3d("i32", x, w, b, (0, 0, 1, 1, 0, 0))
    for kind in ("f32", "f64"):
        assert np.array_equal(oracle.conv3d(kind, x, w, b, (0, 0, 1, 1, 0, 0)), want.astype(np.float64))
    xt, wt = x[:, 0], w[:, 0]
    want = oracle.transpose_conv2d("i32", xt, wt, b, (0, 1, 0, 0), (2, 1))
    for kind in ("f32", "f64"):
        assert np.array_equal(oracle.transpose_conv2d(kind, xt, wt, b, (0, 1, 0, 0), (2, 1)), want.astype(np.float64))
    assert np.array_equal(oracle.transpose_conv2d("f64", -xt, wt, -b, (0, 1, 0, 0), (2, 1), abs_mode=True),
                          oracle.transpose_conv2d("f64", np.abs(xt), np.abs(wt), np.abs(b), (0, 1, 0, 0), (2, 1)))
