"""GPU parity of TRANSPOSE_CONV2D and CONV3D (evaluated as re-laid-out CONV2D problems) against the CPU oracle,
through the C ABI.  int8 bit for bit; fp16 with the reference's DOT_PRODUCT bound against the fp64 oracle."""
import numpy as np
import pytest

import dot_product_check as dp
import gpu_ops
import oracle
from reference_model_amd import Context, TmiError, capi
from test_oracle_conv3d_tconv import CONV3D_SHAPES, TCONV_SHAPES, ZP_CASES_2X2, ZP_CASES_2X2X2

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module", params=[capi.KERNEL_AUTO, capi.KERNEL_DIRECT], ids=["auto", "direct"])
def ctx(request):
    c = Context(0)
    c.set_kernel_choice(request.param)
    yield c
    c.close()


@pytest.mark.parametrize("case", ZP_CASES_2X2)
def test_transpose_conv2d_reference_zero_point_cases(ctx, case):
    vals, wts, izp, wzp = case
    x = np.array(vals, np.int8).reshape(1, 2, 2, 1)
    w = np.array(wts, np.int8).reshape(1, 2, 2, 1)
    b = np.zeros(1, np.int32)
    got, st = gpu_ops.transpose_conv2d(ctx, x, w, b, in_zp=izp, w_zp=wzp)
    assert st == capi.VALID and np.array_equal(got, oracle.transpose_conv2d("i8", x, w, b, in_zp=izp, w_zp=wzp))


@pytest.mark.parametrize("case", ZP_CASES_2X2X2)
def test_conv3d_reference_zero_point_cases(ctx, case):
    vals, wts, izp, wzp = case
    x = np.array(vals, np.int8).reshape(1, 2, 2, 2, 1)
    w = np.array(wts, np.int8).reshape(1, 2, 2, 2, 1)
    got, st = gpu_ops.conv3d(ctx, x, w, np.zeros(1, np.int32), in_zp=izp, w_zp=wzp)
    assert st == capi.VALID and got.reshape(-1).tolist() == [sum((a - izp) * (c - wzp) for a, c in zip(vals, wts))]


BIG_TCONV = [
    (2, 14, 14, 64, 48, 3, 3, (0, 0, 0, 0), (2, 2)),      # a decoder-style 2x upsampling layer
    (1, 9, 12, 32, 40, 4, 4, (-1, -1, -1, -1), (2, 2)),   # negative out_pad crops the border
    (1, 20, 20, 16, 16, 5, 1, (2, 0, 0, 3), (1, 3)),
]


@pytest.mark.parametrize("shape", TCONV_SHAPES + BIG_TCONV)
@pytest.mark.parametrize("zps", [(-3, 9), (0, 0), (-128, 127)])
def test_transpose_conv2d_i8_bit_exact(ctx, shape, zps):
    n, ih, iw, ic, oc, kh, kw, out_pad, stride = shape
    rng = np.random.default_rng(sum(shape[:7]) + zps[0] + 500)
    x = rng.integers(-128, 128, (n, ih, iw, ic)).astype(np.int8)
    w = rng.integers(-128, 128, (oc, kh, kw, ic)).astype(np.int8)
    for bias in (rng.integers(-9999, 9999, oc).astype(np.int32), np.array([77], np.int32)):
        want = oracle.transpose_conv2d("i8", x, w, bias, out_pad, stride, *zps)
        got, st = gpu_ops.transpose_conv2d(ctx, x, w, bias, out_pad, stride, *zps)
        assert st == capi.VALID and np.array_equal(got, want), int(np.count_nonzero(got != want))


SLAB_TCONV = [  # 3x3 taps, 64 / 96 / 128 input channels, zero weight_zp: both operands are read where they lie
    (2, 14, 14, 64, 48, (0, 0, 0, 0), (2, 2)),        # a decoder-style 2x upsampling layer
    (4, 28, 28, 128, 64, (0, -1, 0, -1), (2, 2)),     # cropped to exactly twice the input
    (3, 9, 11, 96, 80, (1, 0, 0, 2), (1, 1)),         # no holes: the flip alone
    (2, 7, 10, 64, 64, (-1, -2, 0, -1), (2, 3)),      # different strides, cropping on three sides
    (1, 6, 5, 128, 112, (0, 0, -2, 0), (3, 1)),
]


@pytest.fixture(scope="module")
def auto_ctx():
    c = Context(0)
    yield c
    c.close()


@pytest.mark.parametrize("shape", SLAB_TCONV)
@pytest.mark.parametrize("in_zp", [0, -7, 127])
def test_transpose_conv2d_slab_reads_operands_in_place(auto_ctx, shape, in_zp):
    ctx = auto_ctx
    n, ih, iw, ic, oc, out_pad, stride = shape
    rng = np.random.default_rng(ih * iw + ic + oc)
    x = rng.integers(-128, 128, (n, ih, iw, ic)).astype(np.int8)
    w = rng.integers(-128, 128, (oc, 3, 3, ic)).astype(np.int8)
    for bias in (rng.integers(-9999, 9999, oc).astype(np.int32), np.array([-77], np.int32)):
        want = oracle.transpose_conv2d("i8", x, w, bias, out_pad, stride, in_zp, 0)
        got, st = gpu_ops.transpose_conv2d(ctx, x, w, bias, out_pad, stride, in_zp, 0)
        assert ctx.last_kernel == "transpose_conv2d_slab_i8"
        assert st == capi.VALID and np.array_equal(got, want), int(np.count_nonzero(got != want))
    assert len(np.unique(got)) > 50
    # a weight zero point, or any other kernel choice, goes through the re-laid-out operands: same result
    ctx.set_kernel_choice(capi.KERNEL_MFMA)
    try:
        got2, st = gpu_ops.transpose_conv2d(ctx, x, w, bias, out_pad, stride, in_zp, 0)
        assert ctx.last_kernel != "transpose_conv2d_slab_i8" and st == capi.VALID and np.array_equal(got2, want)
    finally:
        ctx.set_kernel_choice(capi.KERNEL_AUTO)


BIG_CONV3D = [
    (1, 8, 12, 12, 16, 32, 3, 3, 3, (1, 1, 1, 1, 1, 1), (1, 1, 1), (1, 1, 1)),
    (2, 6, 9, 9, 32, 24, 2, 3, 3, (0, 0, 1, 1, 1, 1), (2, 2, 2), (1, 1, 1)),
]


@pytest.mark.parametrize("shape", CONV3D_SHAPES + BIG_CONV3D)
@pytest.mark.parametrize("zps", [(6, -2), (0, 0)])
def test_conv3d_i8_bit_exact(ctx, shape, zps):
    n, idp, ih, iw, ic, oc, kd, kh, kw, pad, stride, dil = shape
    rng = np.random.default_rng(sum(shape[:9]) + zps[0])
    x = rng.integers(-128, 128, (n, idp, ih, iw, ic)).astype(np.int8)
    w = rng.integers(-128, 128, (oc, kd, kh, kw, ic)).astype(np.int8)
    for bias in (rng.integers(-9999, 9999, oc).astype(np.int32), np.array([-5], np.int32)):
        want = oracle.conv3d("i8", x, w, bias, pad, stride, dil, *zps)
        got, st = gpu_ops.conv3d(ctx, x, w, bias, pad, stride, dil, *zps)
        assert st == capi.VALID and np.array_equal(got, want), int(np.count_nonzero(got != want))


SLAB_CONV3D = [  # 3x3 taps in the plane, KD x IC = 64 / 96 / 128 bytes per pixel, zero weight_zp: operands read in place
    (2, 8, 14, 14, 32, 64, 3, (1, 1, 1, 1, 1, 1), (1, 1, 1), (1, 1, 1)),    # the bench configuration's geometry, small
    (1, 6, 9, 11, 32, 48, 2, (0, 1, 1, 0, 2, 1), (1, 1, 1), (1, 1, 1)),     # two depth taps, uneven padding
    (2, 9, 10, 10, 32, 80, 4, (2, 1, 1, 1, 1, 1), (2, 1, 1), (1, 1, 1)),    # four depth taps, depth stride 2
    (1, 7, 8, 8, 64, 64, 2, (1, 1, 1, 1, 1, 1), (1, 1, 1), (2, 1, 1)),      # 64 channels, depth dilation 2
    (1, 7, 13, 9, 32, 64, 3, (1, 1, 0, 0, 1, 1), (1, 2, 1), (1, 1, 1)),     # stride 2 along the height
    (3, 5, 6, 6, 32, 112, 3, (3, 3, 1, 1, 1, 1), (1, 1, 1), (1, 1, 1)),     # depth padding larger than the taps reach
]


@pytest.mark.parametrize("shape", SLAB_CONV3D)
@pytest.mark.parametrize("in_zp", [0, 6, -128])
def test_conv3d_slab_reads_operands_in_place(auto_ctx, shape, in_zp):
    ctx = auto_ctx
    n, idp, ih, iw, ic, oc, kd, pad, stride, dil = shape
    rng = np.random.default_rng(idp * ih + iw + ic + oc + kd)
    x = rng.integers(-128, 128, (n, idp, ih, iw, ic)).astype(np.int8)
    w = rng.integers(-128, 128, (oc, kd, 3, 3, ic)).astype(np.int8)
    for bias in (rng.integers(-9999, 9999, oc).astype(np.int32), np.array([-5], np.int32)):
        want = oracle.conv3d("i8", x, w, bias, pad, stride, dil, in_zp, 0)
        got, st = gpu_ops.conv3d(ctx, x, w, bias, pad, stride, dil, in_zp, 0)
        assert ctx.last_kernel == "conv3d_slab_i8"
        assert st == capi.VALID and np.array_equal(got, want), int(np.count_nonzero(got != want))
    assert len(np.unique(got)) > 50
    # any other kernel choice goes through the re-laid-out operands: same result
    ctx.set_kernel_choice(capi.KERNEL_MFMA)
    try:
        got2, st = gpu_ops.conv3d(ctx, x, w, bias, pad, stride, dil, in_zp, 0)
        assert ctx.last_kernel != "conv3d_slab_i8" and st == capi.VALID and np.array_equal(got2, want)
    finally:
        ctx.set_kernel_choice(capi.KERNEL_AUTO)


def test_fp16_variants_within_dot_product_bound(ctx):
    rng = np.random.default_rng(12)
    x = rng.normal(0, 1, (1, 6, 6, 32)).astype(np.float16)
    w = rng.normal(0, 0.1, (16, 3, 3, 32)).astype(np.float16)
    b = rng.normal(0, 0.1, 16).astype(np.float16)
    got, st = gpu_ops.transpose_conv2d(ctx, x, w, b, (0, 1, 0, 1), (2, 2))
    ref = oracle.transpose_conv2d("f64", x, w, b, (0, 1, 0, 1), (2, 2))
    bnd = oracle.transpose_conv2d("f64", x, w, b, (0, 1, 0, 1), (2, 2), abs_mode=True)
    res = dp.check(got.astype(np.float64), ref, bnd, "fp16", dp.kernel_size_bound(9 * 32, "fp16", has_bias=True))
    # tolerance: |imp-ref| <= 2*ksb * max(bnd*2^-11, 2^-14) per element and sum err^2 <= 1.6*ksb*T (DOT_PRODUCT)
    assert st == capi.VALID and res["ok"], res
    x3 = rng.normal(0, 1, (1, 4, 5, 5, 16)).astype(np.float16)
    w3 = rng.normal(0, 0.1, (8, 2, 3, 3, 16)).astype(np.float16)
    b3 = rng.normal(0, 0.1, 8).astype(np.float16)
    got, st = gpu_ops.conv3d(ctx, x3, w3, b3, (0, 0, 1, 1, 1, 1))
    ref = oracle.conv3d("f64", x3, w3, b3, (0, 0, 1, 1, 1, 1))
    bnd = oracle.conv3d("f64", x3, w3, b3, (0, 0, 1, 1, 1, 1), abs_mode=True)
    res = dp.check(got.astype(np.float64), ref, bnd, "fp16", dp.kernel_size_bound(18 * 16, "fp16", has_bias=True))
    assert st == capi.VALID and res["ok"], res


def test_fp32_variants_within_dot_product_bound(ctx):
    """FP32 TRANSPOSE_CONV2D and CONV3D (tensor_ops.cpp:2234, 2288) run as a CONV2D on re-laid-out operands: the order of
    the sum is not the reference's (it scatters TRANSPOSE_CONV2D tap by tap and walks CONV3D's depth taps first), so the
    test is the DOT_PRODUCT bound against the fp64 oracle, and closeness to the oracle's fp32 loop nest"""
    rng = np.random.default_rng(13)
    x = rng.normal(0, 1, (2, 6, 5, 24)).astype(np.float32)
    w = rng.normal(0, 0.1, (10, 3, 2, 24)).astype(np.float32)
    b = rng.normal(0, 0.1, 10).astype(np.float32)
    got, st = gpu_ops.transpose_conv2d(ctx, x, w, b, (0, 1, -1, 1), (2, 3))
    ref = oracle.transpose_conv2d("f64", x, w, b, (0, 1, -1, 1), (2, 3))
    bnd = oracle.transpose_conv2d("f64", x, w, b, (0, 1, -1, 1), (2, 3), abs_mode=True)
    res = dp.check(got.astype(np.float64), ref, bnd, "fp32", dp.kernel_size_bound(6 * 24, "fp32", has_bias=True))
    assert st == capi.VALID and got.dtype == np.float32 and res["ok"], res
    assert np.allclose(got, oracle.transpose_conv2d("f32", x, w, b, (0, 1, -1, 1), (2, 3)), rtol=1e-4, atol=1e-5)
    x3 = rng.normal(0, 1, (1, 4, 5, 5, 12)).astype(np.float32)
    w3 = rng.normal(0, 0.1, (6, 2, 3, 3, 12)).astype(np.float32)
    b3 = rng.normal(0, 0.1, 1).astype(np.float32)
    got, st = gpu_ops.conv3d(ctx, x3, w3, b3, (0, 0, 1, 1, 1, 1))
    ref = oracle.conv3d("f64", x3, w3, b3, (0, 0, 1, 1, 1, 1))
    bnd = oracle.conv3d("f64", x3, w3, b3, (0, 0, 1, 1, 1, 1), abs_mode=True)
    res = dp.check(got.astype(np.float64), ref, bnd, "fp32", dp.kernel_size_bound(18 * 12, "fp32", has_bias=True))
    assert st == capi.VALID and got.dtype == np.float32 and res["ok"], res
    assert np.allclose(got, oracle.conv3d("f32", x3, w3, b3, (0, 0, 1, 1, 1, 1)), rtol=1e-4, atol=1e-5)


def test_shape_rules_are_errors(ctx):
    x, w, b = np.zeros((1, 2, 2, 1), np.int8), np.zeros((1, 3, 3, 1), np.int8), np.zeros(1, np.int32)
    with pytest.raises(TmiError) as e:
        gpu_ops.transpose_conv2d(ctx, x, w, b, out_pad=(-3, 0, 0, 0), out_hw=(1, 4))
    assert e.value.status == capi.ERROR and "out_pad" in e.value.message
    with pytest.raises(TmiError) as e:
        gpu_ops.transpose_conv2d(ctx, x, w, b, out_hw=(5, 4))
    assert "Mismatch between output shape" in e.value.message
    x3, w3 = np.zeros((1, 4, 4, 4, 1), np.int8), np.zeros((1, 2, 2, 2, 1), np.int8)
    with pytest.raises(TmiError) as e:
        gpu_ops.conv3d(ctx, x3, w3, b, stride=(3, 1, 1), out_dhw=(1, 3, 3))
    assert "exact integer output dimensions" in e.value.message
