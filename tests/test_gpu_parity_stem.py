"""The first-layer form of int8 CONV2D (3 x 3 ... 7 x 7 taps over at most 4 channels: a pre-pass that materialises the
padding, then a matrix-core kernel with a K step per row of taps) through the C ABI, bit for bit against the CPU oracle
(tensor_ops.cpp:828-882, then type_conversion.cpp:224-421): channel counts, tap sizes, strides, paddings, vertical dilation,
ragged channel tiles, all result types, and the named networks' first layers."""
import numpy as np
import pytest

import cases
import gpu_ops
import oracle
from reference_model_amd import Context, TmiError, capi

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def ctx():
    c = Context(0)
    c.set_kernel_choice(capi.KERNEL_POINTWISE)
    yield c
    c.close()


SHAPES = [
    # n, ih, iw, ic, oc, kh, kw, pad, stride, dilation
    (2, 17, 19, 3, 8, 3, 3, (1, 1, 1, 1), (1, 1), (1, 1)),
    (1, 16, 18, 3, 32, 3, 3, (0, 1, 0, 1), (2, 2), (1, 1)),
    (2, 23, 21, 3, 64, 7, 7, (3, 3, 3, 3), (2, 2), (1, 1)),
    (1, 21, 24, 1, 24, 5, 5, (2, 2, 2, 2), (1, 1), (1, 1)),
    (3, 9, 9, 4, 40, 7, 7, (3, 3, 3, 3), (1, 1), (1, 1)),
    (1, 15, 15, 2, 16, 5, 3, (2, 2, 1, 1), (1, 1), (1, 1)),
    (1, 20, 12, 3, 16, 3, 3, (2, 2, 1, 1), (1, 1), (2, 1)),      # vertical dilation
    (2, 12, 40, 3, 72, 3, 7, (1, 1, 3, 3), (1, 3), (1, 1)),      # 3 x 7 taps, horizontal stride 3
    (1, 7, 7, 4, 8, 7, 7, (0, 0, 0, 0), (1, 1), (1, 1)),         # one output pixel per image
    (5, 6, 6, 3, 8, 3, 3, (0, 0, 0, 0), (1, 1), (1, 1)),         # no padding
    (2, 9, 30, 1, 16, 3, 11, (1, 1, 5, 5), (1, 1), (1, 1)),      # 11 taps a row: the copy keeps a pixel per byte
    (1, 11, 27, 2, 8, 5, 9, (2, 2, 4, 4), (2, 2), (1, 1)),       # 9 taps of 2 channels: a pixel every 2 bytes
    (1, 12, 29, 4, 24, 3, 8, (1, 1, 3, 4), (1, 1), (1, 1)),      # 8 taps of 4 channels: a row of taps fills the K step
]


@pytest.mark.parametrize("shape", SHAPES)
def test_stem_int32_results(ctx, shape):
    n, ih, iw, ic, oc, kh, kw, pad, stride, dil = shape
    rng = np.random.default_rng(sum(shape[:7]))
    x = rng.integers(-128, 128, (n, ih, iw, ic)).astype(np.int8)
    w = rng.integers(-128, 128, (oc, kh, kw, ic)).astype(np.int8)
    bias = rng.integers(-(1 << 16), 1 << 16, oc).astype(np.int32)
    for in_zp in (0, -128, 11):
        want = oracle.conv2d("i8", x, w, bias, pad, stride, dil, in_zp=in_zp, w_zp=0)
        got, st = gpu_ops.conv2d(ctx, x, w, bias, pad, stride, dil, in_zp=in_zp, w_zp=0)
        assert ctx.last_kernel == "conv2d_stem_i8"
        assert st == capi.VALID and np.array_equal(got, want), int(np.count_nonzero(got != want))


@pytest.mark.parametrize("shape", SHAPES[:8])
@pytest.mark.parametrize("out_dtype,out_zp", [(np.int8, 3), (np.int16, 0)])
def test_stem_fused_rescale(ctx, shape, out_dtype, out_zp):
    n, ih, iw, ic, oc, kh, kw, pad, stride, dil = shape
    rng = np.random.default_rng(sum(shape[:7]) + 5)
    x = rng.integers(-128, 128, (n, ih, iw, ic)).astype(np.int8)
    w = rng.integers(-128, 128, (oc, kh, kw, ic)).astype(np.int8)
    bias = rng.integers(-3000, 3000, oc).astype(np.int32)
    mult = rng.integers(1 << 30, 1 << 31, oc).astype(np.int32)
    acc = oracle.conv2d("i8", x, w, bias, pad, stride, dil, in_zp=-5, w_zp=0)
    for shift in (rng.integers(38, 44, oc).astype(np.int8), np.where(np.arange(oc) % 2 > 0, 40, 30).astype(np.int8)):
        for mode in (capi.ROUND_SINGLE, capi.ROUND_DOUBLE):
            want, wst = oracle.rescale(acc, mult, shift, out_zp=out_zp, out_dtype=out_dtype, rounding_mode=mode)
            got, st = gpu_ops.conv2d(ctx, x, w, bias, pad, stride, dil, in_zp=-5, w_zp=0,
                                     rescale=dict(mult=mult, shift=shift, out_zp=out_zp, out_dtype=out_dtype, rounding_mode=mode))
            assert ctx.last_kernel == "conv2d_stem_i8_rescale"
            assert st == wst and np.array_equal(got, want), (st, wst, int(np.count_nonzero(got != want)))


@pytest.mark.parametrize("shape", [(8, 224, 3, 64, 7, 3, 2), (8, 224, 3, 32, 3, 1, 2), (2, 299, 3, 32, 3, 0, 2)])
def test_stem_first_layers_of_networks(ctx, shape):
    """ResNet-50's 7 x 7 stride 2, MobileNetV2's 3 x 3 stride 2 (padding 0 / 1 at the top and left), Inception's 3 x 3 stride 2
    without padding, at batch 8 and 2; twice in a row, so that the second call finds the scratch buffer in place"""
    n, hw, ic, oc, k, p, s = shape
    rng = np.random.default_rng(hw + k)
    x = rng.integers(-128, 128, (n, hw, hw, ic)).astype(np.int8)
    w = np.clip(np.rint(rng.normal(0, 40, (oc, k, k, ic))), -127, 127).astype(np.int8)
    bias = rng.integers(-(1 << 12), 1 << 12, oc).astype(np.int32)
    pad = (p, p, p, p) if (hw + 2 * p - k) % s == 0 else (p - 1 if p else 0, p, p - 1 if p else 0, p)
    mult = rng.integers(1 << 30, 1 << 31, oc).astype(np.int32)
    shift = rng.integers(38, 41, oc).astype(np.int8)
    acc = cases.conv2d_exact_blas(x, w, bias, pad, (s, s), (1, 1), -128, 0)
    want, wst = oracle.rescale(acc, mult, shift, out_zp=-128)
    for _ in range(2):
        got, st = gpu_ops.conv2d(ctx, x, w, bias, pad, (s, s), in_zp=-128, w_zp=0, rescale=dict(mult=mult, shift=shift, out_zp=-128))
        assert ctx.last_kernel == "conv2d_stem_i8_rescale"
        assert st == wst == capi.VALID and np.array_equal(got, want), int(np.count_nonzero(got != want))
    assert len(np.unique(got)) > 100


def test_stem_declines_what_it_does_not_take(ctx):
    rng = np.random.default_rng(1)
    for ic, oc, k, dil, w_zp in ((5, 8, 3, (1, 1), 0), (3, 12, 3, (1, 1), 0), (3, 8, 3, (1, 2), 0), (3, 8, 3, (1, 1), 1), (4, 8, 9, (1, 1), 0)):
        x = rng.integers(-128, 128, (1, 20, 20, ic)).astype(np.int8)
        w = rng.integers(-128, 128, (oc, k, k, ic)).astype(np.int8)
        with pytest.raises(TmiError, match="no MFMA / vector kernel is eligible"):
            gpu_ops.conv2d(ctx, x, w, np.zeros(oc, np.int32), (0, 0, 0, 0), (1, 1), dil, in_zp=0, w_zp=w_zp)


def test_stem_form_is_skipped_when_the_result_lies_in_the_scratch_buffer():
    """a fused first layer under precise mode is the convolution into the context's scratch buffer plus the stand-alone
    RESCALE (type_conversion.cpp:326-346): the first-layer form, which needs that buffer for its own copies, stands back;
    before and after, the same layer takes it"""
    rng = np.random.default_rng(12)
    x = rng.integers(-128, 128, (4, 64, 60, 3), dtype=np.int8)    # (large enough not to be left to the one-result-per-lane kernel)
    w = rng.integers(-128, 128, (16, 3, 3, 3), dtype=np.int8)
    bias = rng.integers(-2000, 2000, 16).astype(np.int32)
    mult = rng.integers(1 << 30, 1 << 31, 16).astype(np.int32)
    shift = rng.integers(36, 40, 16).astype(np.int8)
    kw = dict(pad=(1, 1, 1, 1), in_zp=-3, w_zp=0)
    acc = oracle.conv2d("i8", x, w, bias, **kw)
    c = Context(0)
    try:
        got, st = gpu_ops.conv2d(c, x, w, bias, **kw)
        assert c.last_kernel == "conv2d_stem_i8" and st == capi.VALID and np.array_equal(got, acc)
        want, wst = oracle.rescale(acc, mult, shift, out_zp=4, rounding_mode=capi.ROUND_INEXACT, inexact_mode=1)
        c.set_precise_mode(1, 0, 0)
        got, st = gpu_ops.conv2d(c, x, w, bias, **kw, rescale=dict(mult=mult, shift=shift, out_zp=4, rounding_mode=capi.ROUND_INEXACT))
        c.set_precise_mode()
        assert c.last_kernel in ("rescale_vec_precise", "rescale_scalar_precise")
        assert st == wst == capi.VALID and np.array_equal(got, want)
        want, wst = oracle.rescale(acc, mult, shift, out_zp=4)
        got, st = gpu_ops.conv2d(c, x, w, bias, **kw, rescale=dict(mult=mult, shift=shift, out_zp=4))
        assert c.last_kernel == "conv2d_stem_i8_rescale" and st == wst == capi.VALID and np.array_equal(got, want)
    finally:
        c.close()
