"""The int8 pointwise kernels (CONV2D 1x1, unit stride, 16 ... 2048 input channels in multiples of 8; from 168 on the form
that splits K over the waves of a workgroup) through the C ABI, bit for bit against the CPU oracle (tensor_ops.cpp:843-882
with one tap, then type_conversion.cpp:224-421): every number of K steps, channel tiles that are ragged by 8 or 16
channels, pixel counts either side of a tile of 32, all three result types, the forms of the requantisation and the
REQUIRE conditions of apply_scale_32."""
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


def _operands(rng, n, h, w, ic, oc, bias_len=None):
    x = rng.integers(-128, 128, (n, h, w, ic)).astype(np.int8)
    wt = rng.integers(-128, 128, (oc, 1, 1, ic)).astype(np.int8)
    bias = rng.integers(-(1 << 16), 1 << 16, bias_len or oc).astype(np.int32)
    return x, wt, bias


@pytest.mark.parametrize("ic", [16, 24, 32, 40, 48, 56, 64, 72, 80, 96, 112, 120, 128, 144, 152, 160])
@pytest.mark.parametrize("oc", [8, 24, 32, 72, 144])
def test_pointwise_int32_results(ctx, ic, oc):
    rng = np.random.default_rng(ic * 1000 + oc)
    x, wt, bias = _operands(rng, 2, 7, 9, ic, oc)
    for in_zp in (0, -11):
        want = oracle.conv2d("i8", x, wt, bias, in_zp=in_zp, w_zp=0)
        got, st = gpu_ops.conv2d(ctx, x, wt, bias, in_zp=in_zp, w_zp=0)
        assert ctx.last_kernel == "conv2d_pointwise_i8"
        assert st == capi.VALID and np.array_equal(got, want), int(np.count_nonzero(got != want))


@pytest.mark.parametrize("pixels", [(1, 1, 1), (1, 1, 31), (1, 3, 11), (3, 5, 13), (2, 56, 56), (8, 112, 112)])
@pytest.mark.parametrize("ic,oc", [(16, 96), (32, 16), (144, 24), (24, 144), (40, 240)])
def test_pointwise_pixel_counts(ctx, pixels, ic, oc):
    """one pixel, a tile less one, a tile and one, many tiles per wave; the largest is a MobileNet layer at batch 8"""
    n, h, w = pixels
    rng = np.random.default_rng(n * h * w + ic)
    x, wt, bias = _operands(rng, n, h, w, ic, oc)
    mult = rng.integers(1 << 30, 1 << 31, oc).astype(np.int32)
    shift = rng.integers(36, 42, oc).astype(np.int8)
    acc = oracle.conv2d("i8", x, wt, bias, in_zp=5, w_zp=0)
    want, wst = oracle.rescale(acc, mult, shift, out_zp=-3)
    got, st = gpu_ops.conv2d(ctx, x, wt, bias, in_zp=5, w_zp=0, rescale=dict(mult=mult, shift=shift, out_zp=-3))
    assert ctx.last_kernel == "conv2d_pointwise_i8_rescale"
    assert st == wst == capi.VALID and np.array_equal(got, want), int(np.count_nonzero(got != want))
    assert pixels[1] < 5 or len(np.unique(got)) > 100


@pytest.mark.parametrize("out_dtype,out_zp", [(np.int8, -128), (np.int8, 127), (np.int16, 0), (np.int8, 5)])
@pytest.mark.parametrize("mode", [capi.ROUND_SINGLE, capi.ROUND_DOUBLE])
@pytest.mark.parametrize("shifts", ["uniform 38", "33 to 40", "32 to 34", "mixed with small", "62"])
def test_pointwise_requantisation_forms(ctx, out_dtype, out_zp, mode, shifts):
    """the high-word form (every shift of a channel tile from 32, or 33 with double rounding, up to what leaves room for the
    zero point) and the general fast form otherwise, per channel tile; both rounding modes; CLAMP merged into the clip"""
    rng = np.random.default_rng(len(shifts) * 7 + mode)
    ic, oc = 48, 72
    x, wt, bias = _operands(rng, 2, 9, 10, ic, oc)
    big = shifts in ("62",)
    if not big and shifts != "uniform 38":
        wt = rng.integers(-3, 4, wt.shape).astype(np.int8)    # small accumulators: shifts of 32 and less leave values in range
        bias = rng.integers(-200, 200, oc).astype(np.int32)
    shift = {"uniform 38": np.full(oc, 38), "33 to 40": rng.integers(33, 41, oc), "32 to 34": rng.integers(32, 35, oc),
             "mixed with small": np.where(np.arange(oc) < 32, rng.integers(33, 40, oc), rng.integers(20, 33, oc)),
             "62": np.full(oc, 62)}[shifts].astype(np.int8)
    mult = rng.integers(1 << 30, 1 << 31, oc).astype(np.int32)
    mult[:3] = [(1 << 31) - 1, 0, 1]
    acc = oracle.conv2d("i8", x, wt, bias, in_zp=-2, w_zp=0)
    want, wst = oracle.rescale(acc, mult, shift, out_zp=out_zp, out_dtype=out_dtype, rounding_mode=mode)
    want = oracle.clamp(want, -100, 1000) if out_dtype == np.int16 else oracle.clamp(want, -100, 90)
    got, st = gpu_ops.conv2d(ctx, x, wt, bias, in_zp=-2, w_zp=0,
                             rescale=dict(mult=mult, shift=shift, out_zp=out_zp, out_dtype=out_dtype, rounding_mode=mode),
                             clamp=(-100, 1000) if out_dtype == np.int16 else (-100, 90))
    assert ctx.last_kernel == "conv2d_pointwise_i8_rescale"
    assert st == wst and np.array_equal(got, want), (st, wst, int(np.count_nonzero(got != want)))


def test_pointwise_reports_require_conditions(ctx):
    """a shift below 32 makes apply_scale_32 check the value range (quant_util.h:59-67): UNPREDICTABLE as the oracle says;
    pixels and channels outside the tensor raise nothing"""
    rng = np.random.default_rng(4)
    x, wt, bias = _operands(rng, 1, 3, 7, 32, 24)
    mult, shift = np.full(24, 1 << 30, np.int32), np.full(24, 12, np.int8)
    acc = oracle.conv2d("i8", x, wt, bias, in_zp=3, w_zp=0)
    want, wst = oracle.rescale(acc, mult, shift)
    got, st = gpu_ops.conv2d(ctx, x, wt, bias, in_zp=3, w_zp=0, rescale=dict(mult=mult, shift=shift))
    assert st == wst == capi.UNPREDICTABLE and ctx.flags & capi.FLAG_SCALE_VALUE
    zero = np.zeros_like(x), np.zeros_like(wt), np.zeros_like(bias)
    got, st = gpu_ops.conv2d(ctx, *zero, in_zp=0, w_zp=0, rescale=dict(mult=mult, shift=shift))
    assert st == capi.VALID and not got.any()


def test_pointwise_broadcast_bias_and_per_tensor_scale(ctx):
    rng = np.random.default_rng(8)
    x, wt, bias = _operands(rng, 2, 6, 6, 64, 40, bias_len=1)
    acc = oracle.conv2d("i8", x, wt, bias, in_zp=-7, w_zp=0)
    mult, shift = np.array([1518500250], np.int32), np.array([40], np.int8)
    want, wst = oracle.rescale(acc, mult, shift, out_zp=4, per_channel=False)
    got, st = gpu_ops.conv2d(ctx, x, wt, bias, in_zp=-7, w_zp=0, rescale=dict(mult=mult, shift=shift, out_zp=4, per_channel=False))
    assert ctx.last_kernel == "conv2d_pointwise_i8_rescale"
    assert st == wst == capi.VALID and np.array_equal(got, want)


def test_pointwise_declines_what_it_does_not_take(ctx):
    rng = np.random.default_rng(9)
    for shape, kw in [((1, 4, 4, 20, 16), {}), ((1, 4, 4, 8, 16), {}), ((1, 4, 4, 2056, 16), {}), ((1, 4, 4, 32, 12), {}), ((1, 4, 4, 32, 16), dict(w_zp=1))]:
        n, h, w, ic, oc = shape
        x, wt, bias = _operands(rng, n, h, w, ic, oc)
        with pytest.raises(TmiError, match="no MFMA / vector kernel is eligible"):
            gpu_ops.conv2d(ctx, x, wt, bias, in_zp=0, w_zp=kw.get("w_zp", 0))
    x, wt, bias = _operands(rng, 1, 5, 5, 32, 16)
    with pytest.raises(TmiError, match="no MFMA / vector kernel is eligible"):
        gpu_ops.conv2d(ctx, x, wt, bias, stride=(2, 2), in_zp=0, w_zp=0)


@pytest.mark.parametrize("ic", [168, 192, 256, 264, 320, 384, 520, 576, 960, 1024, 1032, 1280, 2048])
@pytest.mark.parametrize("oc", [8, 24, 64, 160])
def test_pointwise_split_k_int32_and_fused(ctx, ic, oc):
    """long channel vectors: the four waves of a workgroup take a quarter of K each (2, 4, 8 or 16 K steps a wave, the last
    wave's share ragged or empty) and meet in LDS"""
    rng = np.random.default_rng(ic * 7 + oc)
    x, wt, bias = _operands(rng, 2, 5, 9, ic, oc)
    acc = oracle.conv2d("i8", x, wt, bias, in_zp=-9, w_zp=0)
    got, st = gpu_ops.conv2d(ctx, x, wt, bias, in_zp=-9, w_zp=0)
    assert ctx.last_kernel == "conv2d_pointwise_ksplit_i8"
    assert st == capi.VALID and np.array_equal(got, acc), int(np.count_nonzero(got != acc))
    mult = rng.integers(1 << 30, 1 << 31, oc).astype(np.int32)
    shift = rng.integers(40, 46, oc).astype(np.int8)
    for out_dtype, out_zp in ((np.int8, 7), (np.int16, 0)):
        want, wst = oracle.rescale(acc, mult, shift, out_zp=out_zp, out_dtype=out_dtype)
        got, st = gpu_ops.conv2d(ctx, x, wt, bias, in_zp=-9, w_zp=0, rescale=dict(mult=mult, shift=shift, out_zp=out_zp, out_dtype=out_dtype))
        assert ctx.last_kernel == "conv2d_pointwise_ksplit_i8_rescale"
        assert st == wst == capi.VALID and np.array_equal(got, want), int(np.count_nonzero(got != want))
    assert len(np.unique(got)) > 50


@pytest.mark.parametrize("shape", [(1, 1, 1, 256, 64), (1, 1, 33, 384, 24), (8, 14, 14, 1024, 256), (8, 7, 7, 2048, 512),
                                   (8, 56, 56, 256, 64), (8, 14, 14, 384, 96)])
@pytest.mark.parametrize("shifts", ["33 to 40", "mixed with small"])
def test_pointwise_split_k_layers_and_forms(ctx, shape, shifts):
    """projection layers of ResNet-50 and MobileNetV2 at batch 8 (several pixel tiles per workgroup on the largest), one
    pixel, a tile and one pixel; the high-word and the general form of the requantisation with zero input_zp and without"""
    n, h, w, ic, oc = shape
    rng = np.random.default_rng(n * h + ic + len(shifts))
    x, wt, bias = _operands(rng, n, h, w, ic, oc)
    small = shifts != "33 to 40"
    if small:
        wt = rng.integers(-1, 2, wt.shape).astype(np.int8)
        bias = rng.integers(-200, 200, oc).astype(np.int32)
    shift = (rng.integers(33, 41, oc) if not small else np.where(np.arange(oc) % 40 < 32, rng.integers(33, 40, oc),
                                                                 rng.integers(22, 33, oc))).astype(np.int8)
    mult = rng.integers(1 << 30, 1 << 31, oc).astype(np.int32)
    for in_zp in (0, 6):
        acc = cases.conv2d_exact_blas(x, wt, bias, (0, 0, 0, 0), (1, 1), (1, 1), in_zp, 0)
        want, wst = oracle.rescale(acc, mult, shift, out_zp=-1)
        got, st = gpu_ops.conv2d(ctx, x, wt, bias, in_zp=in_zp, w_zp=0, rescale=dict(mult=mult, shift=shift, out_zp=-1))
        assert ctx.last_kernel == "conv2d_pointwise_ksplit_i8_rescale"
        assert st == wst and np.array_equal(got, want), (st, wst, int(np.count_nonzero(got != want)))
