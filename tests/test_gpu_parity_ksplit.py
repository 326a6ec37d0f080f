"""The int8 CONV2D kernel that splits K over the waves of a workgroup (small layers with taps and a long reduction) through
the C ABI, bit for bit against the CPU oracle (tensor_ops.cpp:828-882, then type_conversion.cpp:224-421): tap counts, strides,
dilations and paddings, every share of K steps per wave, four, eight and sixteen waves, ragged channel tiles, all result types and
both forms of the requantisation."""
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
    (2, 7, 7, 32, 8, 3, 3, (1, 1, 1, 1), (1, 1), (1, 1)),         # 9 K steps on four waves: shares of 3, 3, 3, 0
    (2, 9, 8, 64, 24, 3, 3, (1, 1, 1, 1), (1, 1), (1, 1)),        # 18 steps: 5, 5, 5, 3
    (1, 14, 14, 128, 40, 3, 3, (1, 1, 1, 1), (1, 1), (1, 1)),     # 36 steps: 9 each
    (2, 14, 14, 256, 72, 3, 3, (1, 1, 1, 1), (1, 1), (1, 1)),     # 72 steps on eight waves: 9 each
    (2, 7, 7, 512, 64, 3, 3, (1, 1, 1, 1), (1, 1), (1, 1)),       # 144 steps on sixteen waves: 9 each
    (1, 9, 9, 288, 16, 3, 3, (0, 0, 0, 0), (1, 1), (1, 1)),       # 81 steps on sixteen waves: 6 x 13 + 3, two waves without a share
    (2, 14, 12, 64, 32, 3, 3, (1, 0, 1, 0), (2, 2), (1, 1)),      # stride 2
    (1, 12, 12, 96, 48, 3, 3, (2, 2, 2, 2), (1, 1), (2, 2)),      # dilation 2
    (1, 10, 11, 64, 16, 5, 5, (2, 2, 2, 2), (1, 1), (1, 1)),      # 50 steps on eight waves: 7 x 7 + 1
    (1, 6, 40, 160, 8, 1, 3, (0, 0, 1, 1), (1, 1), (1, 1)),       # 1 x 3 taps, 15 steps
    (3, 5, 5, 32, 104, 2, 2, (0, 1, 0, 1), (1, 1), (1, 1)),       # 4 steps, one each; four channel tiles, the last of 8
]


@pytest.mark.parametrize("shape", SHAPES)
def test_ksplit_int32_results(ctx, shape):
    n, ih, iw, ic, oc, kh, kw, pad, stride, dil = shape
    rng = np.random.default_rng(sum(shape[:7]))
    x = rng.integers(-128, 128, (n, ih, iw, ic)).astype(np.int8)
    w = rng.integers(-128, 128, (oc, kh, kw, ic)).astype(np.int8)
    bias = rng.integers(-(1 << 16), 1 << 16, oc).astype(np.int32)
    for in_zp in (0, -128, 9):
        want = oracle.conv2d("i8", x, w, bias, pad, stride, dil, in_zp=in_zp, w_zp=0)
        got, st = gpu_ops.conv2d(ctx, x, w, bias, pad, stride, dil, in_zp=in_zp, w_zp=0)
        assert ctx.last_kernel == "conv2d_ksplit_i8"
        assert st == capi.VALID and np.array_equal(got, want), int(np.count_nonzero(got != want))


@pytest.mark.parametrize("shape", SHAPES[1:8])
@pytest.mark.parametrize("out_dtype,out_zp", [(np.int8, -4), (np.int16, 0)])
@pytest.mark.parametrize("shifts", ["36 to 44", "mixed with small"])
def test_ksplit_fused_rescale(ctx, shape, out_dtype, out_zp, shifts):
    n, ih, iw, ic, oc, kh, kw, pad, stride, dil = shape
    rng = np.random.default_rng(sum(shape[:7]) + len(shifts))
    x = rng.integers(-128, 128, (n, ih, iw, ic)).astype(np.int8)
    small = shifts != "36 to 44"
    w = (rng.integers(-1, 2, (oc, kh, kw, ic)) if small else rng.integers(-128, 128, (oc, kh, kw, ic))).astype(np.int8)
    bias = rng.integers(-300, 300, oc).astype(np.int32)
    mult = rng.integers(1 << 30, 1 << 31, oc).astype(np.int32)
    shift = (rng.integers(36, 45, oc) if not small else np.where(np.arange(oc) % 3 > 0, rng.integers(33, 40, oc),
                                                                 rng.integers(24, 33, oc))).astype(np.int8)
    acc = oracle.conv2d("i8", x, w, bias, pad, stride, dil, in_zp=-6, w_zp=0)
    for mode in (capi.ROUND_SINGLE, capi.ROUND_DOUBLE):
        want, wst = oracle.rescale(acc, mult, shift, out_zp=out_zp, out_dtype=out_dtype, rounding_mode=mode)
        want = oracle.clamp(want, -90, 110)
        got, st = gpu_ops.conv2d(ctx, x, w, bias, pad, stride, dil, in_zp=-6, w_zp=0, clamp=(-90, 110),
                                 rescale=dict(mult=mult, shift=shift, out_zp=out_zp, out_dtype=out_dtype, rounding_mode=mode))
        assert ctx.last_kernel == "conv2d_ksplit_i8_rescale"
        assert st == wst and np.array_equal(got, want), (st, wst, int(np.count_nonzero(got != want)))
    assert len(np.unique(got)) > 20


@pytest.mark.parametrize("shape", [(8, 14, 14, 256, 256, 1), (8, 7, 7, 512, 512, 1), (8, 28, 28, 256, 256, 2), (8, 14, 14, 512, 512, 2),
                                   (32, 14, 14, 256, 256, 1)])
def test_ksplit_resnet_layers(ctx, shape):
    """the 3x3 layers of ResNet-50's last two stages at batch 8 (and one at batch 32: several pixel tiles per workgroup)"""
    n, hw, _, ic, oc, s = shape
    rng = np.random.default_rng(ic + hw)
    x = rng.integers(-128, 128, (n, hw, hw, ic)).astype(np.int8)
    w = np.clip(np.rint(rng.normal(0, 25, (oc, 3, 3, ic))), -127, 127).astype(np.int8)
    bias = rng.integers(-(1 << 14), 1 << 14, oc).astype(np.int32)
    pad = (1, 1, 1, 1) if s == 1 else (1, 0, 1, 0)
    mult = rng.integers(1 << 30, 1 << 31, oc).astype(np.int32)
    shift = rng.integers(38, 42, oc).astype(np.int8)
    acc = cases.conv2d_exact_blas(x, w, bias, pad, (s, s), (1, 1), 4, 0)
    want, wst = oracle.rescale(acc, mult, shift, out_zp=1)
    got, st = gpu_ops.conv2d(ctx, x, w, bias, pad, (s, s), in_zp=4, w_zp=0, rescale=dict(mult=mult, shift=shift, out_zp=1))
    assert ctx.last_kernel == "conv2d_ksplit_i8_rescale"
    assert st == wst == capi.VALID and np.array_equal(got, want), int(np.count_nonzero(got != want))
    assert len(np.unique(got)) > 100


def test_ksplit_reports_require_conditions_and_declines(ctx):
    rng = np.random.default_rng(2)
    x = rng.integers(-128, 128, (1, 6, 6, 64)).astype(np.int8)
    w = rng.integers(-128, 128, (16, 3, 3, 64)).astype(np.int8)
    bias = np.zeros(16, np.int32)
    mult, shift = np.full(16, 1 << 30, np.int32), np.full(16, 12, np.int8)
    acc = oracle.conv2d("i8", x, w, bias, (1, 1, 1, 1), in_zp=3, w_zp=0)
    want, wst = oracle.rescale(acc, mult, shift)
    got, st = gpu_ops.conv2d(ctx, x, w, bias, (1, 1, 1, 1), in_zp=3, w_zp=0, rescale=dict(mult=mult, shift=shift))
    assert ctx.last_kernel == "conv2d_ksplit_i8_rescale"
    assert st == wst == capi.UNPREDICTABLE and ctx.flags & capi.FLAG_SCALE_VALUE
    for ic, oc, w_zp in ((48, 16, 0), (64, 12, 0), (64, 16, 2), (1024, 16, 0)):
        xx = rng.integers(-128, 128, (1, 6, 6, ic)).astype(np.int8)
        ww = rng.integers(-128, 128, (oc, 3, 3, ic)).astype(np.int8)
        with pytest.raises(TmiError, match="no MFMA / vector kernel is eligible"):
            gpu_ops.conv2d(ctx, xx, ww, np.zeros(oc, np.int32), (1, 1, 1, 1), in_zp=0, w_zp=w_zp)
