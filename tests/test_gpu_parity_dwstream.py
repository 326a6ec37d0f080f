"""GPU parity of the DEPTHWISE_CONV2D kernel that keeps both operands of the matrix instruction in registers (int8,
multiplier 1, 3x3 taps: the pixel operand loaded straight from global memory, no LDS patch, no barrier; a wave keeps
one channel block and walks pixel tiles with the next tile's loads in flight; optional fused RESCALE / CLAMP) against
the CPU oracle, through the C ABI.  Integer work: results are compared bit for bit."""
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
    c.set_kernel_choice(capi.KERNEL_STREAM)
    yield c
    c.close()


DW_SHAPES = [  # n, ih, iw, c, pad, stride, dilation
    (2, 28, 28, 96, (0, 1, 0, 1), (2, 2), (1, 1)),      # the MobileNet layer's geometry, small
    (3, 17, 19, 32, (1, 1, 1, 1), (1, 1), (1, 1)),      # one channel block, ragged tiles
    (2, 12, 13, 48, (1, 1, 1, 1), (1, 1), (1, 1)),      # a ragged second channel block
    (1, 5, 5, 112, (1, 1, 1, 1), (1, 1), (1, 1)),       # seven chunks per pixel, one small tile
    (2, 20, 20, 256, (2, 1, 0, 1), (1, 1), (1, 1)),     # eight channel blocks, uneven padding
    (1, 14, 14, 320, (1, 1, 1, 1), (1, 1), (1, 1)),     # more channels than four waves have lanes
    (2, 24, 24, 64, (2, 2, 2, 2), (1, 1), (2, 2)),      # dilation 2
    (2, 33, 31, 64, (1, 1, 0, 0), (2, 1), (1, 1)),      # stride 2 x 1, no horizontal padding
    (40, 9, 9, 96, (1, 1, 1, 1), (1, 1), (1, 1)),       # many small images
    (2, 14, 14, 576, (1, 1, 1, 1), (1, 1), (1, 1)),     # 18 channel blocks: more channels than eight waves have lanes
    (2, 7, 7, 960, (1, 1, 1, 1), (1, 1), (1, 1)),       # 30 channel blocks
    (1, 10, 10, 1024, (0, 1, 0, 1), (2, 2), (1, 1)),    # the most channels the kernel takes
    (3, 29, 33, 1024, (0, 2, 0, 2), (1, 1), (1, 1)),    # 32 channel blocks on several tiles per wave
    (16, 56, 56, 96, (0, 1, 0, 1), (2, 2), (1, 1)),     # waves that walk more than two tiles
    (1, 70, 3, 32, (1, 1, 1, 1), (1, 1), (1, 1)),       # a narrow image: tiles of 32 rows x 1 column ... 
    (1, 3, 70, 32, (1, 1, 1, 1), (1, 1), (1, 1)),       # ... and of 1 row x 32 columns
]


def _operands(shape, seed):
    n, ih, iw, c, pad, stride, dil = shape
    rng = np.random.default_rng(seed)
    x = rng.integers(-128, 128, (n, ih, iw, c)).astype(np.int8)
    w = rng.integers(-128, 128, (3, 3, c, 1)).astype(np.int8)
    bias = rng.integers(-(1 << 16), 1 << 16, c).astype(np.int32)
    return x, w, bias


@pytest.mark.parametrize("shape", DW_SHAPES)
@pytest.mark.parametrize("in_zp", [0, 4, -128, 127])
def test_depthwise_stream_int32_bit_exact(ctx, shape, in_zp):
    n, ih, iw, c, pad, stride, dil = shape
    x, w, bias = _operands(shape, ih * iw + c)
    got, st = gpu_ops.conv2d(ctx, x, w, bias, pad, stride, dil, in_zp=in_zp, w_zp=0, depthwise=True)
    assert st == capi.VALID and ctx.last_kernel == "depthwise_stream_i8"
    assert np.array_equal(got, oracle.depthwise_conv2d("i8", x, w, bias, pad, stride, dil, in_zp=in_zp, w_zp=0))


@pytest.mark.parametrize("shape", DW_SHAPES)
@pytest.mark.parametrize("zps", [(4, 0), (-7, -3), (127, 100)])
@pytest.mark.parametrize("out_dtype", [np.int8, np.int16])
def test_depthwise_stream_fused_rescale_bit_exact(ctx, shape, zps, out_dtype):
    n, ih, iw, c, pad, stride, dil = shape
    x, w, bias = _operands(shape, ih + iw + c)
    rng = np.random.default_rng(c + ih)
    mult = rng.integers(1 << 30, 1 << 31, c).astype(np.int32)
    shift = rng.integers(34, 40, c).astype(np.int8)
    out_zp = zps[1] if out_dtype == np.int8 else 0
    clamp = (-100, 110) if out_dtype == np.int8 else None
    got, st = gpu_ops.conv2d(ctx, x, w, bias, pad, stride, dil, in_zp=zps[0], w_zp=0, depthwise=True,
                             rescale=dict(mult=mult, shift=shift, out_zp=out_zp, out_dtype=out_dtype), clamp=clamp)
    assert ctx.last_kernel == "depthwise_stream_i8_rescale"
    acc = oracle.depthwise_conv2d("i8", x, w, bias, pad, stride, dil, in_zp=zps[0], w_zp=0)
    want, wst = oracle.rescale(acc, mult, shift, out_zp=out_zp, out_dtype=out_dtype)
    if clamp is not None:
        want = oracle.clamp(want, *clamp)
    assert st == wst == capi.VALID and np.array_equal(got, want), int(np.count_nonzero(got != want))
    assert len(np.unique(got)) > 50


def test_depthwise_stream_config4_full_size(ctx):
    """the named configuration with its own operands: [8,112,112,96], stride 2, per-channel shifts 34..40"""
    c = cases.c4()
    got, st = gpu_ops.conv2d(ctx, c["x"], c["w"], c["bias"], c["pad"], c["stride"], c["dilation"], c["in_zp"], c["w_zp"],
                             depthwise=True, rescale=dict(mult=c["mult"], shift=c["shift"], out_zp=c["out_zp"]))
    assert ctx.last_kernel == "depthwise_stream_i8_rescale" and st == capi.VALID
    acc = oracle.depthwise_conv2d("i8", c["x"], c["w"], c["bias"], c["pad"], c["stride"], c["dilation"],
                                  in_zp=c["in_zp"], w_zp=c["w_zp"])
    want, wst = oracle.rescale(acc, c["mult"], c["shift"], out_zp=c["out_zp"])
    assert wst == oracle.VALID and np.array_equal(got, want)


def test_depthwise_stream_one_shift_for_all_channels_and_single_rounding(ctx):
    shape = (2, 16, 16, 96, (1, 1, 1, 1), (1, 1), (1, 1))
    x, w, bias = _operands(shape, 9)
    rng = np.random.default_rng(2)
    mult = rng.integers(1 << 30, 1 << 31, 96).astype(np.int32)
    for mode in (capi.ROUND_SINGLE, capi.ROUND_DOUBLE):
        for shift in (np.full(96, 36, np.int8), np.array([1518500250 % 5 + 34] * 96, np.int8)):
            got, st = gpu_ops.conv2d(ctx, x, w, bias, shape[4], in_zp=-3, w_zp=0, depthwise=True,
                                     rescale=dict(mult=mult, shift=shift, out_zp=-5, rounding_mode=mode))
            acc = oracle.depthwise_conv2d("i8", x, w, bias, shape[4], in_zp=-3, w_zp=0)
            want, wst = oracle.rescale(acc, mult, shift, out_zp=-5, rounding_mode=mode)
            assert st == wst == capi.VALID and np.array_equal(got, want)
    # bias of length 1 (tensor_ops.cpp:1191-1197)
    got, st = gpu_ops.conv2d(ctx, x, w, np.array([777], np.int32), shape[4], in_zp=5, w_zp=0, depthwise=True)
    assert st == capi.VALID and ctx.last_kernel == "depthwise_stream_i8"
    assert np.array_equal(got, oracle.depthwise_conv2d("i8", x, w, np.array([777], np.int32), shape[4], in_zp=5, w_zp=0))


def test_depthwise_stream_reports_require_conditions(ctx):
    shape = (1, 9, 9, 48, (1, 1, 1, 1), (1, 1), (1, 1))
    x, w, bias = _operands(shape, 5)
    mult, shift = np.full(48, 1 << 30, np.int32), np.full(48, 9, np.int8)
    got, st = gpu_ops.conv2d(ctx, x, w, bias, shape[4], in_zp=3, w_zp=0, depthwise=True,
                             rescale=dict(mult=mult, shift=shift, out_zp=0))
    acc = oracle.depthwise_conv2d("i8", x, w, bias, shape[4], in_zp=3, w_zp=0)
    _, wst = oracle.rescale(acc, mult, shift, out_zp=0)
    assert st == wst == capi.UNPREDICTABLE and ctx.flags & capi.FLAG_SCALE_VALUE
    z = np.zeros_like(x)
    got, st = gpu_ops.conv2d(ctx, z, np.zeros_like(w), np.zeros(48, np.int32), shape[4], in_zp=0, w_zp=0, depthwise=True,
                             rescale=dict(mult=mult, shift=shift, out_zp=0))
    assert st == capi.VALID and ctx.flags == 0 and not got.any()


def test_depthwise_stream_refuses_what_it_cannot_take(ctx):
    rng = np.random.default_rng(1)
    x = rng.integers(-128, 128, (1, 8, 8, 64)).astype(np.int8)
    w = rng.integers(-128, 128, (3, 3, 64, 1)).astype(np.int8)
    bias = np.zeros(64, np.int32)
    with pytest.raises(TmiError):      # a weight zero point
        gpu_ops.conv2d(ctx, x, w, bias, (1, 1, 1, 1), in_zp=0, w_zp=3, depthwise=True)
    with pytest.raises(TmiError):      # channel multiplier 2
        gpu_ops.conv2d(ctx, x, rng.integers(-128, 128, (3, 3, 64, 2)).astype(np.int8), np.zeros(128, np.int32), (1, 1, 1, 1),
                       depthwise=True)
    with pytest.raises(TmiError):      # 24 channels
        gpu_ops.conv2d(ctx, x[..., :24], w[:, :, :24], bias[:24], (1, 1, 1, 1), depthwise=True)
    with pytest.raises(TmiError):      # 5x5 taps
        gpu_ops.conv2d(ctx, x, rng.integers(-128, 128, (5, 5, 64, 1)).astype(np.int8), bias, (2, 2, 2, 2), depthwise=True)


# shifts at the borders between the epilogue's forms (chosen per block of 32 channels): 32 with double rounding takes the
# general form, 33 the high-word form; single rounding takes the high-word form from 32 on; mixtures; shifts too large
# for output_zp * 2^shift to ride in the rounding term; multipliers at their extremes
_FORM_CASES = [
    ("uniform 32", lambda rng, c: np.full(c, 32)), ("uniform 33", lambda rng, c: np.full(c, 33)),
    ("32..34", lambda rng, c: rng.integers(32, 35, c)), ("33..36", lambda rng, c: rng.integers(33, 37, c)),
    ("30..34", lambda rng, c: rng.integers(30, 35, c)), ("52..62", lambda rng, c: rng.integers(52, 63, c)),
    ("64 x 33, then 33..36", lambda rng, c: np.concatenate([np.full(64, 33), rng.integers(33, 37, c - 64)])),
]


@pytest.mark.parametrize("name,shifts", _FORM_CASES, ids=[c[0] for c in _FORM_CASES])
@pytest.mark.parametrize("mode", [capi.ROUND_SINGLE, capi.ROUND_DOUBLE])
@pytest.mark.parametrize("out_dtype,out_zp", [(np.int8, -128), (np.int8, 127), (np.int16, 0)])
def test_depthwise_stream_epilogue_form_borders(ctx, name, shifts, mode, out_dtype, out_zp):
    n, ih, iw, c, pad = 2, 13, 11, 160, (1, 1, 1, 1)
    rng = np.random.default_rng(len(name) + mode)
    shift = shifts(rng, c).astype(np.int8)
    small = int(shift.max()) < 40
    x = rng.integers(-128, 128, (n, ih, iw, c)).astype(np.int8)
    w = rng.integers(-128, 128, (3, 3, c, 1)).astype(np.int8)
    bias = rng.integers(-300, 300, c).astype(np.int32) if small else rng.integers(-(1 << 28), 1 << 28, c).astype(np.int32)
    mult = rng.integers(1 << 30, 1 << 31, c).astype(np.int32)
    mult[:4] = [(1 << 31) - 1, 1 << 30, 0, 1]
    got, st = gpu_ops.conv2d(ctx, x, w, bias, pad, in_zp=-3, w_zp=0, depthwise=True,
                             rescale=dict(mult=mult, shift=shift, out_zp=out_zp, out_dtype=out_dtype, rounding_mode=mode))
    assert ctx.last_kernel == "depthwise_stream_i8_rescale"
    acc = oracle.depthwise_conv2d("i8", x, w, bias, pad, in_zp=-3, w_zp=0)
    want, wst = oracle.rescale(acc, mult, shift, out_zp=out_zp, out_dtype=out_dtype, rounding_mode=mode)
    assert st == wst and np.array_equal(got, want), (st, wst, int(np.count_nonzero(got != want)))
    if small and out_dtype == np.int16:
        assert len(np.unique(got)) > 50


def test_automatic_choice_takes_this_kernel_for_large_layers_with_few_channels():
    c = Context(0)
    try:
        for shape, kernel in [((4, 112, 112, 32, (1, 1, 1, 1), (1, 1), (1, 1)), "depthwise_stream_i8"),
                              ((9, 56, 56, 48, (0, 1, 0, 1), (1, 1), (1, 1)), "depthwise_mfma_i8"),     # 1.3 M results
                              ((2, 112, 112, 64, (1, 1, 1, 1), (1, 1), (1, 1)), "depthwise_mfma_i8")]:  # 64 channels
            x, w, bias = _operands(shape, 21)
            got, st = gpu_ops.conv2d(c, x, w, bias, shape[4], shape[5], in_zp=-9, depthwise=True)
            assert st == capi.VALID and c.last_kernel == kernel
            assert np.array_equal(got, oracle.depthwise_conv2d("i8", x, w, bias, shape[4], shape[5], in_zp=-9, w_zp=0))
    finally:
        c.close()


def _geometry(rng):
    """a legal (ih, iw, pad, stride, dilation) for 3x3 taps: (ih - 1 + pad - 2 * dilation) % stride == 0"""
    while True:
        stride = (int(rng.integers(1, 4)), int(rng.integers(1, 4)))
        dil = (int(rng.integers(1, 4)), int(rng.integers(1, 3)))
        pad = tuple(int(v) for v in rng.integers(0, 4, 4))
        oh, ow = int(rng.integers(1, 70)), int(rng.integers(1, 70))
        ih = (oh - 1) * stride[0] + 2 * dil[0] + 1 - pad[0] - pad[1]
        iw = (ow - 1) * stride[1] + 2 * dil[1] + 1 - pad[2] - pad[3]
        if ih >= 1 and iw >= 1:
            return ih, iw, pad, stride, dil


@pytest.mark.parametrize("seed", range(48))
def test_depthwise_stream_random_geometry(ctx, seed):
    """random strides, dilations, paddings (wider than the taps reach, too), image shapes from a single pixel to many tiles
    per wave, and channel counts that give groups of one, two and three blocks and a ragged last block"""
    rng = np.random.default_rng(7000 + seed)
    ih, iw, pad, stride, dil = _geometry(rng)
    n = int(rng.choice([1, 2, 3, 5, 33]))
    c = int(rng.choice([32, 48, 64, 80, 96, 128, 144, 192, 288]))
    in_zp = int(rng.integers(-128, 128))
    x = rng.integers(-128, 128, (n, ih, iw, c)).astype(np.int8)
    w = rng.integers(-128, 128, (3, 3, c, 1)).astype(np.int8)
    bias = rng.integers(-(1 << 16), 1 << 16, c if seed % 5 else 1).astype(np.int32)
    acc = oracle.depthwise_conv2d("i8", x, w, bias, pad, stride, dil, in_zp=in_zp, w_zp=0)
    got, st = gpu_ops.conv2d(ctx, x, w, bias, pad, stride, dil, in_zp=in_zp, w_zp=0, depthwise=True)
    assert st == capi.VALID and ctx.last_kernel == "depthwise_stream_i8"
    assert np.array_equal(got, acc), (n, ih, iw, c, pad, stride, dil)
    mult = rng.integers(1 << 30, 1 << 31, c).astype(np.int32)
    shift = rng.integers(33, 40, c).astype(np.int8) if seed % 3 else np.full(c, 35, np.int8)
    out_zp = int(rng.integers(-20, 20))
    out_dtype = np.int16 if seed % 4 == 3 else np.int8
    got, st = gpu_ops.conv2d(ctx, x, w, bias, pad, stride, dil, in_zp=in_zp, w_zp=0, depthwise=True,
                             rescale=dict(mult=mult, shift=shift, out_zp=out_zp if out_dtype == np.int8 else 0, out_dtype=out_dtype))
    want, wst = oracle.rescale(acc, mult, shift, out_zp=out_zp if out_dtype == np.int8 else 0, out_dtype=out_dtype)
    assert st == wst == capi.VALID and ctx.last_kernel == "depthwise_stream_i8_rescale"
    assert np.array_equal(got, want), (n, ih, iw, c, pad, stride, dil)
