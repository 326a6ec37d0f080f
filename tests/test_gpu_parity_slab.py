"""GPU parity of the slab kernel (int8 3x3 CONV2D with 64 input channels: weight slab and input patch loaded
straight into LDS, optional fused RESCALE / CLAMP) against exact float64 BLAS products and the CPU oracle, through
the C ABI.  Everything here is integer work: results are compared bit for bit."""
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
    c.set_kernel_choice(capi.KERNEL_SLAB)
    yield c
    c.close()


SLAB_SHAPES = [  # n, ih, iw, oc, pad, stride, dilation[, ic: 64 unless given]
    (8, 56, 56, 64, (1, 1, 1, 1), (1, 1), (1, 1)),      # the headline layer
    (3, 30, 29, 64, (1, 1, 1, 1), (1, 1), (1, 1)),      # ragged tiles in both directions
    (1, 5, 5, 64, (1, 1, 1, 1), (1, 1), (1, 1)),        # one small tile
    (2, 17, 23, 48, (0, 0, 0, 0), (1, 1), (1, 1)),      # no padding, 48 channels (the second channel tile half empty)
    (2, 20, 20, 128, (1, 1, 1, 1), (1, 1), (1, 1)),     # two channel blocks
    (2, 20, 20, 80, (2, 1, 0, 1), (1, 1), (1, 1)),      # a ragged second block, uneven padding
    (4, 57, 57, 64, (1, 1, 1, 1), (2, 2), (1, 1)),      # stride 2
    (2, 34, 31, 64, (0, 1, 1, 0), (2, 1), (1, 1)),      # stride 2 x 1
    (2, 24, 24, 64, (2, 2, 2, 2), (1, 1), (2, 2)),      # dilation 2
    (33, 14, 14, 64, (1, 1, 1, 1), (1, 1), (1, 1)),     # more workgroups than compute units, odd count
    (4, 28, 28, 128, (1, 1, 1, 1), (1, 1), (1, 1), 128),    # 128 input channels: four MFMA steps per tap
    (2, 19, 17, 80, (1, 0, 2, 1), (1, 1), (1, 1), 128),     # ragged tiles and channel block
    (2, 29, 29, 64, (1, 1, 1, 1), (2, 2), (1, 1), 128),     # stride 2
    (3, 21, 22, 64, (1, 1, 1, 1), (1, 1), (1, 1), 96),      # 96 input channels: three MFMA steps per tap
    # unit stride and more 124-pixel tiles than the chip has CUs: two accumulator tiles per wave on tiles of up to 252 pixels
    (20, 37, 41, 64, (1, 1, 1, 1), (1, 1), (1, 1)),         # ragged tiles
    (12, 50, 50, 80, (1, 0, 1, 2), (1, 1), (1, 1), 128),    # 128 input channels, a ragged second channel block
    (70, 14, 14, 128, (1, 1, 1, 1), (1, 1), (1, 1)),        # one tile per image: the last wave's second tile is empty
    (24, 40, 40, 64, (2, 2, 2, 2), (1, 1), (2, 2)),         # dilation 2
    (28, 36, 36, 64, (1, 1, 1, 1), (1, 1), (1, 1), 96),     # 96 input channels
]


def fused_kernel(ic, stride):
    """the fused form of a 3x3 layer with 64 input channels and unit stride keeps the weights in registers"""
    return "conv2d_slab_wreg_i8_rescale" if ic == 64 and tuple(stride) == (1, 1) else "conv2d_slab_i8_rescale"


def _operands(shape, seed):
    n, ih, iw, oc, pad, stride, dil = shape[:7]
    ic = shape[7] if len(shape) > 7 else 64
    rng = np.random.default_rng(seed)
    x = rng.integers(-128, 128, (n, ih, iw, ic)).astype(np.int8)
    w = rng.integers(-128, 128, (oc, 3, 3, ic)).astype(np.int8)
    bias = rng.integers(-(1 << 18), 1 << 18, oc).astype(np.int32)
    return x, w, bias


@pytest.mark.parametrize("shape", SLAB_SHAPES)
@pytest.mark.parametrize("in_zp", [0, -7, 127, -128])
def test_slab_conv_int32_bit_exact(ctx, shape, in_zp):
    n, ih, iw, oc, pad, stride, dil = shape[:7]
    x, w, bias = _operands(shape, ih * iw + oc)
    got, st = gpu_ops.conv2d(ctx, x, w, bias, pad, stride, dil, in_zp=in_zp, w_zp=0)
    assert st == capi.VALID and ctx.last_kernel == "conv2d_slab_i8"
    assert np.array_equal(got, cases.conv2d_exact_blas(x, w, bias, pad, stride, dil, in_zp, 0))
    # the last image's first channels against the oracle's own loop nest
    sub = oracle.conv2d("i8", x[-1:], w[:5], bias[:5], pad, stride, dil, in_zp=in_zp, w_zp=0)
    assert np.array_equal(got[-1:, :, :, :5], sub)


def test_slab_conv_bias_broadcast_and_extremes(ctx):
    """a bias of length 1 goes to every channel (tensor_ops.cpp:747, :816-823); all-extreme operands reach the
    largest accumulators the type allows: 576 * 128 * 255 < 2^31"""
    x = np.full((2, 9, 9, 64), -128, np.int8)
    w = np.full((64, 3, 3, 64), -128, np.int8)
    w[1::2] = 127
    bias = np.array([-12345], np.int32)
    got, st = gpu_ops.conv2d(ctx, x, w, bias, (1, 1, 1, 1), in_zp=127, w_zp=0)
    assert st == capi.VALID and ctx.last_kernel == "conv2d_slab_i8"
    assert np.array_equal(got, cases.conv2d_exact_blas(x, w, bias, (1, 1, 1, 1), (1, 1), (1, 1), 127, 0))
    assert got.max() == 576 * 255 * 128 - 12345 and got.min() == -576 * 255 * 127 - 12345


def _fused(ctx, c, out_dtype):
    got, st = gpu_ops.conv2d(ctx, c["x"], c["w"], c["bias"], c["pad"], c["stride"], c["dilation"], c["in_zp"], 0,
                             rescale=dict(mult=c["mult"], shift=c["shift"], out_zp=c["out_zp"], out_dtype=out_dtype,
                                          rounding_mode=c.get("mode", capi.ROUND_DOUBLE),
                                          per_channel=c.get("per_channel", True)),
                             clamp=c["clamp"])
    acc = cases.conv2d_exact_blas(c["x"], c["w"], c["bias"], c["pad"], c["stride"], c["dilation"], c["in_zp"], 0)
    want, wst = oracle.rescale(acc, c["mult"], c["shift"], out_zp=c["out_zp"], out_dtype=out_dtype,
                               rounding_mode=c.get("mode", oracle.ROUND_DOUBLE), per_channel=c.get("per_channel", True))
    if c["clamp"] is not None:
        want = oracle.clamp(want, *c["clamp"])
    return got, st, want, wst


@pytest.mark.parametrize("shape", SLAB_SHAPES)
@pytest.mark.parametrize("zps", [(-7, 0), (4, -3), (-128, 100)])
@pytest.mark.parametrize("out_dtype", [np.int8, np.int16])
def test_slab_conv_fused_rescale_bit_exact(ctx, shape, zps, out_dtype):
    n, ih, iw, oc, pad, stride, dil = shape[:7]
    x, _, _ = _operands(shape, ih + iw + oc)
    rng = np.random.default_rng(oc + ih)
    c = dict(x=x, w=np.clip(np.rint(rng.normal(0, 30, (oc, 3, 3, x.shape[3]))), -127, 127).astype(np.int8),
             bias=np.rint(rng.normal(0, 1 << 14, oc)).astype(np.int32), in_zp=zps[0], pad=pad, stride=stride,
             dilation=dil, mult=rng.integers(1 << 30, 1 << 31, oc).astype(np.int32),
             shift=rng.integers(36, 42, oc).astype(np.int8), out_zp=zps[1] if out_dtype == np.int8 else 0,
             clamp=(-100, 110) if out_dtype == np.int8 else None)
    got, st, want, wst = _fused(ctx, c, out_dtype)
    assert ctx.last_kernel == fused_kernel(x.shape[3], stride)
    assert st == wst == capi.VALID and np.array_equal(got, want), int(np.count_nonzero(got != want))
    assert len(np.unique(got)) > 50


@pytest.mark.parametrize("shape", [  # n, ih, iw, ic, oc, pad, stride
    (8, 56, 56, 64, 256, (0, 0, 0, 0), (1, 1)),         # a bottleneck block's expanding 1x1 layer
    (4, 28, 28, 128, 512, (0, 0, 0, 0), (1, 1)),
    (4, 29, 29, 128, 64, (0, 0, 0, 0), (2, 2)),         # a down-sampling shortcut
    (4, 28, 28, 96, 64, (0, 0, 0, 0), (1, 1)),          # a MobileNet projection layer
    (3, 17, 13, 64, 80, (1, 0, 0, 2), (1, 1)),          # padding on a pointwise layer: the border is bias only
    (9, 61, 47, 64, 192, (0, 0, 0, 0), (1, 1)),         # two accumulator tiles per wave, ragged tiles
    (5, 33, 35, 128, 320, (1, 0, 0, 2), (1, 1)),        # the same with padding and five channel blocks
    (2, 28, 28, 256, 64, (0, 0, 0, 0), (1, 1)),         # 256 input channels: 8 K steps, 17 chunks per patch pixel
    (3, 14, 14, 256, 208, (0, 0, 0, 0), (1, 1)),        # ... four channel blocks, the last of 16
    (2, 28, 28, 512, 128, (0, 0, 0, 0), (1, 1)),        # 512 input channels: 16 K steps
    (2, 15, 13, 512, 80, (0, 0, 1, 1), (2, 2)),         # ... with a stride and padding
    (9, 40, 40, 256, 64, (0, 0, 0, 0), (1, 1)),         # 256 channels, two accumulator tiles per wave
    (2, 14, 14, 160, 64, (0, 0, 0, 0), (1, 1)),         # every other channel count the kernel is built for: 5 K steps
    (10, 38, 38, 192, 48, (0, 0, 0, 0), (1, 1)),        # ... 6, two accumulator tiles per wave
    (2, 14, 14, 320, 96, (0, 0, 0, 0), (1, 1)),         # ... 10
    (2, 15, 14, 384, 64, (1, 1, 0, 0), (1, 1)),         # ... 12
    (2, 14, 14, 480, 112, (0, 0, 0, 0), (1, 1)),        # ... 15
    (2, 14, 14, 576, 96, (0, 0, 0, 0), (1, 1)),         # ... 18
    (2, 9, 14, 768, 64, (0, 0, 0, 0), (1, 1)),          # ... 24
    (2, 7, 7, 960, 160, (0, 0, 0, 0), (1, 1)),          # ... 30
    (3, 14, 14, 1024, 144, (0, 0, 0, 0), (1, 1)),       # ... 32 K steps of a weight row of 1 KB, tiles of 62 pixels
])
@pytest.mark.parametrize("in_zp", [0, -7])
def test_slab_pointwise_layers_bit_exact(ctx, shape, in_zp):
    """1x1 taps with 64 ... 512 input channels: little K for the GEMM kernel, 2 ... 16 MFMA steps here"""
    n, ih, iw, ic, oc, pad, stride = shape
    rng = np.random.default_rng(ih * oc + ic)
    x = rng.integers(-128, 128, (n, ih, iw, ic)).astype(np.int8)
    w = rng.integers(-128, 128, (oc, 1, 1, ic)).astype(np.int8)
    bias = rng.integers(-(1 << 18), 1 << 18, oc).astype(np.int32)
    got, st = gpu_ops.conv2d(ctx, x, w, bias, pad, stride, in_zp=in_zp, w_zp=0)
    assert st == capi.VALID and ctx.last_kernel == "conv2d_slab_i8"
    acc = cases.conv2d_exact_blas(x, w, bias, pad, stride, (1, 1), in_zp, 0)
    assert np.array_equal(got, acc)
    assert np.array_equal(got[:1, :, :, :3], oracle.conv2d("i8", x[:1], w[:3], bias[:3], pad, stride, in_zp=in_zp, w_zp=0))
    mult = rng.integers(1 << 30, 1 << 31, oc).astype(np.int32)
    shift = rng.integers(35, 41, oc).astype(np.int8)
    got, st = gpu_ops.conv2d(ctx, x, w, bias, pad, stride, in_zp=in_zp, w_zp=0,
                             rescale=dict(mult=mult, shift=shift, out_zp=3), clamp=(-128, 100))
    want, wst = oracle.rescale(acc, mult, shift, out_zp=3)
    assert st == wst == capi.VALID and ctx.last_kernel == "conv2d_slab_i8_rescale"
    assert np.array_equal(got, oracle.clamp(want, -128, 100))


def test_slab_config3_full_size(ctx):
    """the named configuration with its own operands: shift 38 for every channel, DOUBLE rounding, CLAMP [0, 127]"""
    c = cases.c3()
    got, st = gpu_ops.conv2d(ctx, c["x"], c["w"], c["bias"], c["pad"], c["stride"], c["dilation"], c["in_zp"], c["w_zp"],
                             rescale=dict(mult=c["mult"], shift=c["shift"], out_zp=c["out_zp"]), clamp=c["clamp"])
    assert ctx.last_kernel == "conv2d_slab_wreg_i8_rescale" and st == capi.VALID
    acc = cases.conv2d_exact_blas(c["x"], c["w"], c["bias"], c["pad"], c["stride"], c["dilation"], c["in_zp"], c["w_zp"])
    want, wst = oracle.rescale(acc, c["mult"], c["shift"], out_zp=c["out_zp"])
    assert wst == oracle.VALID and np.array_equal(got, oracle.clamp(want, *c["clamp"]))


def test_slab_tile_width_follows_the_number_of_tiles(ctx):
    """a single round of 124-pixel tiles keeps one accumulator tile per wave; more tiles than CUs at unit stride get
    the two-tile form on tiles of up to 252 pixels (fewer, larger workgroups); stride 2 never does"""
    rng = np.random.default_rng(3)

    def grid_of(n, hw, stride):
        x = rng.integers(-128, 128, (n, hw, hw, 64)).astype(np.int8)
        w = rng.integers(-128, 128, (64, 3, 3, 64)).astype(np.int8)
        bias = np.zeros(64, np.int32)
        _, st = gpu_ops.conv2d(ctx, x, w, bias, (1, 1, 1, 1), (stride, stride), in_zp=-7, w_zp=0)
        assert st == capi.VALID and ctx.last_kernel == "conv2d_slab_i8"
        return ctx.last_launch_shape()[0]

    assert grid_of(8, 56, 1) == 256          # 7 x 14 tiles, 32 per image
    assert grid_of(32, 56, 1) == 512         # 14 x 14 tiles, 16 per image, instead of 1024 tiles of 7 x 14
    assert grid_of(32, 57, 2) > 32 * 29 * 29 // 252 * 2    # stride 2: tiles of at most 124 pixels


@pytest.mark.parametrize("n,hw,shifts,oc", [(8, 56, "uniform", 64), (32, 56, "uniform", 64), (32, 56, "mixed", 64),
                                            (5, 50, "uniform", 64), (40, 28, "mixed", 64), (3, 112, "uniform", 64),
                                            (16, 56, "uniform", 80), (12, 56, "mixed", 48)])
def test_slab_weights_in_registers_form_on_large_tiles(ctx, n, hw, shifts, oc):
    """fused 3x3 layers with 64 input channels: one workgroup per CU walks a tile of several hundred pixels with the
    weights in registers; with one shift for all channels the requantisation of a pixel tile runs inside the K loop of
    the next one, otherwise (mixed shifts) after its own.  From five pixel tiles per workgroup on the weight slab is
    loaded through registers (32 and 16 images of 56 x 56, 3 of 112 x 112; with 80 and 48 output channels a channel block
    of 16 and 48 weight rows, whose loads past the last row are clamped)"""
    rng = np.random.default_rng(n * hw)
    x = rng.integers(-128, 128, (n, hw, hw, 64)).astype(np.int8)
    w = np.clip(np.rint(rng.normal(0, 30, (oc, 3, 3, 64))), -127, 127).astype(np.int8)
    bias = np.rint(rng.normal(0, 1 << 14, oc)).astype(np.int32)
    mult = rng.integers(1 << 30, 1 << 31, oc).astype(np.int32)
    shift = np.full(oc, 38, np.int8) if shifts == "uniform" else rng.integers(31, 41, oc).astype(np.int8)
    c = dict(x=x, w=w, bias=bias, in_zp=-7, pad=(1, 1, 1, 1), stride=(1, 1), dilation=(1, 1), mult=mult, shift=shift,
             out_zp=2, clamp=(0, 127))
    got, st, want, wst = _fused(ctx, c, np.int8)
    assert ctx.last_kernel == "conv2d_slab_wreg_i8_rescale" and st == wst
    assert np.array_equal(got, want), int(np.count_nonzero(got != want))
    if hw == 56 and n in (8, 32) and oc == 64:
        assert ctx.last_launch_shape()[0] == 256    # one round of workgroups: 7 x 14 and 7 x 56 pixels each


@pytest.mark.parametrize("mode", [capi.ROUND_SINGLE, capi.ROUND_DOUBLE])
def test_slab_fused_rescale_per_tensor_scale_and_rounding_modes(ctx, mode):
    shape = (2, 20, 20, 64, (1, 1, 1, 1), (1, 1), (1, 1))
    x, w, bias = _operands(shape, 77)
    c = dict(x=x, w=w, bias=bias, in_zp=3, pad=shape[4], stride=shape[5], dilation=shape[6],
             mult=np.array([1518500250], np.int32), shift=np.array([44], np.int8), out_zp=-5, clamp=None, mode=mode,
             per_channel=False)
    got, st, want, wst = _fused(ctx, c, np.int8)
    assert ctx.last_kernel == "conv2d_slab_wreg_i8_rescale"
    assert st == wst == capi.VALID and np.array_equal(got, want)


def test_slab_fused_rescale_reports_require_conditions(ctx):
    """a shift below 32 makes apply_scale_32 check the value range (quant_util.h:59-67): UNPREDICTABLE, as the
    oracle says for the same operands; pixels and channels outside the tensor raise nothing"""
    shape = (1, 9, 9, 48, (1, 1, 1, 1), (1, 1), (1, 1))
    x, w, bias = _operands(shape, 5)
    c = dict(x=x, w=w, bias=np.zeros(48, np.int32), in_zp=3, pad=shape[4], stride=shape[5], dilation=shape[6],
             mult=np.full(48, 1 << 30, np.int32), shift=np.full(48, 12, np.int8), out_zp=0, clamp=None)
    got, st, want, wst = _fused(ctx, c, np.int8)
    assert ctx.last_kernel == "conv2d_slab_wreg_i8_rescale"
    assert st == wst == capi.UNPREDICTABLE and ctx.flags & capi.FLAG_SCALE_VALUE
    # all-zero operands: every value is legal, also in the lanes that hold no pixel or channel of the tensor
    c["x"], c["w"], c["in_zp"] = np.zeros_like(x), np.zeros_like(w), 0
    got, st, want, wst = _fused(ctx, c, np.int8)
    assert st == wst == capi.VALID and ctx.flags == 0 and np.array_equal(got, want)


def test_slab_kernel_refuses_what_it_cannot_take(ctx):
    rng = np.random.default_rng(1)
    bias = np.zeros(64, np.int32)
    x = rng.integers(-128, 128, (1, 8, 8, 64)).astype(np.int8)
    w = rng.integers(-128, 128, (64, 3, 3, 64)).astype(np.int8)
    with pytest.raises(TmiError):      # a weight zero point
        gpu_ops.conv2d(ctx, x, w, bias, (1, 1, 1, 1), in_zp=0, w_zp=3)
    with pytest.raises(TmiError):      # 32 input channels
        gpu_ops.conv2d(ctx, x[..., :32], w[..., :32], bias, (1, 1, 1, 1))
    with pytest.raises(TmiError):      # 5x5 taps
        gpu_ops.conv2d(ctx, x, rng.integers(-128, 128, (64, 5, 5, 64)).astype(np.int8), bias, (2, 2, 2, 2))
    with pytest.raises(TmiError):      # 40 output channels
        gpu_ops.conv2d(ctx, x, w[:40], bias[:40], (1, 1, 1, 1))


def test_automatic_choice_takes_the_slab_kernel_for_its_layers():
    c = Context(0)
    try:
        shape = (2, 28, 28, 64, (1, 1, 1, 1), (1, 1), (1, 1))
        x, w, bias = _operands(shape, 3)
        got, st = gpu_ops.conv2d(c, x, w, bias, shape[4], in_zp=-7)
        assert st == capi.VALID and c.last_kernel == "conv2d_slab_i8"
        c.set_kernel_choice(capi.KERNEL_MFMA)
        other, st = gpu_ops.conv2d(c, x, w, bias, shape[4], in_zp=-7)
        assert st == capi.VALID and c.last_kernel == "conv2d_mfma_i8" and np.array_equal(got, other)
        c.set_kernel_choice(capi.KERNEL_AUTO)
        got, st = gpu_ops.conv2d(c, x, w, bias, shape[4], in_zp=-7, w_zp=2)     # weight zero point: the patch kernel
        assert st == capi.VALID and c.last_kernel == "conv2d_mfma_i8"
    finally:
        c.close()


# shifts at the borders between the epilogue's forms: 32 with double rounding takes the general form, 33 the
# high-word form; single rounding takes the high-word form from 32 on; a mixture of both; shifts too large for
# output_zp * 2^shift to ride in the rounding term; every multiplier at its extremes
_FORM_CASES = [
    ("uniform 32", lambda rng, oc: np.full(oc, 32)), ("uniform 33", lambda rng, oc: np.full(oc, 33)),
    ("32..34", lambda rng, oc: rng.integers(32, 35, oc)), ("33..36", lambda rng, oc: rng.integers(33, 37, oc)),
    ("30..34", lambda rng, oc: rng.integers(30, 35, oc)), ("uniform 58", lambda rng, oc: np.full(oc, 58)),
    ("52..62", lambda rng, oc: rng.integers(52, 63, oc)),
]


@pytest.mark.parametrize("name,shifts", _FORM_CASES, ids=[c[0] for c in _FORM_CASES])
@pytest.mark.parametrize("mode", [capi.ROUND_SINGLE, capi.ROUND_DOUBLE])
@pytest.mark.parametrize("out_dtype,out_zp", [(np.int8, -128), (np.int8, 127), (np.int16, 0)])
def test_slab_fused_rescale_epilogue_form_borders(ctx, name, shifts, mode, out_dtype, out_zp):
    shape = (2, 13, 11, 80, (1, 1, 1, 1), (1, 1), (1, 1))
    x, _, _ = _operands(shape, 5)
    rng = np.random.default_rng(len(name) + mode)
    oc = shape[3]
    shift = shifts(rng, oc).astype(np.int8)
    # accumulators of a few thousand, so that a shift of 30..36 leaves values inside the output range; the large
    # shifts get accumulators near 2^24 and multipliers near 2^31
    small = int(shift.max()) < 40
    w = rng.integers(-2, 3, (oc, 3, 3, 64)).astype(np.int8) if small else rng.integers(-127, 128, (oc, 3, 3, 64)).astype(np.int8)
    bias = rng.integers(-300, 300, oc).astype(np.int32) if small else rng.integers(-(1 << 24), 1 << 24, oc).astype(np.int32)
    mult = rng.integers(1 << 30, 1 << 31, oc).astype(np.int32)
    mult[:4] = [(1 << 31) - 1, 1 << 30, 0, 1]
    c = dict(x=x, w=w, bias=bias, in_zp=-3, pad=shape[4], stride=shape[5], dilation=shape[6], mult=mult, shift=shift,
             out_zp=out_zp, clamp=None, mode=mode)
    got, st, want, wst = _fused(ctx, c, out_dtype)
    assert ctx.last_kernel == "conv2d_slab_wreg_i8_rescale"
    assert st == wst and np.array_equal(got, want), (st, wst, int(np.count_nonzero(got != want)))
    if small and out_dtype == np.int16:
        assert len(np.unique(got)) > 50
