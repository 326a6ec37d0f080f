"""GPU parity of the MFMA CONV2D kernel (implicit GEMM with fused bias / zero-point / RESCALE / CLAMP
epilogue) against the CPU oracle, through the C ABI.  int8 results are compared bit for bit; fp16 / bf16
results with the reference's DOT_PRODUCT bound against the fp64 oracle (tolerance printed in the assert)."""
import numpy as np
import pytest

import cases
import dot_product_check as dp
import gpu_ops
import oracle
from reference_model_amd import Context, TmiError, capi
from test_oracle_kats import CONV_SHAPES

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def ctx():
    c = Context(0)
    c.set_kernel_choice(capi.KERNEL_MFMA)
    yield c
    c.close()


MFMA_SHAPES = CONV_SHAPES + [
    # n, ih, iw, ic, oc, kh, kw, pad, stride, dilation
    (1, 32, 32, 8, 16, 1, 1, (0, 0, 0, 0), (1, 1), (1, 1)),       # config 1 geometry
    (2, 14, 14, 64, 64, 3, 3, (1, 1, 1, 1), (1, 1), (1, 1)),      # config 3 geometry, small
    (1, 9, 9, 16, 16, 3, 3, (1, 1, 1, 1), (2, 2), (1, 1)),
    (1, 10, 10, 32, 40, 3, 3, (2, 2, 2, 2), (1, 1), (2, 2)),      # dilation, OC not a multiple of 16
    (1, 6, 200, 24, 20, 1, 3, (0, 0, 1, 1), (1, 1), (1, 1)),      # wide rows split into two tiles
    (1, 7, 7, 160, 96, 3, 3, (1, 1, 1, 1), (1, 1), (1, 1)),       # three channel blocks, two OC blocks
    (2, 5, 5, 100, 33, 2, 2, (0, 1, 0, 1), (1, 1), (1, 1)),       # ragged channel tail (100 = 64 + 36)
    (1, 3, 65, 3, 8, 1, 1, (0, 0, 0, 0), (1, 1), (1, 1)),
    (1, 16, 16, 48, 64, 5, 5, (2, 2, 2, 2), (1, 1), (1, 1)),
    (1, 1, 1, 1, 1, 1, 1, (0, 0, 0, 0), (1, 1), (1, 1)),
]


@pytest.mark.parametrize("shape", MFMA_SHAPES)
@pytest.mark.parametrize("zps", [(-7, 3), (5, 0), (0, -4), (0, 0), (-128, 127)])
def test_conv2d_i8_mfma_bit_exact(ctx, shape, zps):
    n, ih, iw, ic, oc, kh, kw, pad, stride, dil = shape
    rng = np.random.default_rng(sum(shape[:7]) + 1000 * (zps[0] + 128) + zps[1] + 128)
    x = rng.integers(-128, 128, (n, ih, iw, ic)).astype(np.int8)
    w = rng.integers(-128, 128, (oc, kh, kw, ic)).astype(np.int8)
    bias = rng.integers(-65536, 65536, oc).astype(np.int32)
    want = oracle.conv2d("i8", x, w, bias, pad, stride, dil, in_zp=zps[0], w_zp=zps[1])
    got, st = gpu_ops.conv2d(ctx, x, w, bias, pad, stride, dil, in_zp=zps[0], w_zp=zps[1])
    assert ctx.last_kernel == "conv2d_mfma_i8"
    assert st == capi.VALID and np.array_equal(got, want), int(np.count_nonzero(got != want))


@pytest.mark.parametrize("ic", [6, 12, 20, 40, 72, 104, 200])
@pytest.mark.parametrize("taps,stride", [(1, 1), (3, 1), (3, 2)])
def test_conv2d_i8_channel_vectors_of_words(ctx, ic, taps, stride):
    """channel vectors that are not whole 16-byte chunks are staged by 8-byte words (40, 72, 104, 200 channels), 4-byte
    words (12, 20) or bytes (6), over one channel block or several (72 and more)"""
    rng = np.random.default_rng(ic * 10 + taps + stride)
    pad = (taps // 2,) * 4
    x = rng.integers(-128, 128, (2, 11, 13, ic)).astype(np.int8)
    w = rng.integers(-128, 128, (24, taps, taps, ic)).astype(np.int8)
    bias = rng.integers(-65536, 65536, 24).astype(np.int32)
    oh, ow = (11 + 2 * pad[0] - taps) // stride + 1, (13 + 2 * pad[0] - taps) // stride + 1
    x = x[:, :(oh - 1) * stride + taps - 2 * pad[0], :(ow - 1) * stride + taps - 2 * pad[0]]
    want = oracle.conv2d("i8", x, w, bias, pad, (stride, stride), (1, 1), in_zp=-5, w_zp=2)
    got, st = gpu_ops.conv2d(ctx, x, w, bias, pad, (stride, stride), (1, 1), in_zp=-5, w_zp=2)
    assert ctx.last_kernel == "conv2d_mfma_i8"
    assert st == capi.VALID and np.array_equal(got, want), int(np.count_nonzero(got != want))


@pytest.mark.parametrize("shape", MFMA_SHAPES[5:9])
def test_conv2d_i8_mfma_broadcast_bias(ctx, shape):
    n, ih, iw, ic, oc, kh, kw, pad, stride, dil = shape
    rng = np.random.default_rng(77)
    x = rng.integers(-128, 128, (n, ih, iw, ic)).astype(np.int8)
    w = rng.integers(-127, 128, (oc, kh, kw, ic)).astype(np.int8)
    bias = np.array([-12345], np.int32)
    want = oracle.conv2d("i8", x, w, bias, pad, stride, dil, in_zp=2, w_zp=0)
    got, st = gpu_ops.conv2d(ctx, x, w, bias, pad, stride, dil, in_zp=2, w_zp=0)
    assert st == capi.VALID and np.array_equal(got, want)


def _fused_expect(c, out_dtype=np.int8):
    acc = oracle.conv2d("i8", c["x"], c["w"], c["bias"], c["pad"], c["stride"], c["dilation"], c["in_zp"], c["w_zp"])
    want, st = oracle.rescale(acc, c["mult"], c["shift"], out_zp=c["out_zp"], out_dtype=out_dtype)
    assert st == oracle.VALID
    if c["clamp"] is not None:
        want = oracle.clamp(want, *c["clamp"])
    return want


def _fused_run(ctx, c, out_dtype=np.int8):
    return gpu_ops.conv2d(ctx, c["x"], c["w"], c["bias"], c["pad"], c["stride"], c["dilation"], c["in_zp"], c["w_zp"],
                          rescale=dict(mult=c["mult"], shift=c["shift"], out_zp=c["out_zp"], out_dtype=out_dtype),
                          clamp=c["clamp"])


def test_config1_conv_rescale(ctx):
    c = cases.c1()
    got, st = _fused_run(ctx, c)
    assert ctx.last_kernel == "conv2d_mfma_i8_rescale"
    assert st == capi.VALID and np.array_equal(got, _fused_expect(c))


def test_config3_resnet_conv_rescale_clamp_full_size(ctx):
    c = cases.c3()
    got, st = _fused_run(ctx, c)
    want = _fused_expect(c)
    assert st == capi.VALID and np.array_equal(got, want), int(np.count_nonzero(got != want))
    assert got.min() == 0 and got.max() == 127  # the clamp range is exercised on both ends


@pytest.mark.parametrize("out_dtype", [np.int8, np.int16, np.int32])
def test_fused_rescale_output_types_and_ragged_channels(ctx, out_dtype):
    rng = np.random.default_rng(5)
    c = dict(x=rng.integers(-128, 128, (2, 9, 13, 20)).astype(np.int8),
             w=rng.integers(-127, 128, (37, 3, 3, 20)).astype(np.int8),
             bias=rng.integers(-5000, 5000, 37).astype(np.int32), in_zp=-11, w_zp=0, pad=(1, 1, 1, 1), stride=(1, 1),
             dilation=(1, 1), mult=rng.integers(1 << 30, 1 << 31, 37).astype(np.int32),
             shift=rng.integers(33, 44, 37).astype(np.int8), out_zp=0 if out_dtype != np.int8 else -6,
             clamp=None)
    got, st = _fused_run(ctx, c, out_dtype)
    assert st == capi.VALID and np.array_equal(got, _fused_expect(c, out_dtype))


@pytest.mark.parametrize("shift", [32, 33, 38, 62])
@pytest.mark.parametrize("zw", [0, 5])
def test_fused_rescale_one_shift_for_all_channels(ctx, shift, zw):
    """All channels share one shift of at least 32: the epilogue variant with scalar rounding terms.  Ragged
    channel counts (37 of 64, 130 of 192) bring channels past OC into the tables."""
    for oc, out_zp in ((37, -6), (130, 9)):
        rng = np.random.default_rng(shift * 7 + oc)
        c = dict(x=rng.integers(-128, 128, (2, 9, 11, 32)).astype(np.int8),
                 w=rng.integers(-127, 128, (oc, 3, 3, 32)).astype(np.int8),
                 bias=rng.integers(-5000, 5000, oc).astype(np.int32), in_zp=-11, w_zp=zw, pad=(1, 1, 1, 1),
                 stride=(1, 1), dilation=(1, 1), mult=rng.integers(1 << 30, 1 << 31, oc).astype(np.int32),
                 shift=np.full(oc, shift, np.int8), out_zp=out_zp, clamp=(-100, 90))
        got, st = _fused_run(ctx, c)
        assert st == capi.VALID and np.array_equal(got, _fused_expect(c)), (oc, shift)


def test_large_shifts_with_output_zero_point_do_not_overflow(ctx):
    """output_zp * 2^shift does not fit 64 bits next to the product for shifts near 62: the kernels that fold the
    zero point into the rounding term must stop doing so there (stand-alone RESCALE, depthwise, CONV2D with
    mixed shifts)."""
    rng = np.random.default_rng(62)
    x = rng.integers(-(1 << 31), 1 << 31, (50, 8), dtype=np.int64).astype(np.int32)
    mult = rng.integers(1 << 30, 1 << 31, 8).astype(np.int32)
    shift = np.array([62, 61, 55, 53, 52, 51, 40, 33], np.int8)
    for out_zp, od, unsigned in ((-128, np.int8, False), (127, np.int8, False)):
        want, wst = oracle.rescale(x, mult, shift, out_zp=out_zp, out_dtype=od, output_unsigned=unsigned)
        got, st = gpu_ops.rescale(ctx, x, mult, shift, out_zp=out_zp, out_dtype=od, output_unsigned=unsigned)
        assert ctx.last_kernel == "rescale_fast" and st == wst == capi.VALID and np.array_equal(got, want)
    c = cases.c4(n=1, hw=12, c=8)
    c["shift"], c["out_zp"] = shift, -128
    got, st = gpu_ops.conv2d(ctx, c["x"], c["w"], c["bias"], c["pad"], c["stride"], c["dilation"], c["in_zp"],
                             c["w_zp"], depthwise=True, rescale=dict(mult=c["mult"], shift=shift, out_zp=-128))
    assert st == capi.VALID and np.array_equal(got, _dw_expect(c))
    c = cases.c1()
    c["shift"], c["out_zp"] = np.resize(shift, 16), 127
    got, st = _fused_run(ctx, c)
    assert st == capi.VALID and np.array_equal(got, _fused_expect(c))


def test_fused_rescale_require_condition_is_reported(ctx):
    c = cases.c1()
    c["shift"] = np.full(16, 12, np.int8)  # |acc| exceeds 2^11: apply_scale_32's value range (quant_util.h:59-67)
    _, st = _fused_run(ctx, c)
    assert st == capi.UNPREDICTABLE and ctx.flags & capi.FLAG_SCALE_VALUE


def test_property_linearity_in_bias_and_zero_weights(ctx):
    """Size-independent properties at the full config-3 shape: zero weights give exactly the bias, and adding
    a constant to the bias adds it to every int32 output."""
    c = cases.c3()
    z = np.zeros_like(c["w"])
    out0, _ = gpu_ops.conv2d(ctx, c["x"], z, c["bias"], c["pad"], in_zp=c["in_zp"])
    assert np.array_equal(out0, np.broadcast_to(c["bias"], out0.shape))
    a, _ = gpu_ops.conv2d(ctx, c["x"], c["w"], c["bias"], c["pad"], in_zp=c["in_zp"])
    b, _ = gpu_ops.conv2d(ctx, c["x"], c["w"], c["bias"] + 1000, c["pad"], in_zp=c["in_zp"])
    assert np.array_equal(b - a, np.full_like(a, 1000))
    # an input equal to the zero point everywhere contributes nothing, padding included
    flat = np.full_like(c["x"], c["in_zp"])
    out1, _ = gpu_ops.conv2d(ctx, flat, c["w"], c["bias"], c["pad"], in_zp=c["in_zp"])
    assert np.array_equal(out1, np.broadcast_to(c["bias"], out1.shape))


@pytest.mark.parametrize("kind", ["fp16", "bf16"])
@pytest.mark.parametrize("shape", [(2, 8, 8, 32, 48, 3, 3, (1, 1, 1, 1), (1, 1), (1, 1)),
                                   (1, 9, 9, 24, 20, 3, 3, (0, 0, 0, 0), (2, 2), (1, 1)),
                                   (1, 7, 7, 256, 64, 3, 3, (1, 1, 1, 1), (1, 1), (1, 1))])
def test_conv2d_fp_mfma_within_dot_product_bound(ctx, kind, shape):
    n, ih, iw, ic, oc, kh, kw, pad, stride, dil = shape
    rng = np.random.default_rng(31 + ic)
    x = rng.normal(0, 1, (n, ih, iw, ic)).astype(np.float32)
    w = rng.normal(0, 1 / np.sqrt(kh * kw * ic), (oc, kh, kw, ic)).astype(np.float32)
    b = rng.normal(0, 0.1, oc).astype(np.float32)
    if kind == "fp16":
        xs, ws, bs = x.astype(np.float16), w.astype(np.float16), b.astype(np.float16)
        xf, wf, bf = (v.astype(np.float64) for v in (xs, ws, bs))
        dtype = capi.FP16
    else:
        xs, ws, bs = (cases.float_to_bf16_bits(v) for v in (x, w, b))
        xf, wf, bf = (cases.bf16_bits_to_float(v).astype(np.float64) for v in (xs, ws, bs))
        dtype = capi.BF16
    ref = oracle.conv2d("f64", xf, wf, bf, pad, stride, dil)
    bnd = oracle.conv2d("f64", xf, wf, bf, pad, stride, dil, abs_mode=True)
    got, st = gpu_ops.conv2d(ctx, xs, ws, bs, pad, stride, dil, dtype=dtype)
    assert ctx.last_kernel == ("conv2d_mfma_f16" if kind == "fp16" else "conv2d_mfma_bf16")
    imp = got.astype(np.float64) if kind == "fp16" else cases.bf16_bits_to_float(got).astype(np.float64)
    ksb = dp.kernel_size_bound(kh * kw * ic, kind)
    res = dp.check(imp, ref, bnd, kind, ksb)
    # tolerance: |imp-ref| <= 2*ksb * max(bnd*2^-(1+frac), normal_min) per element, sum err^2 <= 1.6*ksb*T
    assert st == capi.VALID and res["ok"], res
    assert res["max_ulp"] <= 2.0, res  # fp32 accumulation: the result is the correctly rounded value +- 1 ulp


@pytest.mark.parametrize("kind", ["fp16", "bf16"])
@pytest.mark.parametrize("ic", [3, 6, 10, 20, 36])
def test_conv2d_fp_channel_vectors_of_words(ctx, kind, ic):
    """16-bit channel vectors of 6 bytes (staged by bytes), 12 and 20 (4-byte words), 40 and 72 (8-byte words)"""
    rng = np.random.default_rng(900 + ic)
    pad, stride, dil = (1, 1, 1, 1), (1, 1), (1, 1)
    x = rng.normal(0, 1, (2, 9, 10, ic)).astype(np.float32)
    w = rng.normal(0, 1 / np.sqrt(9 * ic), (20, 3, 3, ic)).astype(np.float32)
    b = rng.normal(0, 0.1, 20).astype(np.float32)
    if kind == "fp16":
        xs, ws, bs = x.astype(np.float16), w.astype(np.float16), b.astype(np.float16)
        xf, wf, bf = (v.astype(np.float64) for v in (xs, ws, bs))
        dtype = capi.FP16
    else:
        xs, ws, bs = (cases.float_to_bf16_bits(v) for v in (x, w, b))
        xf, wf, bf = (cases.bf16_bits_to_float(v).astype(np.float64) for v in (xs, ws, bs))
        dtype = capi.BF16
    ref = oracle.conv2d("f64", xf, wf, bf, pad, stride, dil)
    bnd = oracle.conv2d("f64", xf, wf, bf, pad, stride, dil, abs_mode=True)
    got, st = gpu_ops.conv2d(ctx, xs, ws, bs, pad, stride, dil, dtype=dtype)
    assert ctx.last_kernel == ("conv2d_mfma_f16" if kind == "fp16" else "conv2d_mfma_bf16")
    imp = got.astype(np.float64) if kind == "fp16" else cases.bf16_bits_to_float(got).astype(np.float64)
    res = dp.check(imp, ref, bnd, kind, dp.kernel_size_bound(9 * ic, kind))
    # tolerance: the DOT_PRODUCT bound of the reference's verifier, and at most 2 ulp of the output type
    assert st == capi.VALID and res["ok"] and res["max_ulp"] <= 2.0, res


# ---- GEMM-sized work: the 128-channel x 256-pixel workgroup shape and pipelined channel blocks ---------------
BIG_SHAPES = [
    # n, ih, iw, ic, oc, kh, kw, pad, stride, dilation
    (1, 256, 256, 128, 128, 1, 1, (0, 0, 0, 0), (1, 1), (1, 1)),    # one 128-byte channel block
    (2, 128, 128, 128, 200, 3, 3, (1, 1, 1, 1), (1, 1), (1, 1)),    # 3x3, four pipelined blocks, ragged OC
    (1, 300, 220, 528, 96, 1, 1, (0, 0, 0, 0), (1, 1), (1, 1)),     # 528 = 4*128 + 16: short last block
    (4, 131, 131, 64, 136, 3, 3, (0, 0, 0, 0), (2, 2), (1, 1)),     # stride 2, rows that do not fill a tile
    (16, 28, 28, 256, 64, 3, 3, (1, 1, 1, 1), (1, 1), (1, 1)),      # 64-channel shape with pipelined blocks
]


@pytest.mark.parametrize("shape", BIG_SHAPES)
@pytest.mark.parametrize("zps", [(-7, 3), (11, 0)])
def test_conv2d_i8_mfma_gemm_sized_bit_exact(ctx, shape, zps):
    """Expected values from the float64-BLAS restatement (checked against the oracle by the CPU suite), plus the
    scalar oracle itself on the first image's first rows."""
    n, ih, iw, ic, oc, kh, kw, pad, stride, dil = shape
    rng = np.random.default_rng(sum(shape[:7]) + zps[0])
    x = rng.integers(-128, 128, (n, ih, iw, ic)).astype(np.int8)
    w = rng.integers(-128, 128, (oc, kh, kw, ic)).astype(np.int8)
    bias = rng.integers(-65536, 65536, oc).astype(np.int32)
    want = cases.conv2d_exact_blas(x, w, bias, pad, stride, dil, *zps)
    got, st = gpu_ops.conv2d(ctx, x, w, bias, pad, stride, dil, in_zp=zps[0], w_zp=zps[1])
    assert ctx.last_kernel == "conv2d_mfma_i8"
    assert st == capi.VALID and np.array_equal(got, want), int(np.count_nonzero(got != want))
    rows = 2 * stride[0] + (kh - 1) * dil[0] + 1 - pad[0]    # input rows behind the first three output rows
    sl = oracle.conv2d("i8", x[:1, :rows], w, bias, (pad[0], 0, pad[2], pad[3]), stride, dil, in_zp=zps[0],
                       w_zp=zps[1])
    assert np.array_equal(got[0, :3], sl[0])


@pytest.mark.parametrize("mode", ["fast", "generic16", "int16out"])
def test_conv2d_i8_gemm_sized_fused_rescale(ctx, mode):
    n, ih, iw, ic, oc, kh, kw, pad, stride, dil = BIG_SHAPES[1]
    rng = np.random.default_rng(99)
    x = rng.integers(-128, 128, (n, ih, iw, ic)).astype(np.int8)
    w = np.clip(np.rint(rng.normal(0, 20, (oc, kh, kw, ic))), -127, 127).astype(np.int8)
    bias = rng.integers(-65536, 65536, oc).astype(np.int32)
    acc = cases.conv2d_exact_blas(x, w, bias, pad, stride, dil, -7, 0)
    if mode == "generic16":
        # a 16-bit multiplier on the int32 accumulator: not the fast path, the staged general RESCALE
        mult, shift, scale32 = rng.integers(1 << 13, 1 << 15, oc).astype(np.int32), np.full(oc, 26, np.int8), False
        rounding = capi.ROUND_SINGLE
    else:
        mult, shift, scale32 = rng.integers(1 << 30, 1 << 31, oc).astype(np.int32), rng.integers(37, 41, oc).astype(np.int8), True
        rounding = capi.ROUND_DOUBLE
    od = np.int16 if mode == "int16out" else np.int8
    out_zp = 0 if mode == "int16out" else -3    # a non-zero output_zp is an ERROR_IF for int16
    want, wst = oracle.rescale(acc, mult, shift, in_zp=0, out_zp=out_zp, out_dtype=od, scale32=scale32,
                               rounding_mode=oracle.ROUND_DOUBLE if scale32 else oracle.ROUND_SINGLE, per_channel=True)
    assert wst == oracle.VALID
    got, st = gpu_ops.conv2d(ctx, x, w, bias, pad, stride, dil, in_zp=-7, w_zp=0,
                             rescale=dict(mult=mult, shift=shift, out_zp=out_zp, out_dtype=od, scale32=scale32,
                                          rounding_mode=rounding))
    assert ctx.last_kernel == "conv2d_mfma_i8_rescale"
    assert st == capi.VALID and np.array_equal(got, want), int(np.count_nonzero(got != want))


def test_mfma_not_eligible_is_an_error_when_forced(ctx):
    # a 31x31 kernel with 64 output channels needs a 4.9 MB weight slab: no MFMA tiling fits LDS
    x = np.zeros((1, 31, 31, 64), np.int8)
    w = np.zeros((64, 31, 31, 64), np.int8)
    with pytest.raises(TmiError) as e:
        gpu_ops.conv2d(ctx, x, w, np.zeros(1, np.int32))
    assert "kernel is eligible" in e.value.message


# ---- MATMUL on the matrix cores ----------------------------------------------------------------------
MATMUL_SHAPES = [(1, 2, 2, 2), (3, 17, 29, 11), (2, 128, 64, 128), (1, 33, 100, 65), (2, 70, 256, 40),
                 (1, 1, 1024, 1), (4, 96, 48, 200)]


@pytest.mark.parametrize("shape", MATMUL_SHAPES)
@pytest.mark.parametrize("zps", [(-5, 3), (0, 0), (127, -128)])
def test_matmul_i8_mfma_bit_exact(ctx, shape, zps):
    n, h, c, w = shape
    rng = np.random.default_rng(n * 1000 + h + c + w)
    a = rng.integers(-128, 128, (n, h, c)).astype(np.int8)
    b = rng.integers(-128, 128, (n, c, w)).astype(np.int8)
    got, st = gpu_ops.matmul(ctx, a, b, *zps)
    assert ctx.last_kernel == "matmul_mfma_i8"
    assert st == capi.VALID and np.array_equal(got, oracle.matmul("i8", a, b, *zps))


@pytest.mark.parametrize("k", [128, 320])
def test_matmul_i8_largest_tile_bit_exact(ctx, k):
    """[4,2048,k] x [4,k,2048]: GEMM-sized enough for the 128-channel x 512-pixel workgroup shape (one channel block
    for k = 128, five pipelined 64-byte blocks for k = 320).  Expected values from a float64 BLAS product (exact)."""
    rng = np.random.default_rng(k)
    a = rng.integers(-128, 128, (4, 2048, k)).astype(np.int8)
    b = rng.integers(-128, 128, (4, k, 2048)).astype(np.int8)
    got, st = gpu_ops.matmul(ctx, a, b, 7, -9)
    assert st == capi.VALID and ctx.last_kernel == "matmul_mfma_i8"
    want = np.matmul(a.astype(np.float64) - 7, b.astype(np.float64) + 9)
    assert np.array_equal(got, want.astype(np.int64).astype(np.int32))
    assert np.array_equal(got[3, :40], oracle.matmul("i8", a[3:4, :40], b[3:4], 7, -9)[0])


def test_config2_matmul_full_size(ctx):
    """[8,1024,1024] x [8,1024,1024] -> int32, a_zp -5, b_zp 3: every element against a float64 BLAS product
    (exact: |sum| < 2^53), one batch against the scalar oracle, plus the transposition property
    (A.B)^T = B^T.A^T computed by the same kernel."""
    c = cases.c2()
    got, st = gpu_ops.matmul(ctx, c["a"], c["b"], c["a_zp"], c["b_zp"])
    assert st == capi.VALID and ctx.last_kernel == "matmul_mfma_i8"
    want = np.matmul(c["a"].astype(np.float64) - c["a_zp"], c["b"].astype(np.float64) - c["b_zp"])
    assert np.array_equal(got, want.astype(np.int64).astype(np.int32))
    assert np.array_equal(got[5], oracle.matmul("i8", c["a"][5:6], c["b"][5:6], c["a_zp"], c["b_zp"])[0])
    at = np.ascontiguousarray(c["a"].transpose(0, 2, 1))
    bt = np.ascontiguousarray(c["b"].transpose(0, 2, 1))
    got_t, _ = gpu_ops.matmul(ctx, bt, at, c["b_zp"], c["a_zp"])
    assert np.array_equal(got_t, got.transpose(0, 2, 1))


@pytest.mark.parametrize("kind", ["fp16", "bf16"])
def test_matmul_fp_mfma_within_dot_product_bound(ctx, kind):
    rng = np.random.default_rng(8)
    n, h, c, w = 2, 96, 512, 72
    a = rng.normal(0, 1 / 8, (n, h, c)).astype(np.float32)
    b = rng.normal(0, 1 / 8, (n, c, w)).astype(np.float32)
    if kind == "fp16":
        a_s, b_s, dtype = a.astype(np.float16), b.astype(np.float16), capi.FP16
        af, bf = a_s.astype(np.float64), b_s.astype(np.float64)
    else:
        a_s, b_s, dtype = cases.float_to_bf16_bits(a), cases.float_to_bf16_bits(b), capi.BF16
        af, bf = cases.bf16_bits_to_float(a_s).astype(np.float64), cases.bf16_bits_to_float(b_s).astype(np.float64)
    got, st = gpu_ops.matmul(ctx, a_s, b_s, dtype=dtype)
    assert st == capi.VALID and got.dtype == np.float32
    ref, bnd = np.matmul(af, bf), np.matmul(np.abs(af), np.abs(bf))
    res = dp.check(got, ref, bnd, "fp32", dp.kernel_size_bound(c, "fp32", has_bias=False))
    # tolerance: |imp-ref| <= 2*C * max(bnd*2^-24, 2^-126) per element and sum err^2 <= 1.6*C*T
    assert res["ok"], res


# ---- DEPTHWISE_CONV2D, four channels per lane with dot4 across taps ---------------------------------------
@pytest.mark.parametrize("shape", [  # n, ih, iw, c, kh, kw, pad, stride, dilation
    (2, 10, 8, 16, 3, 3, (0, 1, 0, 1), (2, 2), (1, 1)),
    (1, 9, 9, 48, 3, 3, (1, 1, 1, 1), (1, 1), (1, 1)),
    (1, 12, 7, 32, 5, 3, (2, 2, 1, 1), (1, 1), (1, 1)),
    (3, 8, 8, 96, 3, 3, (2, 2, 2, 2), (1, 1), (2, 2)),
    (1, 11, 13, 20, 5, 5, (2, 2, 2, 2), (1, 1), (1, 1)),      # 25 taps, channels a multiple of 4 only
    (2, 7, 9, 4, 1, 1, (0, 0, 0, 0), (2, 2), (1, 1)),         # one tap, one channel group
    (1, 6, 40, 260, 2, 2, (0, 0, 1, 1), (1, 1), (1, 1)),      # 65 channel groups: three pixels per iteration
    (1, 70, 70, 1024, 1, 2, (0, 0, 0, 1), (1, 1), (1, 1)),    # a whole workgroup per pixel, several iterations
])
@pytest.mark.parametrize("zps", [(4, 0), (-3, 7), (0, 0)])
def test_depthwise_dot4_bit_exact(ctx, shape, zps):
    n, ih, iw, c, kh, kw, pad, stride, dil = shape
    rng = np.random.default_rng(c + kh)
    x = rng.integers(-128, 128, (n, ih, iw, c)).astype(np.int8)
    w = rng.integers(-127, 128, (kh, kw, c, 1)).astype(np.int8)
    for bias in (rng.integers(-30000, 30000, c).astype(np.int32), np.array([-77], np.int32)):
        want = oracle.depthwise_conv2d("i8", x, w, bias, pad, stride, dil, *zps)
        got, st = gpu_ops.conv2d(ctx, x, w, bias, pad, stride, dil, *zps, depthwise=True)
        assert ctx.last_kernel == "depthwise_dot4_i8"
        assert st == capi.VALID and np.array_equal(got, want)


def _dw_expect(c, out_dtype=np.int8):
    acc = oracle.depthwise_conv2d("i8", c["x"], c["w"], c["bias"], c["pad"], c["stride"], c["dilation"], c["in_zp"],
                                  c["w_zp"])
    want, st = oracle.rescale(acc, c["mult"], c["shift"], out_zp=c["out_zp"], out_dtype=out_dtype)
    assert st == oracle.VALID
    return want if c["clamp"] is None else oracle.clamp(want, *c["clamp"])


def test_config4_depthwise_rescale_full_size(ctx):
    c = cases.c4()
    got, st = gpu_ops.conv2d(ctx, c["x"], c["w"], c["bias"], c["pad"], c["stride"], c["dilation"], c["in_zp"],
                             c["w_zp"], depthwise=True, rescale=dict(mult=c["mult"], shift=c["shift"],
                                                                     out_zp=c["out_zp"]))
    assert ctx.last_kernel == "depthwise_dot4_i8_rescale"
    want = _dw_expect(c)
    assert st == capi.VALID and got.shape == (8, 56, 56, 96) and np.array_equal(got, want)


@pytest.mark.parametrize("out_dtype", [np.int16, np.int32])
def test_depthwise_rescale_other_outputs_and_clamp(ctx, out_dtype):
    c = cases.c4(n=1, hw=16, c=32)
    c["clamp"] = None
    got, st = gpu_ops.conv2d(ctx, c["x"], c["w"], c["bias"], c["pad"], c["stride"], c["dilation"], c["in_zp"],
                             c["w_zp"], depthwise=True, rescale=dict(mult=c["mult"], shift=c["shift"],
                                                                     out_zp=0, out_dtype=out_dtype))
    assert st == capi.VALID and np.array_equal(got, _dw_expect(c, out_dtype))
    c["clamp"] = (-5, 60)
    got, st = gpu_ops.conv2d(ctx, c["x"], c["w"], c["bias"], c["pad"], c["stride"], c["dilation"], c["in_zp"],
                             c["w_zp"], depthwise=True, clamp=c["clamp"],
                             rescale=dict(mult=c["mult"], shift=c["shift"], out_zp=0))
    assert st == capi.VALID and np.array_equal(got, _dw_expect(c))


def test_depthwise_small_shifts_take_the_checked_path(ctx):
    """Shifts below 32 switch on apply_scale_32's value-range test (quant_util.h:59-67): legal values stay VALID
    and bit-exact, a violation is reported as UNPREDICTABLE."""
    c = cases.c4(n=1, hw=16, c=32)
    c["mult"] = np.full(32, 1 << 20, np.int32)
    c["shift"] = np.full(32, 24, np.int8)    # |acc| < 2^23 holds: 9 * 128 * 132 + 2^15 < 2^18
    kw = dict(depthwise=True, rescale=dict(mult=c["mult"], shift=c["shift"], out_zp=c["out_zp"]))
    got, st = gpu_ops.conv2d(ctx, c["x"], c["w"], c["bias"], c["pad"], c["stride"], c["dilation"], c["in_zp"],
                             c["w_zp"], **kw)
    assert ctx.last_kernel == "depthwise_dot4_i8_rescale"
    assert st == capi.VALID and np.array_equal(got, _dw_expect(c))
    c["shift"] = np.full(32, 10, np.int8)    # now |acc| exceeds 2^9 somewhere
    kw["rescale"]["shift"] = c["shift"]
    _, st = gpu_ops.conv2d(ctx, c["x"], c["w"], c["bias"], c["pad"], c["stride"], c["dilation"], c["in_zp"],
                           c["w_zp"], **kw)
    assert st == capi.UNPREDICTABLE and ctx.flags & capi.FLAG_SCALE_VALUE


def test_depthwise_multiplier_falls_back_to_direct_kernel():
    c2 = Context(0)
    try:
        rng = np.random.default_rng(1)
        x = rng.integers(-128, 128, (1, 6, 6, 16)).astype(np.int8)
        w = rng.integers(-127, 128, (3, 3, 16, 2)).astype(np.int8)
        bias = rng.integers(-100, 100, 32).astype(np.int32)
        got, st = gpu_ops.conv2d(c2, x, w, bias, (1, 1, 1, 1), in_zp=3, depthwise=True)
        assert c2.last_kernel == "depthwise_direct_i8"
        assert np.array_equal(got, oracle.depthwise_conv2d("i8", x, w, bias, (1, 1, 1, 1), in_zp=3))
    finally:
        c2.close()
