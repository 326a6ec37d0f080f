"""INT16 x INT8 -> INT48 CONV2D / DEPTHWISE_CONV2D and INT16 x INT16 -> INT48 MATMUL (tensor_ops.cpp:2225, 2247, 2257) through
the C ABI, bit for bit against the CPU oracle: int64 accumulation, the weights' zero point, the 48-bit clip of the
result, the argument rules that differ from the INT8 instantiations."""
import numpy as np
import pytest

import gpu_ops
import oracle
from reference_model_amd import Context, TmiError, capi

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def ctx():
    c = Context(0)
    yield c
    c.close()


SHAPES = [
    # n, h, w, ic, oc, kh, kw, pad, stride, dilation
    (1, 8, 8, 16, 8, 3, 3, (1, 1, 1, 1), (1, 1), (1, 1)),
    (2, 10, 7, 5, 3, 3, 2, (1, 0, 0, 1), (2, 1), (1, 1)),
    (1, 11, 13, 7, 4, 2, 3, (0, 1, 2, 0), (1, 2), (2, 1)),
    (3, 5, 5, 33, 17, 1, 1, (0, 0, 0, 0), (1, 1), (1, 1)),
]


@pytest.mark.parametrize("shape", SHAPES)
@pytest.mark.parametrize("w_zp", [0, -7])
def test_conv2d_int16_to_int48(ctx, shape, w_zp):
    n, h, w_, ic, oc, kh, kw, pad, stride, dil = shape
    rng = np.random.default_rng(hash((shape, w_zp)) & 0xffff)
    x = rng.integers(-32768, 32768, (n, h, w_, ic)).astype(np.int16)
    wt = rng.integers(-128, 128, (oc, kh, kw, ic)).astype(np.int8)
    bias = rng.integers(-(1 << 44), 1 << 44, oc).astype(np.int64)
    out_hw = oracle.conv_out_hw(h, w_, kh, kw, pad, stride, dil)
    assert out_hw is not None
    want = oracle.conv2d("i16", x, wt, bias, pad, stride, dil, w_zp=w_zp)
    got, st = gpu_ops.conv2d(ctx, x, wt, bias, pad, stride, dil, w_zp=w_zp)
    assert st == capi.VALID and ctx.last_kernel == "conv2d_direct_i16_i48"
    assert got.dtype == np.int64 and np.array_equal(got, want)


@pytest.mark.parametrize("m", [1, 2])
def test_depthwise_int16_to_int48(ctx, m):
    rng = np.random.default_rng(40 + m)
    x = rng.integers(-32768, 32768, (2, 10, 9, 12)).astype(np.int16)
    wt = rng.integers(-128, 128, (3, 3, 12, m)).astype(np.int8)
    bias = rng.integers(-(1 << 40), 1 << 40, 12 * m).astype(np.int64)
    want = oracle.depthwise_conv2d("i16", x, wt, bias, (1, 1, 1, 1), w_zp=5)
    got, st = gpu_ops.conv2d(ctx, x, wt, bias, (1, 1, 1, 1), w_zp=5, depthwise=True)
    assert st == capi.VALID and ctx.last_kernel == "depthwise_direct_i16_i48" and np.array_equal(got, want)


def test_matmul_int16_to_int48(ctx):
    rng = np.random.default_rng(3)
    a = rng.integers(-32768, 32768, (3, 17, 40)).astype(np.int16)
    b = rng.integers(-32768, 32768, (3, 40, 9)).astype(np.int16)
    want = oracle.matmul("i16", a, b)
    got, st = gpu_ops.matmul(ctx, a, b)
    assert st == capi.VALID and ctx.last_kernel == "matmul_direct_i16_i48" and np.array_equal(got, want)


def test_int48_results_are_clipped_to_48_bits(ctx):
    """sums beyond 2^47 (every product at its largest, and a bias at the edge of the range) come back as the 48-bit limits"""
    lim = (1 << 47) - 1
    x = np.full((1, 1, 1, 4096), -32768, np.int16)
    wt = np.stack([np.full((1, 1, 4096), -128, np.int8), np.full((1, 1, 4096), 127, np.int8)])    # [2,1,1,4096]
    bias = np.array([lim, -lim - 1], np.int64)
    want = oracle.conv2d("i16", x, wt, bias)
    got, st = gpu_ops.conv2d(ctx, x, wt, bias)
    assert st == capi.VALID and np.array_equal(got, want) and got.ravel().tolist() == [lim, -lim - 1]
    a = np.full((1, 2, 140000), 32767, np.int16)
    a[0, 1] = -32768
    b = np.full((1, 140000, 1), 32767, np.int16)
    got, st = gpu_ops.matmul(ctx, a, b)    # 140000 * 2^30 > 2^47
    assert st == capi.VALID and np.array_equal(got, oracle.matmul("i16", a, b)) and got.ravel().tolist() == [lim, -lim - 1]


def test_int16_argument_rules(ctx):
    """only INT8 tensors have a zero point (tensor_ops.cpp:805, 1433-1434); the INT8 weights of an INT16 convolution keep
    theirs; an INT16 convolution has an INT48 result and accumulator, and no fused RESCALE"""
    x = np.zeros((1, 4, 4, 4), np.int16)
    wt = np.zeros((2, 1, 1, 4), np.int8)
    bias = np.zeros(2, np.int64)
    with pytest.raises(TmiError, match="Input zero point must be zero"):
        gpu_ops.conv2d(ctx, x, wt, bias, in_zp=1)
    a = np.zeros((1, 2, 2), np.int16)
    with pytest.raises(TmiError, match="A zeropoint must be zero"):
        gpu_ops.matmul(ctx, a, a, a_zp=1)
    d = ctx.conv_desc(capi.INT16, capi.INT32, x.shape, 2, 1, 1, (4, 4), (0, 0, 0, 0), (1, 1), (1, 1), 2)
    with pytest.raises(TmiError, match="Output data type"):
        ctx.conv2d(d, ctx.upload(x), ctx.upload(wt), ctx.upload(bias), 0, 0, ctx.empty((1, 4, 4, 2), capi.INT48, np.int64))
    d = ctx.conv_desc(capi.INT16, capi.INT48, x.shape, 2, 1, 1, (4, 4), (0, 0, 0, 0), (1, 1), (1, 1), 2, acc_dtype=capi.INT32)
    with pytest.raises(TmiError, match="accumulator type"):
        ctx.conv2d(d, ctx.upload(x), ctx.upload(wt), ctx.upload(bias), 0, 0, ctx.empty((1, 4, 4, 2), capi.INT48, np.int64))
    d = ctx.conv_desc(capi.INT16, capi.INT48, x.shape, 2, 1, 1, (4, 4), (0, 0, 0, 0), (1, 1), (1, 1), 2)
    r = ctx.rescale_desc(capi.INT32, capi.INT8, 2, 2)
    with pytest.raises(TmiError, match="fused rescale needs an INT8 convolution"):
        ctx.conv2d_rescale_clamp(d, ctx.upload(x), ctx.upload(wt), ctx.upload(bias), 0, 0, r,
                                 ctx.upload(np.full(2, 1 << 30, np.int32)), ctx.upload(np.full(2, 30, np.int8)),
                                 ctx.empty((1, 4, 4, 2), capi.INT8, np.int8))
    for t in list(ctx._owned):
        ctx._free(t)


@pytest.mark.parametrize("geom", [((2, 6, 7, 16), (8, 3, 3, 16), (0, 1, -1, 0), (2, 2)), ((1, 9, 5, 12), (5, 2, 4, 12), (1, 1, 0, 2), (1, 3)),
                                  ((3, 4, 4, 40), (24, 3, 3, 40), (0, 0, 0, 0), (1, 1))])
@pytest.mark.parametrize("w_zp", [0, 9])
def test_transpose_conv2d_int16_to_int48(ctx, geom, w_zp):
    """INT16 x INT8 -> INT48 TRANSPOSE_CONV2D (tensor_ops.cpp:2291): tap flip and hole insertion on operands of two element
    sizes, then the 64-bit one-result-per-lane kernel"""
    xs, ws, out_pad, stride = geom
    rng = np.random.default_rng(xs[1] * 7 + ws[0])
    x = rng.integers(-32768, 32768, xs).astype(np.int16)
    w = rng.integers(-128, 128, ws).astype(np.int8)
    bias = rng.integers(-(1 << 40), 1 << 40, ws[0]).astype(np.int64)
    got, st = gpu_ops.transpose_conv2d(ctx, x, w, bias, out_pad, stride, w_zp=w_zp)
    assert st == capi.VALID and got.dtype == np.int64
    assert np.array_equal(got, oracle.transpose_conv2d("i16", x, w, bias, out_pad, stride, w_zp=w_zp))


@pytest.mark.parametrize("geom", [((1, 4, 5, 5, 8), (4, 2, 3, 3, 8), (1, 0, 1, 1, 1, 1), (1, 1, 1), (1, 1, 1)),
                                  ((2, 6, 7, 4, 12), (6, 3, 1, 2, 12), (1, 2, 0, 0, 1, 0), (2, 1, 1), (1, 2, 1)),
                                  ((1, 3, 9, 9, 32), (16, 1, 3, 3, 32), (0, 0, 1, 1, 1, 1), (1, 2, 2), (1, 1, 1))])
@pytest.mark.parametrize("w_zp", [0, -3])
def test_conv3d_int16_to_int48(ctx, geom, w_zp):
    """INT16 x INT8 -> INT48 CONV3D (tensor_ops.cpp:2237): depth gather and weight permutation on operands of two element
    sizes, then the 64-bit one-result-per-lane kernel"""
    xs, ws, pad, stride, dil = geom
    rng = np.random.default_rng(xs[2] * 5 + ws[0])
    x = rng.integers(-32768, 32768, xs).astype(np.int16)
    w = rng.integers(-128, 128, ws).astype(np.int8)
    bias = rng.integers(-(1 << 40), 1 << 40, 1 if ws[0] == 6 else ws[0]).astype(np.int64)
    got, st = gpu_ops.conv3d(ctx, x, w, bias, pad, stride, dil, w_zp=w_zp)
    assert st == capi.VALID and got.dtype == np.int64
    assert np.array_equal(got, oracle.conv3d("i16", x, w, bias, pad, stride, dil, w_zp=w_zp))


def test_transpose_conv2d_and_conv3d_int16_rules(ctx):
    x = np.zeros((1, 3, 3, 4), np.int16)
    w = np.zeros((2, 2, 2, 4), np.int8)
    with pytest.raises(TmiError, match="Input zero point must be zero"):
        gpu_ops.transpose_conv2d(ctx, x, w, np.zeros(2, np.int64), in_zp=1)
    with pytest.raises(TmiError, match="Input zero point must be zero"):
        gpu_ops.conv3d(ctx, x[None], w[:, None], np.zeros(2, np.int64), in_zp=-1)
    lim = (1 << 47) - 1
    one = np.full((1, 1, 1, 8), 32767, np.int16)
    wt = np.full((1, 1, 1, 8), 127, np.int8)
    got, st = gpu_ops.transpose_conv2d(ctx, one, wt, np.array([lim], np.int64))
    assert st == capi.VALID and got.ravel().tolist() == [lim]
    got, st = gpu_ops.conv3d(ctx, -one[None], wt[None], np.array([-lim - 1], np.int64))
    assert st == capi.VALID and got.ravel().tolist() == [-lim - 1]
