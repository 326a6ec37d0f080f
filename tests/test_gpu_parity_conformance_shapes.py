"""The target shapes of the reference's conformance generator for the operators of this path
(verif/conformance/tosa_ext_profile_ops_info.json, groups tosa-pro-int: conv2d :2508-2560, and the depthwise,
transpose, conv3d, matmul, rescale, pooling and clamp groups beside it): axes of 65535..65539 elements next to
axes of 1..3, and the odd mid-sized shapes.  Every case runs with the automatic kernel choice, as a caller of the C
ABI would, and is compared bit for bit with the CPU oracle; kernel and output extents are seeded draws from the
ranges the generator arguments give (--tensor-dim-range), small enough that the oracle takes seconds."""
import numpy as np
import pytest

import gpu_ops
import oracle
from reference_model_amd import Context, capi

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def ctx():
    c = Context(0)
    yield c
    c.close()


def fit(extent, k, dil, stride, lo):
    """pad_hi >= 0 such that (extent - 1 + lo + hi - (k - 1) * dil) is a non-negative multiple of stride"""
    base = extent - 1 + lo - (k - 1) * dil
    hi = (-base) % stride
    while base + hi < 0:
        hi += stride
    return hi


def rescale_operands(rng, oc, lo_shift=30, hi_shift=40):
    return rng.integers(1 << 30, 1 << 31, oc).astype(np.int32), rng.integers(lo_shift, hi_shift, oc).astype(np.int8)


CONV2D = [  # input shape, (OC, KH, KW), stride, dilation, leading pads (top, left)
    ((3, 49, 14, 28), (16, 3, 3), (1, 1), (1, 1), (1, 1)),
    ((3, 49, 14, 28), (7, 5, 2), (2, 3), (2, 1), (2, 0)),
    ((3, 49, 14, 28), (1, 1, 1), (1, 1), (1, 1), (0, 0)),
    ((3, 49, 14, 28), (13, 16, 9), (4, 2), (1, 1), (3, 5)),
    ((1, 11, 44, 13), (9, 3, 3), (1, 1), (1, 1), (1, 1)),
    ((1, 11, 44, 13), (16, 2, 7), (3, 2), (1, 3), (0, 4)),
    ((1, 11, 44, 13), (5, 11, 1), (1, 5), (1, 1), (0, 0)),
    ((1, 65535, 3, 1), (8, 3, 3), (1, 1), (1, 1), (1, 1)),
    ((1, 65535, 3, 1), (1, 8, 1), (7, 2), (1, 1), (0, 0)),
    ((1, 65535, 3, 1), (5, 1, 3), (1, 1), (1, 1), (0, 1)),
    ((1, 2, 65536, 1), (8, 2, 5), (1, 3), (1, 1), (0, 2)),
    ((1, 2, 65536, 1), (3, 1, 1), (2, 1), (1, 1), (0, 0)),
    ((1, 2, 65536, 1), (6, 3, 8), (1, 8), (1, 1), (1, 0)),
]


@pytest.mark.parametrize("case", CONV2D, ids=lambda c: "x".join(map(str, c[0])) + "_k" + "x".join(map(str, c[1])))
def test_conv2d_int8_conformance_target_shapes(ctx, case):
    shape, (oc, kh, kw), stride, dil, (pt, pl) = case
    rng = np.random.default_rng(sum(shape) + 31 * oc + kh)
    pad = (pt, fit(shape[1], kh, dil[0], stride[0], pt), pl, fit(shape[2], kw, dil[1], stride[1], pl))
    x = rng.integers(-128, 128, shape).astype(np.int8)
    w = rng.integers(-128, 128, (oc, kh, kw, shape[3])).astype(np.int8)
    bias = rng.integers(-(1 << 20), 1 << 20, oc).astype(np.int32)
    in_zp, w_zp = int(rng.integers(-128, 128)), int(rng.integers(-128, 128))
    want = oracle.conv2d("i8", x, w, bias, pad, stride, dil, in_zp=in_zp, w_zp=w_zp)
    got, st = gpu_ops.conv2d(ctx, x, w, bias, pad, stride, dil, in_zp=in_zp, w_zp=w_zp)
    assert st == capi.VALID and np.array_equal(got, want), ctx.last_kernel
    mult, shift = rescale_operands(rng, oc)
    got, st = gpu_ops.conv2d(ctx, x, w, bias, pad, stride, dil, in_zp=in_zp, w_zp=w_zp,
                             rescale=dict(mult=mult, shift=shift, out_zp=-5), clamp=(-100, 90))
    ref, rst = oracle.rescale(want, mult, shift, out_zp=-5)
    assert st == rst and np.array_equal(got, oracle.clamp(ref, -100, 90)), ctx.last_kernel


DEPTHWISE = [  # input shape, (KH, KW, M), stride, dilation, leading pads
    ((1, 9, 44, 3), (3, 3, 1), (1, 1), (1, 1), (1, 1)),
    ((1, 9, 44, 3), (2, 5, 4), (2, 3), (2, 1), (0, 2)),
    ((4, 11, 33, 1), (3, 3, 16), (1, 1), (1, 1), (1, 1)),
    ((4, 11, 33, 1), (11, 4, 2), (1, 2), (1, 1), (0, 1)),
    ((1, 65532, 2, 1), (3, 2, 1), (1, 1), (1, 1), (1, 0)),
    ((1, 65532, 2, 1), (16, 1, 3), (4, 1), (1, 1), (0, 0)),
    ((1, 4, 65537, 1), (3, 3, 2), (1, 1), (1, 1), (1, 1)),
    ((1, 4, 65537, 1), (1, 9, 1), (1, 8), (1, 1), (0, 0)),
]


@pytest.mark.parametrize("case", DEPTHWISE, ids=lambda c: "x".join(map(str, c[0])) + "_k" + "x".join(map(str, c[1])))
def test_depthwise_conv2d_int8_conformance_target_shapes(ctx, case):
    shape, (kh, kw, m), stride, dil, (pt, pl) = case
    c = shape[3]
    rng = np.random.default_rng(sum(shape) + 17 * m + kw)
    pad = (pt, fit(shape[1], kh, dil[0], stride[0], pt), pl, fit(shape[2], kw, dil[1], stride[1], pl))
    x = rng.integers(-128, 128, shape).astype(np.int8)
    w = rng.integers(-128, 128, (kh, kw, c, m)).astype(np.int8)
    bias = rng.integers(-(1 << 16), 1 << 16, c * m).astype(np.int32)
    in_zp, w_zp = int(rng.integers(-128, 128)), int(rng.integers(-128, 128))
    want = oracle.depthwise_conv2d("i8", x, w, bias, pad, stride, dil, in_zp=in_zp, w_zp=w_zp)
    got, st = gpu_ops.conv2d(ctx, x, w, bias, pad, stride, dil, in_zp=in_zp, w_zp=w_zp, depthwise=True)
    assert st == capi.VALID and np.array_equal(got, want), ctx.last_kernel
    mult, shift = rescale_operands(rng, c * m, 26, 36)
    got, st = gpu_ops.conv2d(ctx, x, w, bias, pad, stride, dil, in_zp=in_zp, w_zp=w_zp, depthwise=True,
                             rescale=dict(mult=mult, shift=shift, out_zp=3))
    ref, rst = oracle.rescale(want, mult, shift, out_zp=3)
    assert st == rst and np.array_equal(got, ref), ctx.last_kernel


TCONV = [  # input shape, (OC, KH, KW), stride, out_pad
    ((2, 25, 33, 1), (8, 3, 3), (1, 1), (0, 0, 0, 0)),
    ((2, 25, 33, 1), (18, 2, 5), (2, 3), (1, 0, 0, 2)),
    ((3, 4, 31, 3), (5, 4, 4), (2, 2), (-1, -1, -1, -1)),
    ((3, 4, 31, 3), (1, 1, 1), (3, 1), (0, 2, 0, 0)),
    ((2, 65536, 1, 1), (4, 3, 1), (1, 1), (0, 0, 0, 0)),
    ((2, 65536, 1, 1), (12, 2, 3), (2, 1), (0, 1, -1, 0)),
]


@pytest.mark.parametrize("case", TCONV, ids=lambda c: "x".join(map(str, c[0])) + "_k" + "x".join(map(str, c[1])))
def test_transpose_conv2d_int8_conformance_target_shapes(ctx, case):
    shape, (oc, kh, kw), stride, out_pad = case
    rng = np.random.default_rng(sum(shape) + 13 * oc + kw)
    x = rng.integers(-128, 128, shape).astype(np.int8)
    w = rng.integers(-128, 128, (oc, kh, kw, shape[3])).astype(np.int8)
    bias = rng.integers(-(1 << 20), 1 << 20, oc).astype(np.int32)
    in_zp, w_zp = int(rng.integers(-128, 128)), int(rng.integers(-128, 128))
    want = oracle.transpose_conv2d("i8", x, w, bias, out_pad, stride, in_zp, w_zp)
    got, st = gpu_ops.transpose_conv2d(ctx, x, w, bias, out_pad, stride, in_zp, w_zp)
    assert st == capi.VALID and np.array_equal(got, want), ctx.last_kernel


CONV3D = [  # input shape, (OC, KD, KH, KW), stride, leading pads (d, h, w)
    ((1, 9, 21, 14, 1), (4, 3, 3, 3), (1, 1, 1), (1, 1, 1)),
    ((3, 3, 11, 12, 3), (2, 2, 4, 1), (1, 2, 3), (0, 1, 0)),
    ((1, 1, 65535, 2, 1), (2, 1, 2, 2), (1, 1, 1), (0, 0, 0)),
    ((2, 1, 1, 65536, 1), (1, 1, 1, 2), (1, 1, 2), (0, 0, 0)),
]


@pytest.mark.parametrize("case", CONV3D, ids=lambda c: "x".join(map(str, c[0])) + "_k" + "x".join(map(str, c[1])))
def test_conv3d_int8_conformance_target_shapes(ctx, case):
    shape, (oc, kd, kh, kw), stride, lead = case
    rng = np.random.default_rng(sum(shape) + 7 * oc + kd)
    pad = []
    for axis, (k, lo) in enumerate(zip((kd, kh, kw), lead)):
        pad += [lo, fit(shape[1 + axis], k, 1, stride[axis], lo)]
    x = rng.integers(-128, 128, shape).astype(np.int8)
    w = rng.integers(-128, 128, (oc, kd, kh, kw, shape[4])).astype(np.int8)
    bias = rng.integers(-(1 << 20), 1 << 20, oc).astype(np.int32)
    in_zp, w_zp = int(rng.integers(-128, 128)), int(rng.integers(-128, 128))
    want = oracle.conv3d("i8", x, w, bias, tuple(pad), stride, (1, 1, 1), in_zp, w_zp)
    got, st = gpu_ops.conv3d(ctx, x, w, bias, tuple(pad), stride, (1, 1, 1), in_zp, w_zp)
    assert st == capi.VALID and np.array_equal(got, want), ctx.last_kernel


@pytest.mark.parametrize("a_shape,w", [((1, 65532, 1), 5), ((1, 2, 65538), 3), ((2000, 1, 1), 1), ((1, 65532, 1), 1),
                                       ((1, 2, 65538), 16), ((2000, 1, 1), 7)])
def test_matmul_int8_conformance_target_shapes(ctx, a_shape, w):
    rng = np.random.default_rng(sum(a_shape) + w)
    a = rng.integers(-128, 128, a_shape).astype(np.int8)
    b = rng.integers(-128, 128, (a_shape[0], a_shape[2], w)).astype(np.int8)
    a_zp, b_zp = int(rng.integers(-128, 128)), int(rng.integers(-128, 128))
    got, st = gpu_ops.matmul(ctx, a, b, a_zp, b_zp)
    assert st == capi.VALID and np.array_equal(got, oracle.matmul("i8", a, b, a_zp, b_zp)), ctx.last_kernel


@pytest.mark.parametrize("shape", [(1, 2, 65533, 1), (1, 65539, 1, 1), (1, 2, 1, 65536)])
@pytest.mark.parametrize("per_channel", [False, True])
def test_rescale_and_clamp_conformance_target_shapes(ctx, shape, per_channel):
    rng = np.random.default_rng(sum(shape))
    x = rng.integers(-128, 128, shape).astype(np.int8)
    nc = shape[-1] if per_channel else 1
    mult, shift = rescale_operands(rng, nc, 30, 38)
    got, st = gpu_ops.rescale(ctx, x, mult, shift, in_zp=-7, out_zp=11, out_dtype=np.int8, per_channel=per_channel)
    want, wst = oracle.rescale(x, mult, shift, in_zp=-7, out_zp=11, out_dtype=np.int8, per_channel=per_channel)
    assert st == wst and np.array_equal(got, want)
    got, st = gpu_ops.clamp(ctx, x, -77, 55)
    assert st == capi.VALID and np.array_equal(got, oracle.clamp(x, -77, 55))


POOL = [  # input shape, kernel, stride, leading pads
    ((1, 49, 42, 28), (3, 3), (2, 2), (1, 1)), ((1, 11, 44, 3), (4, 2), (1, 3), (0, 0)),
    ((1, 65535, 5, 1), (3, 2), (2, 1), (1, 0)), ((1, 3, 65537, 1), (2, 5), (1, 4), (0, 2)),
    ((1, 4, 75, 3), (2, 3), (2, 3), (0, 0)), ((1, 3, 2, 1), (3, 2), (1, 1), (0, 0)),
]


@pytest.mark.parametrize("case", POOL, ids=lambda c: "x".join(map(str, c[0])))
@pytest.mark.parametrize("avg", [False, True])
def test_pooling_int8_conformance_target_shapes(ctx, case, avg):
    shape, kernel, stride, (pt, pl) = case
    rng = np.random.default_rng(sum(shape) + kernel[0])
    pad = (pt, min(fit(shape[1], kernel[0], 1, stride[0], pt), kernel[0] - 1), pl,
           min(fit(shape[2], kernel[1], 1, stride[1], pl), kernel[1] - 1))
    assert oracle.pool_out_hw(shape[1], shape[2], kernel, stride, pad) is not None
    x = rng.integers(-128, 128, shape).astype(np.int8)
    if avg:
        want = oracle.avg_pool2d(x, kernel, stride, pad, -3, 4)
        got, st = gpu_ops.pool2d(ctx, x, kernel, stride, pad, True, -3, 4)
    else:
        want = oracle.max_pool2d(x, kernel, stride, pad)
        got, st = gpu_ops.pool2d(ctx, x, kernel, stride, pad, False)
    assert st == capi.VALID and np.array_equal(got, want), ctx.last_kernel


# ---- the sizes of the generator's --level-8k-sizes groups: kernels, strides, dilations and pads at MAX_KERNEL =
# MAX_STRIDE = 8192 (tosa_ext_profile_ops_info.json, third group of each operator), with the level set: the
# operators stay VALID at the limit
@pytest.fixture()
def ctx_8k():
    c = Context(0)
    c.set_level(capi.LEVEL_EIGHTK)
    yield c
    c.close()


CONV_8K = [  # input shape, (OC, KH, KW), stride, dilation, pad
    ((1, 8193, 2, 2), (3, 8192, 1), (1, 1), (1, 1), (0, 0, 0, 0)),
    ((1, 3, 8195, 1), (2, 2, 8192), (1, 3), (1, 1), (0, 0, 0, 0)),
    ((1, 8193, 3, 3), (2, 1, 2), (8192, 1), (1, 1), (0, 0, 0, 0)),
    ((1, 4097, 2, 2), (2, 2, 1), (1, 1), (4096, 1), (0, 0, 0, 0)),
    ((2, 2, 2, 4), (3, 2, 2), (1, 1), (1, 1), (8192, 0, 0, 0)),
    ((1, 2, 3, 2), (2, 3, 2), (1, 1), (1, 1), (0, 1, 0, 8192)),
]


@pytest.mark.parametrize("case", CONV_8K, ids=lambda c: "x".join(map(str, c[0])) + "_k" + "x".join(map(str, c[1])))
def test_conv2d_and_depthwise_at_the_8k_level_limits(ctx_8k, case):
    shape, (oc, kh, kw), stride, dil, pad = case
    rng = np.random.default_rng(sum(shape) + kh + kw)
    x = rng.integers(-128, 128, shape).astype(np.int8)
    w = rng.integers(-128, 128, (oc, kh, kw, shape[3])).astype(np.int8)
    bias = rng.integers(-(1 << 20), 1 << 20, oc).astype(np.int32)
    want = oracle.conv2d("i8", x, w, bias, pad, stride, dil, in_zp=-3, w_zp=5)
    got, st = gpu_ops.conv2d(ctx_8k, x, w, bias, pad, stride, dil, in_zp=-3, w_zp=5)
    assert st == capi.VALID and ctx_8k.flags == 0 and np.array_equal(got, want), ctx_8k.last_kernel
    wd = rng.integers(-128, 128, (kh, kw, shape[3], 2)).astype(np.int8)
    bd = rng.integers(-(1 << 16), 1 << 16, shape[3] * 2).astype(np.int32)
    want = oracle.depthwise_conv2d("i8", x, wd, bd, pad, stride, dil, in_zp=-3, w_zp=5)
    got, st = gpu_ops.conv2d(ctx_8k, x, wd, bd, pad, stride, dil, in_zp=-3, w_zp=5, depthwise=True)
    assert st == capi.VALID and np.array_equal(got, want), ctx_8k.last_kernel


def test_pooling_and_transpose_conv2d_at_the_8k_level_limits(ctx_8k):
    rng = np.random.default_rng(8192)
    x = rng.integers(-128, 128, (1, 8193, 3, 2)).astype(np.int8)
    got, st = gpu_ops.pool2d(ctx_8k, x, (8192, 1), (1, 1), avg=False)
    assert st == capi.VALID and np.array_equal(got, oracle.max_pool2d(x, (8192, 1), (1, 1)))
    got, st = gpu_ops.pool2d(ctx_8k, x, (8192, 2), (1, 1), (0, 0, 0, 0), True, -5, 7)
    assert st == capi.VALID and np.array_equal(got, oracle.avg_pool2d(x, (8192, 2), (1, 1), (0, 0, 0, 0), -5, 7))
    got, st = gpu_ops.pool2d(ctx_8k, x, (2, 1), (8191, 2), avg=False)
    assert st == capi.VALID and np.array_equal(got, oracle.max_pool2d(x, (2, 1), (8191, 2)))
    xt = rng.integers(-128, 128, (1, 2, 2, 3)).astype(np.int8)
    wt = rng.integers(-128, 128, (2, 2, 3, 3)).astype(np.int8)
    bt = rng.integers(-1000, 1000, 2).astype(np.int32)
    got, st = gpu_ops.transpose_conv2d(ctx_8k, xt, wt, bt, (0, 0, 0, 0), (8192, 1), -4, 0)
    assert st == capi.VALID and np.array_equal(got, oracle.transpose_conv2d("i8", xt, wt, bt, (0, 0, 0, 0), (8192, 1), -4, 0))
    wk = rng.integers(-128, 128, (1, 8192, 1, 3)).astype(np.int8)
    got, st = gpu_ops.transpose_conv2d(ctx_8k, xt, wk, bt[:1], (0, 0, 0, 0), (1, 1), -4, 2)
    assert st == capi.VALID and np.array_equal(got, oracle.transpose_conv2d("i8", xt, wk, bt[:1], (0, 0, 0, 0), (1, 1), -4, 2))
