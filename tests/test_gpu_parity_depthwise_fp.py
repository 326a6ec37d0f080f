"""The fp16 / bf16 DEPTHWISE_CONV2D vector kernel (8 channels per lane, fp32 accumulation over the taps in (ky, kx) order, taps
outside the image skipped, bias added last) through the C ABI: bit for bit against the CPU oracle's fp32 loop nest
(tensor_ops.cpp:1262-1340) on the same fp16 / bf16 operands with the result rounded to the tensor's type - a product of two
such values is exact in fp32, so the kernel's fused multiply-adds round as the reference's multiply and add do - and inside
the reference's DOT_PRODUCT bound against the fp64 oracle (verify_dot_product.cpp:30-139)."""
import numpy as np
import pytest

import cases
import dot_product_check as dp
import gpu_ops
import oracle
from reference_model_amd import Context, capi

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def ctx():
    c = Context(0)
    yield c
    c.close()


SHAPES = [  # n, ih, iw, c, kh, kw, pad, stride, dilation
    (2, 28, 28, 96, 3, 3, (0, 1, 0, 1), (2, 2), (1, 1)),      # the MobileNet layer's geometry, small
    (3, 17, 19, 32, 3, 3, (1, 1, 1, 1), (1, 1), (1, 1)),
    (1, 9, 9, 8, 3, 3, (1, 1, 1, 1), (1, 1), (1, 1)),         # one channel group
    (2, 12, 13, 40, 3, 3, (2, 2, 2, 2), (1, 1), (2, 2)),      # dilation 2, 5 groups: 51 pixels an iteration, one lane idle
    (1, 2, 2, 16, 3, 3, (1, 1, 1, 1), (1, 1), (1, 1)),        # an image smaller than the window: no interior pixel
    (2, 14, 14, 576, 3, 3, (1, 1, 1, 1), (1, 1), (1, 1)),     # 72 groups: 3 pixels an iteration
    (1, 7, 7, 2048, 3, 3, (1, 1, 1, 1), (1, 1), (1, 1)),      # the most channels: one pixel an iteration
    (2, 15, 11, 24, 5, 3, (2, 2, 1, 1), (1, 1), (1, 1)),      # 5 x 3 taps: the loop over taps
    (1, 21, 21, 64, 7, 7, (3, 3, 3, 3), (2, 2), (1, 1)),      # 7 x 7, stride 2
    (40, 30, 30, 48, 3, 3, (1, 1, 1, 1), (1, 1), (1, 1)),     # several iterations per workgroup
    (1, 6, 6, 16, 1, 1, (0, 0, 0, 0), (1, 1), (1, 1)),        # one tap
]


@pytest.mark.parametrize("shape", SHAPES, ids=[f"c{s[3]}k{s[4]}x{s[5]}n{s[0]}" for s in SHAPES])
@pytest.mark.parametrize("kind", ["fp16", "bf16"])
def test_depthwise_fp_vec_matches_the_loop_nest(ctx, kind, shape):
    n, ih, iw, c, kh, kw, pad, stride, dil = shape
    rng = np.random.default_rng(ih * 7 + c + kh)
    x = rng.normal(0, 1, (n, ih, iw, c)).astype(np.float32)
    w = rng.normal(0, 0.4, (kh, kw, c, 1)).astype(np.float32)
    b = rng.normal(0, 0.5, c if c != 40 else 1).astype(np.float32)    # (one layer with a broadcast bias)
    if kind == "fp16":
        xs, ws, bs = x.astype(np.float16), w.astype(np.float16), b.astype(np.float16)
        x32, w32, b32 = (v.astype(np.float32) for v in (xs, ws, bs))
        dtype, narrow = capi.FP16, lambda v: v.astype(np.float16)
    else:
        xs, ws, bs = (cases.float_to_bf16_bits(v) for v in (x, w, b))
        x32, w32, b32 = (cases.bf16_bits_to_float(v).astype(np.float32) for v in (xs, ws, bs))
        dtype, narrow = capi.BF16, cases.float_to_bf16_bits
    got, st = gpu_ops.conv2d(ctx, xs, ws, bs, pad, stride, dil, dtype=dtype, depthwise=True)
    assert st == capi.VALID and ctx.last_kernel == ("depthwise_vec_f16" if kind == "fp16" else "depthwise_vec_bf16")
    want = narrow(oracle.depthwise_conv2d("f32", x32, w32, b32, pad, stride, dil))
    assert np.array_equal(got.view(np.uint16), want.view(np.uint16)), int(np.count_nonzero(got.view(np.uint16) != want.view(np.uint16)))
    # and the reference's own criterion against fp64
    xf, wf, bf = (v.astype(np.float64) for v in (x32, w32, b32))
    ref = oracle.depthwise_conv2d("f64", xf, wf, bf, pad, stride, dil)
    bnd = oracle.depthwise_conv2d("f64", xf, wf, bf, pad, stride, dil, abs_mode=True)
    imp = got.astype(np.float64) if kind == "fp16" else cases.bf16_bits_to_float(got).astype(np.float64)
    assert dp.check(imp, ref, bnd, kind, dp.kernel_size_bound(kh * kw, kind))["ok"]


def test_depthwise_fp_vec_skips_taps_outside_the_image(ctx):
    """an infinite weight under a tap that lies outside the image for a border pixel must not reach that pixel (0 * inf
    would be NaN): the reference skips the tap (tensor_ops.cpp:1302-1313)"""
    x = np.ones((1, 5, 5, 8), np.float16)
    w = np.full((3, 3, 8, 1), 0.5, np.float16)
    w[0, 0, :, 0] = np.inf                       # the top-left tap
    b = np.zeros(8, np.float16)
    got, st = gpu_ops.conv2d(ctx, x, w, b, (1, 1, 1, 1), dtype=capi.FP16, depthwise=True)
    assert st == capi.VALID and ctx.last_kernel == "depthwise_vec_f16"
    assert np.isfinite(got[0, 0, :, :]).all() and np.isfinite(got[0, :, 0, :]).all()    # first row and column: tap outside
    assert np.isinf(got[0, 1:, 1:, :]).all()


def test_depthwise_fp_other_shapes_take_the_general_kernel(ctx):
    rng = np.random.default_rng(3)
    x = rng.normal(0, 1, (1, 8, 8, 12)).astype(np.float16)     # 12 channels: no groups of 8
    w = rng.normal(0, 0.4, (3, 3, 12, 1)).astype(np.float16)
    got, st = gpu_ops.conv2d(ctx, x, w, np.zeros(12, np.float16), (1, 1, 1, 1), dtype=capi.FP16, depthwise=True)
    assert st == capi.VALID and ctx.last_kernel == "depthwise_direct_f16"
    w2 = rng.normal(0, 0.4, (3, 3, 16, 2)).astype(np.float16)   # channel multiplier 2
    x2 = rng.normal(0, 1, (1, 8, 8, 16)).astype(np.float16)
    got, st = gpu_ops.conv2d(ctx, x2, w2, np.zeros(32, np.float16), (1, 1, 1, 1), dtype=capi.FP16, depthwise=True)
    assert st == capi.VALID and ctx.last_kernel == "depthwise_direct_f16"
