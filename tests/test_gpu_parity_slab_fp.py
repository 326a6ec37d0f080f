"""The slab kernel's fp16 / bf16 instantiations (CONV2D with 3x3 taps on channel vectors of 64 ... 128 bytes, 1x1 taps on up
to 1024 bytes; fp32 accumulation from the bias, results rounded to the tensor's type) through the C ABI against the fp64
oracle (tensor_ops.cpp:828-882) with the reference's DOT_PRODUCT bound (verify_dot_product.cpp:30-139), plus at most 2 ulp of
the output type on results that are no cancellation: strides, dilation, padding, ragged tiles and channel blocks, both
accumulator-tile forms, every channel-vector size the kernel is built for."""
import numpy as np
import pytest

import cases
import dot_product_check as dp
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


SHAPES = [  # n, ih, iw, ic, oc, k, pad, stride, dilation
    (2, 20, 20, 64, 64, 3, (1, 1, 1, 1), (1, 1), (1, 1)),
    (3, 17, 19, 32, 48, 3, (1, 1, 1, 1), (1, 1), (1, 1)),       # ragged tiles, one channel block of 48
    (2, 21, 23, 48, 80, 3, (0, 0, 0, 0), (2, 2), (1, 1)),       # stride 2, two channel blocks, the second of 16
    (1, 24, 24, 64, 128, 3, (2, 2, 2, 2), (1, 1), (2, 2)),      # dilation 2
    (9, 40, 40, 32, 64, 3, (1, 1, 1, 1), (1, 1), (1, 1)),       # more tiles than CUs: two accumulator tiles per wave
    (2, 28, 28, 64, 256, 1, (0, 0, 0, 0), (1, 1), (1, 1)),      # pointwise, 128-byte channel vectors
    (2, 14, 14, 80, 64, 1, (0, 0, 0, 0), (1, 1), (1, 1)),       # every other size: 160 bytes
    (10, 38, 38, 96, 48, 1, (0, 0, 0, 0), (1, 1), (1, 1)),      # 192, two accumulator tiles per wave
    (2, 14, 14, 128, 96, 1, (1, 0, 0, 1), (1, 1), (1, 1)),      # 256, padding on a pointwise layer
    (2, 15, 13, 160, 64, 1, (0, 0, 0, 0), (2, 2), (1, 1)),      # 320, stride 2
    (2, 14, 14, 192, 112, 1, (0, 0, 0, 0), (1, 1), (1, 1)),     # 384
    (2, 14, 14, 256, 64, 1, (0, 0, 0, 0), (1, 1), (1, 1)),      # 512
    (2, 9, 14, 384, 64, 1, (0, 0, 0, 0), (1, 1), (1, 1)),       # 768
    (3, 14, 14, 512, 144, 1, (0, 0, 0, 0), (1, 1), (1, 1)),     # 1024 bytes: tiles of 62 pixels
]


@pytest.mark.parametrize("shape", SHAPES, ids=[f"{s[3]}to{s[4]}k{s[5]}" for s in SHAPES])
@pytest.mark.parametrize("kind", ["fp16", "bf16"])
def test_slab_fp_within_dot_product_bound(ctx, kind, shape):
    n, ih, iw, ic, oc, k, pad, stride, dil = shape
    rng = np.random.default_rng(ih * 31 + ic + oc)
    x = rng.normal(0, 1, (n, ih, iw, ic)).astype(np.float32)
    w = rng.normal(0, 1 / np.sqrt(k * k * ic), (oc, k, k, ic)).astype(np.float32)
    b = rng.normal(0, 0.5, oc if ic != 80 else 1).astype(np.float32)    # (one layer with a broadcast bias)
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
    assert st == capi.VALID and ctx.last_kernel == ("conv2d_slab_f16" if kind == "fp16" else "conv2d_slab_bf16")
    imp = got.astype(np.float64) if kind == "fp16" else cases.bf16_bits_to_float(got).astype(np.float64)
    res = dp.check(imp, ref, bnd, kind, dp.kernel_size_bound(k * k * ic, kind))
    # tolerance: |imp - ref| <= 2 ksb max(bnd 2^-(1+frac), normal_min) per element and the variance limit of the check; and at
    # most 2 ulp of the output type where the result is at least an eighth of the sum of |products|
    assert res["ok"] and res["max_ulp_conditioned"] <= 2.0, res
    assert np.isfinite(imp).all() and len(np.unique(got)) > 100


def test_slab_fp_special_values(ctx):
    """infinities and NaNs travel through the accumulators as IEEE arithmetic has them; padding contributes exact zeros"""
    rng = np.random.default_rng(5)
    x = rng.normal(0, 1, (1, 8, 8, 64)).astype(np.float16)
    w = rng.normal(0, 0.05, (64, 3, 3, 64)).astype(np.float16)
    b = np.zeros(64, np.float16)
    x[0, 2, 2, 5], x[0, 6, 6, 7] = np.inf, np.nan
    got, st = gpu_ops.conv2d(ctx, x, w, b, (1, 1, 1, 1), dtype=capi.FP16)
    assert st == capi.VALID and ctx.last_kernel == "conv2d_slab_f16"
    ref = oracle.conv2d("f64", x.astype(np.float64), w.astype(np.float64), b.astype(np.float64), (1, 1, 1, 1))
    assert np.array_equal(np.isnan(got), np.isnan(ref))
    fin = np.isfinite(ref)
    assert np.array_equal(np.isinf(got) & ~np.isnan(got), np.isinf(ref) & ~np.isnan(ref))
    assert np.allclose(got[fin].astype(np.float64), ref[fin], rtol=2e-3, atol=2e-3)    # fp16 rounding of an fp32 sum


def test_slab_fp_refuses_what_it_cannot_take(ctx):
    rng = np.random.default_rng(1)
    x = rng.normal(0, 1, (1, 8, 8, 128)).astype(np.float16)
    w = rng.normal(0, 0.05, (64, 3, 3, 128)).astype(np.float16)
    with pytest.raises(TmiError):      # 3x3 taps on 256-byte channel vectors
        gpu_ops.conv2d(ctx, x, w, np.zeros(64, np.float16), (1, 1, 1, 1), dtype=capi.FP16)
    with pytest.raises(TmiError):      # 40 output channels
        gpu_ops.conv2d(ctx, x[..., :64], w[:40, :, :, :64], np.zeros(40, np.float16), (1, 1, 1, 1), dtype=capi.FP16)


def test_automatic_choice_takes_the_slab_kernel_for_small_fp_layers():
    c = Context(0)
    try:
        rng = np.random.default_rng(2)
        for shape, kernel in (((2, 28, 28, 64, 64, 3, 1), "conv2d_slab_f16"),       # 3x3 on 128-byte vectors
                              ((2, 14, 14, 256, 128, 1, 0), "conv2d_slab_f16"),     # pointwise, 50 176 results
                              ((8, 56, 56, 64, 256, 1, 0), "gemm_mfma_f16")):       # pointwise, 6.4 M results: whole-line stores
            n, ih, iw, ic, oc, k, p = shape
            x = rng.normal(0, 1, (n, ih, iw, ic)).astype(np.float16)
            w = rng.normal(0, 1 / np.sqrt(k * k * ic), (oc, k, k, ic)).astype(np.float16)
            b = rng.normal(0, 0.1, oc).astype(np.float16)
            got, st = gpu_ops.conv2d(c, x, w, b, (p, p, p, p), dtype=capi.FP16)
            assert st == capi.VALID and c.last_kernel == kernel
    finally:
        c.close()
