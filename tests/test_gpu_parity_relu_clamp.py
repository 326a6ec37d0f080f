"""The fused RESCALE with double rounding where the result's lower limit is at or above output_zp (a ReLU-style CLAMP, or
output_zp at the type's minimum): a negative accumulator is clamped away with either rounding term, so the kernels'
high-word forms skip the sign test there (apply_scale_32's double rounding: quant_util.h:60-90; the limits:
type_conversion.cpp:372-389, and the CLAMP after it).  Every kernel that has the form, per-channel and uniform shifts,
bit for bit against the CPU oracle; each case also runs with a limit one below output_zp, where the sign test must stay."""
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


# kernel choice, (n, ih, iw, ic, oc, k, pad, stride), depthwise, kernel expected
LAYERS = [
    (capi.KERNEL_POINTWISE, (2, 20, 20, 32, 72, 1, 0, 1), False, "conv2d_pointwise_i8_rescale"),
    (capi.KERNEL_POINTWISE, (2, 12, 12, 24, 40, 1, 0, 1), False, "conv2d_pointwise_i8_rescale"),
    (capi.KERNEL_POINTWISE, (2, 12, 12, 320, 72, 1, 0, 1), False, "conv2d_pointwise_ksplit_i8_rescale"),
    (capi.KERNEL_POINTWISE, (2, 10, 10, 96, 40, 3, 1, 1), False, "conv2d_ksplit_i8_rescale"),
    (capi.KERNEL_POINTWISE, (2, 31, 31, 3, 24, 3, 1, 2), False, "conv2d_stem_i8_rescale"),
    (capi.KERNEL_SLAB, (2, 20, 20, 64, 64, 3, 1, 1), False, "conv2d_slab_wreg_i8_rescale"),
    (capi.KERNEL_SLAB, (2, 20, 20, 128, 96, 3, 1, 1), False, "conv2d_slab_i8_rescale"),
    (capi.KERNEL_SLAB, (2, 20, 20, 128, 96, 1, 0, 1), False, "conv2d_slab_i8_rescale"),
    (capi.KERNEL_SLAB, (2, 21, 21, 96, 96, 3, 1, 1), True, "depthwise_mfma_i8_rescale"),
    (capi.KERNEL_SLAB, (1, 15, 15, 320, 320, 3, 1, 2), True, "depthwise_mfma_i8_rescale"),
    (capi.KERNEL_STREAM, (2, 21, 21, 96, 96, 3, 1, 1), True, "depthwise_stream_i8_rescale"),
    (capi.KERNEL_STREAM, (1, 15, 15, 336, 336, 3, 1, 2), True, "depthwise_stream_i8_rescale"),
]


@pytest.mark.parametrize("choice,shape,depthwise,kernel", LAYERS, ids=[f"{l[3]}-{l[1][3]}" for l in LAYERS])
@pytest.mark.parametrize("shifts", ["per channel", "uniform"])
@pytest.mark.parametrize("out_dtype", [np.int8, np.int16])
def test_lower_limit_at_or_above_output_zp(ctx, choice, shape, depthwise, kernel, shifts, out_dtype):
    n, ih, iw, ic, oc, k, p, s = shape
    rng = np.random.default_rng(ic * 7 + oc + k)
    x = rng.integers(-128, 128, (n, ih, iw, ic)).astype(np.int8)
    w = rng.integers(-128, 128, (k, k, ic, 1) if depthwise else (oc, k, k, ic)).astype(np.int8)
    bias = rng.integers(-2000, 2000, oc).astype(np.int32)
    mult = rng.integers(1 << 30, 1 << 31, oc).astype(np.int32)
    shift = (rng.integers(33, 41, oc) if shifts == "per channel" else np.full(oc, 36)).astype(np.int8)
    pad, stride = (p, p, p, p), (s, s)
    oh = (ih + 2 * p - k) // s + 1
    assert (ih + 2 * p - k) % s == 0
    conv = oracle.depthwise_conv2d if depthwise else oracle.conv2d
    acc = conv("i8", x, w, bias, pad, stride, (1, 1), in_zp=-5, w_zp=0)
    assert acc.shape[1] == oh and (acc < 0).mean() > 0.2 and (acc > 0).mean() > 0.2
    ctx.set_kernel_choice(choice)
    try:
        # (output_zp, CLAMP): the type's minimum without a CLAMP; a CLAMP from output_zp; from above it; from one below it
        zmin = int(np.iinfo(out_dtype).min)
        cases = [(-128, None), (-20, (-20, 100)), (7, (30, 127)), (7, (6, 127))] if out_dtype == np.int8 else \
                [(0, (0, 30000)), (0, (100, 20000)), (0, (-1, 30000))]
        for out_zp, clamp in cases:
            for mode in (capi.ROUND_DOUBLE, capi.ROUND_SINGLE):
                want, wst = oracle.rescale(acc, mult, shift, out_zp=out_zp, out_dtype=out_dtype, rounding_mode=mode)
                if clamp is not None:
                    want = oracle.clamp(want, *clamp)
                got, st = gpu_ops.conv2d(ctx, x, w, bias, pad, stride, (1, 1), in_zp=-5, w_zp=0, depthwise=depthwise, clamp=clamp,
                                         rescale=dict(mult=mult, shift=shift, out_zp=out_zp, out_dtype=out_dtype, rounding_mode=mode))
                assert ctx.last_kernel == kernel
                assert st == wst == capi.VALID
                assert np.array_equal(got, want), (out_zp, clamp, mode, int(np.count_nonzero(got != want)))
                lowest = zmin if clamp is None else clamp[0]
                assert (got == lowest).mean() > 0.1 and len(np.unique(got)) > 20
    finally:
        ctx.set_kernel_choice(capi.KERNEL_AUTO)


def test_a_negative_multiplier_is_still_reported(ctx):
    """A negative multiplier fails apply_scale_32's REQUIRE (quant_util.h:48-52); the form without the sign test is not taken
    for such a tile (its argument needs multipliers >= 0), and the status says UNPREDICTABLE as the oracle's does."""
    rng = np.random.default_rng(99)
    n, hw, ic, oc = 2, 14, 32, 40
    x = rng.integers(-128, 128, (n, hw, hw, ic)).astype(np.int8)
    w = rng.integers(-128, 128, (oc, 1, 1, ic)).astype(np.int8)
    bias = rng.integers(-2000, 2000, oc).astype(np.int32)
    mult = rng.integers(1 << 30, 1 << 31, oc).astype(np.int64)
    mult[::3] = -mult[::3]
    mult = mult.astype(np.int32)
    shift = rng.integers(33, 41, oc).astype(np.int8)
    acc = oracle.conv2d("i8", x, w, bias, in_zp=-5, w_zp=0)
    want, wst = oracle.rescale(acc, mult, shift, out_zp=-128, out_dtype=np.int8, rounding_mode=capi.ROUND_DOUBLE)
    got, st = gpu_ops.conv2d(ctx, x, w, bias, in_zp=-5, w_zp=0,
                             rescale=dict(mult=mult, shift=shift, out_zp=-128, out_dtype=np.int8, rounding_mode=capi.ROUND_DOUBLE))
    assert wst == capi.UNPREDICTABLE and st == wst
