"""Attributes of the operator interface that change what is computed or reported, through the C ABI on the device:
`local_bound` of the bounds pass, the accumulator type in the convolution descriptors, the TOSA level checks and
the floating-point CLAMP with its NaN mode - each against the oracle."""
import numpy as np
import pytest

import cases
import gpu_ops
import oracle
from reference_model_amd import Context, TmiError, capi
from test_gpu_compliance_passes import narrow

pytestmark = pytest.mark.gpu


@pytest.fixture()
def ctx():
    c = Context(0)
    yield c
    c.close()


# ---- bounds pass without local_bound (tensor_ops.cpp:790-802, 1245-1257) ----------------------------------------
@pytest.mark.parametrize("kind", ["fp16", "bf16", "fp32"])
@pytest.mark.parametrize("geom", [((1, 1, 1, 1), (1, 1), (1, 1)), ((2, 0, 1, 2), (2, 1), (1, 2)), ((0, 0, 0, 0), (1, 1), (1, 1))])
def test_conv2d_bounds_without_local_bound_uses_the_largest_input_magnitude(ctx, kind, geom):
    pad, stride, dil = geom
    rng = np.random.default_rng(41)
    n, ih, iw, ic, oc, kh, kw = 2, 10, 9, 12, 7, 3, 3
    while (ih - 1 + pad[0] + pad[1] - (kh - 1) * dil[0]) % stride[0]:
        ih += 1
    while (iw - 1 + pad[2] + pad[3] - (kw - 1) * dil[1]) % stride[1]:
        iw += 1
    xs, xf, dtype = narrow(rng.normal(0, 1, (n, ih, iw, ic)).astype(np.float32), kind)
    ws, wf, _ = narrow(rng.normal(0, 1, (oc, kh, kw, ic)).astype(np.float32), kind)
    bs, bf, _ = narrow(rng.normal(0, 1, oc).astype(np.float32), kind)
    oh, ow = oracle.conv_out_hw(ih, iw, kh, kw, pad, stride, dil)
    d = ctx.conv_desc(dtype, dtype, xs.shape, oc, kh, kw, (oh, ow), pad, stride, dil, oc)
    tx, tw, tb = ctx.upload(xs, dtype), ctx.upload(ws, dtype), ctx.upload(bs, dtype)
    out = ctx.empty((n, oh, ow, oc), capi.F64)
    ctx.conv2d_precise(d, tx, tw, tb, True, out, local_bound=False)
    assert ctx.sync() == capi.VALID
    flat = out.numpy().copy()
    assert np.array_equal(flat, oracle.conv2d("f64", xf, wf, bf, pad, stride, dil, abs_mode=True, local_bound=False))
    # the attribute only matters in the bounds pass, and the next call starts from a fresh maximum
    ctx.conv2d_precise(d, tx, tw, tb, False, out, local_bound=False)
    assert ctx.sync() == capi.VALID
    assert np.array_equal(out.numpy(), oracle.conv2d("f64", xf, wf, bf, pad, stride, dil))
    x2s, x2f, _ = narrow((0.5 * rng.normal(0, 1, (n, ih, iw, ic))).astype(np.float32), kind)
    ctx.conv2d_precise(d, ctx.upload(x2s, dtype), tw, tb, True, out, local_bound=False)
    assert ctx.sync() == capi.VALID
    assert np.array_equal(out.numpy(), oracle.conv2d("f64", x2f, wf, bf, pad, stride, dil, abs_mode=True,
                                                     local_bound=False))
    ctx.conv2d_precise(d, tx, tw, tb, True, out, local_bound=True)
    assert ctx.sync() == capi.VALID
    local = out.numpy()
    assert np.array_equal(local, oracle.conv2d("f64", xf, wf, bf, pad, stride, dil, abs_mode=True))
    assert np.all(flat >= local) and not np.array_equal(flat, local)


@pytest.mark.parametrize("kind", ["fp16", "bf16", "fp32"])
def test_depthwise_bounds_without_local_bound(ctx, kind):
    rng = np.random.default_rng(43)
    n, ih, iw, c, m, kh, kw = 2, 9, 7, 12, 2, 3, 3
    xs, xf, dtype = narrow(rng.normal(0, 1, (n, ih, iw, c)).astype(np.float32), kind)
    ws, wf, _ = narrow(rng.normal(0, 1, (kh, kw, c, m)).astype(np.float32), kind)
    bs, bf, _ = narrow(rng.normal(0, 1, c * m).astype(np.float32), kind)
    pad, stride, dil = (1, 1, 1, 1), (2, 2), (1, 1)
    oh, ow = oracle.conv_out_hw(ih, iw, kh, kw, pad, stride, dil)
    d = ctx.conv_desc(dtype, dtype, xs.shape, c * m, kh, kw, (oh, ow), pad, stride, dil, c * m)
    out = ctx.empty((n, oh, ow, c * m), capi.F64)
    ctx.conv2d_precise(d, ctx.upload(xs, dtype), ctx.upload(ws, dtype), ctx.upload(bs, dtype), True, out,
                       depthwise=True, local_bound=False)
    assert ctx.sync() == capi.VALID
    assert np.array_equal(out.numpy(), oracle.depthwise_conv2d("f64", xf, wf, bf, pad, stride, dil, abs_mode=True,
                                                               local_bound=False))


# ---- accumulator type (op_factory.h:97-118; instantiations tensor_ops.cpp:2219-2251) ------------------------------
def test_accumulator_types_that_are_not_built_are_refused(ctx):
    rng = np.random.default_rng(3)
    x = rng.normal(0, 1, (1, 6, 6, 8)).astype(np.float16)
    w = rng.normal(0, 1, (8, 3, 3, 8)).astype(np.float16)
    b = np.zeros(8, np.float16)
    tx, tw, tb = ctx.upload(x), ctx.upload(w), ctx.upload(b)
    out = ctx.empty((1, 4, 4, 8), capi.FP16)
    good = ctx.conv_desc(capi.FP16, capi.FP16, x.shape, 8, 3, 3, (4, 4), (0, 0, 0, 0), (1, 1), (1, 1), 8)
    assert good.acc_dtype == capi.FP32
    ctx.conv2d(good, tx, tw, tb, 0, 0, out)
    assert ctx.sync() == capi.VALID
    want = out.numpy().copy()
    # fp16 inputs with an fp16 accumulator are a legal TOSA combination this library does not implement: an error,
    # never a silently wider accumulation
    bad = ctx.conv_desc(capi.FP16, capi.FP16, x.shape, 8, 3, 3, (4, 4), (0, 0, 0, 0), (1, 1), (1, 1), 8, acc_dtype=capi.FP16)
    with pytest.raises(TmiError, match="accumulator"):
        ctx.conv2d(bad, tx, tw, tb, 0, 0, out)
    assert np.array_equal(out.numpy(), want)
    with pytest.raises(TmiError, match="accumulator"):
        ctx.conv2d_precise(bad, tx, tw, tb, False, ctx.empty((1, 4, 4, 8), capi.F64))
    xi = rng.integers(-128, 128, (1, 6, 6, 8), dtype=np.int8)
    wi = rng.integers(-128, 128, (8, 3, 3, 8), dtype=np.int8)
    bi = np.zeros(8, np.int32)
    bad_i = ctx.conv_desc(capi.INT8, capi.INT32, xi.shape, 8, 3, 3, (4, 4), (0, 0, 0, 0), (1, 1), (1, 1), 8, acc_dtype=capi.FP32)
    with pytest.raises(TmiError, match="accumulator"):
        ctx.conv2d(bad_i, ctx.upload(xi), ctx.upload(wi), ctx.upload(bi), 0, 0, ctx.empty((1, 4, 4, 8), capi.INT32))

    # a descriptor zeroed by a caller that predates the field: 0 stands for the operand type's accumulator
    zeroed = ctx.conv_desc(capi.INT8, capi.INT32, xi.shape, 8, 3, 3, (4, 4), (0, 0, 0, 0), (1, 1), (1, 1), 8, acc_dtype=0)
    assert zeroed.acc_dtype == 0
    oi = ctx.empty((1, 4, 4, 8), capi.INT32)
    ctx.conv2d(zeroed, ctx.upload(xi), ctx.upload(wi), ctx.upload(bi), 0, 0, oi)
    assert ctx.sync() == capi.VALID and np.array_equal(oi.numpy(), oracle.conv2d("i8", xi, wi, bi))

    td = capi.TconvDesc()
    td.in_dtype, td.out_dtype = capi.INT8, capi.INT32
    assert td.acc_dtype == capi.INT32
    td.N, td.IH, td.IW, td.IC, td.OC, td.KH, td.KW, td.OH, td.OW = 1, 6, 6, 8, 8, 3, 3, 8, 8
    td.stride[:] = [1, 1]
    td.bias_len = 8
    to = ctx.empty((1, 8, 8, 8), capi.INT32)
    ctx.transpose_conv2d(td, ctx.upload(xi), ctx.upload(wi), ctx.upload(bi), 0, 0, to)
    assert ctx.sync() == capi.VALID
    assert np.array_equal(to.numpy(), oracle.transpose_conv2d("i8", xi, wi, bi))
    td.acc_dtype = capi.FP16
    with pytest.raises(TmiError, match="accumulator"):
        ctx.transpose_conv2d(td, ctx.upload(xi), ctx.upload(wi), ctx.upload(bi), 0, 0, to)

    cd = capi.Conv3dDesc()
    cd.in_dtype, cd.out_dtype = capi.INT8, capi.INT32
    cd.N, cd.ID, cd.IH, cd.IW, cd.IC, cd.OC, cd.KD, cd.KH, cd.KW, cd.OD, cd.OH, cd.OW = 1, 3, 6, 6, 8, 8, 2, 3, 3, 2, 4, 4
    cd.stride[:] = [1, 1, 1]
    cd.dilation[:] = [1, 1, 1]
    cd.bias_len = 8
    x3 = rng.integers(-128, 128, (1, 3, 6, 6, 8), dtype=np.int8)
    w3 = rng.integers(-128, 128, (8, 2, 3, 3, 8), dtype=np.int8)
    o3 = ctx.empty((1, 2, 4, 4, 8), capi.INT32)
    ctx.conv3d(cd, ctx.upload(x3), ctx.upload(w3), ctx.upload(bi), 0, 0, o3)
    assert ctx.sync() == capi.VALID
    assert np.array_equal(o3.numpy(), oracle.conv3d("i8", x3, w3, bi))
    cd.acc_dtype = capi.FP32
    with pytest.raises(TmiError, match="accumulator"):
        ctx.conv3d(cd, ctx.upload(x3), ctx.upload(w3), ctx.upload(bi), 0, 0, o3)


# ---- TOSA level (func_debug.h:132-141; EIGHTK in func_config.h) ---------------------------------------------------
def test_level_checks_latch_unpredictable_and_leave_the_result_alone(ctx):
    rng = np.random.default_rng(5)
    x = rng.integers(-128, 128, (1, 4, 3, 8), dtype=np.int8)
    w = rng.integers(-128, 128, (8, 1, 1, 8), dtype=np.int8)
    b = rng.integers(-1000, 1000, 8, dtype=np.int32)
    pad = (8193, 0, 0, 0)                                   # pad_top > MAX_KERNEL (tensor_ops.cpp:766)
    want = oracle.conv2d("i8", x, w, b, pad, in_zp=3)
    out, st = gpu_ops.conv2d(ctx, x, w, b, pad, in_zp=3)
    assert st == capi.VALID and np.array_equal(out, want)
    ctx.set_level(capi.LEVEL_EIGHTK)
    out, st = gpu_ops.conv2d(ctx, x, w, b, pad, in_zp=3)
    assert st == capi.UNPREDICTABLE and ctx.flags == capi.FLAG_LEVEL and np.array_equal(out, want)
    out, st = gpu_ops.conv2d(ctx, x, w, b, (1, 1, 1, 1), in_zp=3)          # the latch is per sync
    assert st == capi.VALID and ctx.flags == 0
    # stride beyond MAX_STRIDE (:770): the output is one pixel
    xs = rng.integers(-128, 128, (1, 4, 1, 8), dtype=np.int8)
    out, st = gpu_ops.conv2d(ctx, xs, w, b, stride=(1, 8193))
    assert st == capi.UNPREDICTABLE and np.array_equal(out, oracle.conv2d("i8", xs, w, b, stride=(1, 8193)))
    # depthwise, pooling and the two re-laid-out convolutions carry their own checks
    wd = rng.integers(-128, 128, (1, 1, 8, 1), dtype=np.int8)
    out, st = gpu_ops.conv2d(ctx, x, wd, b, pad, depthwise=True)
    assert st == capi.UNPREDICTABLE and np.array_equal(out, oracle.depthwise_conv2d("i8", x, wd, b, pad))
    xp = rng.integers(-128, 128, (1, 4, 2, 8), dtype=np.int8)
    out, st = gpu_ops.pool2d(ctx, xp, (1, 2), stride=(1, 8193), avg=False)
    assert st == capi.UNPREDICTABLE and np.array_equal(out, oracle.max_pool2d(xp, (1, 2), (1, 8193)))
    out, st = gpu_ops.transpose_conv2d(ctx, x, w, b, stride=(8193, 1))
    assert st == capi.UNPREDICTABLE and np.array_equal(out, oracle.transpose_conv2d("i8", x, w, b, stride=(8193, 1)))
    # inside the level nothing is flagged; without a level nothing is checked
    out, st = gpu_ops.conv2d(ctx, x, w, b, (8192, 0, 0, 0))
    assert st == capi.VALID
    ctx.set_level(capi.LEVEL_NONE)
    out, st = gpu_ops.conv2d(ctx, x, w, b, pad, in_zp=3)
    assert st == capi.VALID and np.array_equal(out, want)


# ---- floating-point CLAMP (activation_funcs.cpp:97-106, applyClip arith_util.h:390-413) ---------------------------
SPECIALS = np.array([np.nan, -np.nan, np.inf, -np.inf, 0.0, -0.0, 1.5, -1.5, 65504.0, -65504.0, 6e-8, -6e-8], np.float32)


@pytest.mark.parametrize("kind", ["fp16", "bf16", "fp32"])
@pytest.mark.parametrize("nan_mode", [1, 2])
@pytest.mark.parametrize("lo,hi", [(-1.0, 1.0), (0.0, 6.0), (-0.0, 0.0), (-np.inf, np.inf), (2.0, 2.0)])
def test_floating_point_clamp_matches_the_oracle_bit_for_bit(ctx, kind, nan_mode, lo, hi):
    rng = np.random.default_rng(11)
    values = np.concatenate([SPECIALS, rng.normal(0, 2, 5000).astype(np.float32)])
    stored, as64, dtype = narrow(values, kind)
    out = ctx.empty(stored.shape, dtype, stored.dtype)
    ctx.clamp_fp(dtype, stored.size, ctx.upload(stored, dtype), lo, hi, nan_mode, out)
    assert ctx.sync() == capi.VALID
    want32 = oracle.clamp(as64.astype(np.float32), lo, hi, nan_mode)     # every storage value is exact in float32
    got = out.numpy()
    if kind == "bf16":
        got32 = cases.bf16_bits_to_float(got)
    else:
        got32 = got.astype(np.float32)
    nan = np.isnan(want32)
    assert np.array_equal(np.isnan(got32), nan)
    assert np.array_equal(got32[~nan].view(np.uint32), want32[~nan].view(np.uint32))      # signed zeros included
    assert nan.sum() == (2 if nan_mode == 1 else 0)


def test_floating_point_clamp_refuses_a_nan_or_inverted_range(ctx):
    x = ctx.upload(np.zeros(4, np.float32))
    out = ctx.empty((4,), capi.FP32)
    with pytest.raises(TmiError):
        ctx.clamp_fp(capi.FP32, 4, x, 1.0, 0.0, 1, out)
    with pytest.raises(TmiError):
        ctx.clamp_fp(capi.FP32, 4, x, float("nan"), 0.0, 1, out)
    with pytest.raises(TmiError):
        ctx.clamp_fp(capi.INT8, 4, x, 0.0, 1.0, 1, out)
    ctx.clamp_fp(capi.FP32, 0, None, 0.0, 1.0, 1, None)               # an empty tensor is a no-op


@pytest.mark.parametrize("mode", [(False, False, False), (True, False, False), (True, True, False), (True, True, True)],
                         ids=["fp32", "precise", "compliance", "compliance-bounds"])
@pytest.mark.parametrize("in_dtype,out_dtype,out_zp", [(np.int8, np.int8, -100), (np.int32, np.int16, 0), (np.int16, np.int32, 0)])
def test_inexact_round_in_precise_mode_matches_the_oracle(ctx, mode, in_dtype, out_dtype, out_zp):
    """INEXACT_ROUND as the reference evaluates it in precise mode (type_conversion.cpp:326-346): FP64 maths truncated,
    and under compliance mode the lower (normal pass) or upper (bounds pass) edge of the error bound"""
    precise, compliance, bounds = mode
    oracle_mode = 0 if not precise else (1 if not compliance else (3 if bounds else 2))
    rng = np.random.default_rng(oracle_mode + 10 * np.dtype(in_dtype).itemsize)
    info = np.iinfo(in_dtype)
    x = rng.integers(max(info.min, -(1 << 24)), min(info.max, 1 << 24), (37, 24)).astype(in_dtype)
    # scales that leave most results inside the output range, so that the rounding is what decides them
    mult = rng.integers(1 << 29 if in_dtype == np.int8 else 1 << 20, 1 << 31, 24).astype(np.int32)
    shift = (rng.integers(30, 34, 24) if in_dtype == np.int8 else rng.integers(28 if in_dtype == np.int32 else 20, 45, 24)).astype(np.int8)
    mult[0], shift[0] = 1 << 30, 31    # halves: the ties are where the edges of the compliance bound leave rint()
    in_zp = 5 if in_dtype == np.int8 else 0
    kw = dict(in_zp=in_zp, out_zp=out_zp, out_dtype=out_dtype, rounding_mode=capi.ROUND_INEXACT)
    want, wst = oracle.rescale(x, mult, shift, inexact_mode=oracle_mode, **kw)
    ctx.set_precise_mode(precise, compliance, bounds)
    try:
        got, st = gpu_ops.rescale(ctx, x, mult, shift, **kw)
    finally:
        ctx.set_precise_mode()
    assert st == wst == capi.VALID and np.array_equal(got, want), int(np.count_nonzero(got != want))
    if precise and (not compliance or in_dtype == np.int8):    # differs from FP32 maths, or the setting did not arrive
        plain, _ = oracle.rescale(x, mult, shift, **kw)
        assert not np.array_equal(plain, want)


@pytest.mark.parametrize("depthwise", [False, True])
@pytest.mark.parametrize("mode", [(True, False, False), (True, True, True)])
def test_fused_rescale_with_inexact_round_in_precise_mode(ctx, depthwise, mode):
    """the fused entry points under precise mode: the convolution's INT32 results are converted by the stand-alone
    RESCALE kernel in FP64 (type_conversion.cpp:326-346), as the reference's two operators in a row would"""
    precise, compliance, bounds = mode
    oracle_mode = 1 if not compliance else (3 if bounds else 2)
    rng = np.random.default_rng(91 + oracle_mode + depthwise)
    c = 16
    x = rng.integers(-128, 128, (2, 9, 11, c), dtype=np.int8)
    w = rng.integers(-128, 128, (3, 3, c, 1) if depthwise else (24, 3, 3, c), dtype=np.int8)
    oc = c if depthwise else 24
    bias = rng.integers(-2000, 2000, oc).astype(np.int32)
    mult = rng.integers(1 << 30, 1 << 31, oc).astype(np.int32)
    shift = rng.integers(38 if depthwise else 42, 46, oc).astype(np.int8)
    kw = dict(pad=(1, 1, 1, 1), in_zp=-3, w_zp=0)
    acc = (oracle.depthwise_conv2d if depthwise else oracle.conv2d)("i8", x, w, bias, **kw)
    want, wst = oracle.rescale(acc, mult, shift, out_zp=4, out_dtype=np.int8, rounding_mode=capi.ROUND_INEXACT,
                               inexact_mode=oracle_mode)
    ctx.set_precise_mode(precise, compliance, bounds)
    try:
        got, st = gpu_ops.conv2d(ctx, x, w, bias, depthwise=depthwise, **kw,
                                 rescale=dict(mult=mult, shift=shift, out_zp=4, rounding_mode=capi.ROUND_INEXACT))
    finally:
        ctx.set_precise_mode()
    assert ctx.last_kernel in ("rescale_vec_precise", "rescale_scalar_precise")
    assert wst == st == capi.VALID and np.array_equal(got, want), int(np.count_nonzero(got != want))
    assert len(np.unique(want)) > 20    # not clipped away

