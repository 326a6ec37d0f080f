"""The floating-point compliance passes on the device: precise mode (fp64) and bounds mode (sums of absolute
values) of CONV2D / DEPTHWISE_CONV2D / MATMUL against the fp64 oracle, the DOT_PRODUCT check as a device
reduction against its numpy restatement, and the whole flow - fast kernel, precise pass, bounds pass, check -
at the full size of the fp16 / bf16 benchmark configurations on the specification's data sets S0..S5."""
import numpy as np
import pytest

import cases
import dot_product_check as dp
import oracle
from reference_model_amd import Context, capi

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def ctx():
    c = Context(0)
    yield c
    c.close()


def narrow(values, kind):
    """float32 values -> (array as it travels to the device, the same values in fp64, TMI dtype)"""
    if kind == "fp16":
        with np.errstate(over="ignore"):     # set 1 puts a bias beyond the fp16 range: it becomes infinity, as
            h = values.astype(np.float16)    # in the reference's generator, and the check's overflow rule applies
        return h, h.astype(np.float64), capi.FP16
    if kind == "fp32":
        return values, values.astype(np.float64), capi.FP32
    b = cases.float_to_bf16_bits(values)
    return b, cases.bf16_bits_to_float(b).astype(np.float64), capi.BF16


def as_f64(t, kind):
    a = t.numpy()
    return a.astype(np.float64) if kind in ("fp16", "fp32") else cases.bf16_bits_to_float(a).astype(np.float64)


CONV_CASES = [  # n, ih, iw, ic, oc, kh, kw, pad, stride, dilation
    (2, 9, 8, 16, 24, 3, 3, (1, 1, 1, 1), (1, 1), (1, 1)),
    (1, 12, 11, 8, 5, 3, 2, (2, 1, 0, 1), (2, 1), (1, 2)),
    (3, 5, 5, 40, 16, 1, 1, (0, 0, 0, 0), (1, 1), (1, 1)),
]


@pytest.mark.parametrize("shape", CONV_CASES)
@pytest.mark.parametrize("kind", ["fp16", "bf16", "fp32"])
@pytest.mark.parametrize("bounds", [False, True])
def test_conv2d_precise_and_bounds_match_the_fp64_oracle(ctx, shape, kind, bounds):
    n, ih, iw, ic, oc, kh, kw, pad, stride, dil = shape
    rng = np.random.default_rng(ih * iw + oc)
    xs, xf, dtype = narrow(rng.normal(0, 1, (n, ih, iw, ic)).astype(np.float32), kind)
    ws, wf, _ = narrow(rng.normal(0, 1, (oc, kh, kw, ic)).astype(np.float32), kind)
    bs, bf, _ = narrow(rng.normal(0, 1, oc).astype(np.float32), kind)
    oh, ow = oracle.conv_out_hw(ih, iw, kh, kw, pad, stride, dil)
    d = ctx.conv_desc(dtype, dtype, xs.shape, oc, kh, kw, (oh, ow), pad, stride, dil, oc)
    out = ctx.empty((n, oh, ow, oc), capi.F64)
    ctx.conv2d_precise(d, ctx.upload(xs, dtype), ctx.upload(ws, dtype), ctx.upload(bs, dtype), bounds, out)
    assert ctx.sync() == capi.VALID
    want = oracle.conv2d("f64", xf, wf, bf, pad, stride, dil, abs_mode=bounds)
    # same products, same order of fp64 additions, bias last: the same fp64 numbers
    assert np.array_equal(out.numpy(), want)


@pytest.mark.parametrize("kind", ["fp16", "bf16", "fp32"])
@pytest.mark.parametrize("bounds", [False, True])
def test_depthwise_and_matmul_precise_match_the_fp64_oracle(ctx, kind, bounds):
    rng = np.random.default_rng(17)
    n, ih, iw, c, m, kh, kw = 2, 9, 7, 12, 2, 3, 3
    xs, xf, dtype = narrow(rng.normal(0, 1, (n, ih, iw, c)).astype(np.float32), kind)
    ws, wf, _ = narrow(rng.normal(0, 1, (kh, kw, c, m)).astype(np.float32), kind)
    bs, bf, _ = narrow(rng.normal(0, 1, c * m).astype(np.float32), kind)
    pad, stride, dil = (1, 1, 1, 1), (2, 2), (1, 1)
    oh, ow = oracle.conv_out_hw(ih, iw, kh, kw, pad, stride, dil)
    d = ctx.conv_desc(dtype, dtype, xs.shape, c * m, kh, kw, (oh, ow), pad, stride, dil, c * m)
    out = ctx.empty((n, oh, ow, c * m), capi.F64)
    ctx.conv2d_precise(d, ctx.upload(xs, dtype), ctx.upload(ws, dtype), ctx.upload(bs, dtype), bounds, out, depthwise=True)
    assert ctx.sync() == capi.VALID
    assert np.array_equal(out.numpy(), oracle.depthwise_conv2d("f64", xf, wf, bf, pad, stride, dil, abs_mode=bounds))

    a_s, af, _ = narrow(rng.normal(0, 1, (3, 17, 96)).astype(np.float32), kind)
    b_s, bf2, _ = narrow(rng.normal(0, 1, (3, 96, 29)).astype(np.float32), kind)
    out = ctx.empty((3, 17, 29), capi.F64)
    ctx.matmul_precise(dtype, 3, 17, 96, 29, ctx.upload(a_s, dtype), ctx.upload(b_s, dtype), bounds, out)
    assert ctx.sync() == capi.VALID
    assert np.array_equal(out.numpy(), oracle.matmul("f64", af, bf2, abs_mode=bounds))


@pytest.mark.parametrize("kind", ["fp16", "bf16", "fp32"])
def test_device_dot_product_check_matches_its_numpy_restatement(ctx, kind):
    rng = np.random.default_rng(5)
    n, ksb = 100_000, 9
    ref = rng.normal(0, 3, n)
    bnd = np.abs(ref) + np.abs(rng.normal(0, 3, n))
    frac = dp.NORMAL_FRAC[kind]
    noise = rng.normal(0, 0.7, n) * bnd * 2.0 ** (-1 - frac)
    imp64 = ref + noise
    bnd[:50], ref[:50], imp64[:50] = 0.0, 0.0, 0.0            # all-zero products
    if kind == "fp16":
        imp = imp64.astype(np.float16)
    elif kind == "bf16":
        imp = cases.float_to_bf16_bits(imp64.astype(np.float32))
    else:
        imp = imp64.astype(np.float32)
    dtype = {"fp16": capi.FP16, "bf16": capi.BF16, "fp32": capi.FP32}[kind]
    impf = imp.astype(np.float64) if kind != "bf16" else cases.bf16_bits_to_float(imp).astype(np.float64)
    want = dp.check(impf, ref, bnd, kind, ksb)
    r = ctx.dot_product_check(dtype, n, ctx.upload(imp, dtype), ctx.upload(ref, capi.F64), ctx.upload(bnd, capi.F64), ksb)
    assert r.elements == n and r.abs_bound == 2 * ksb and r.variance_bound == pytest.approx(1.6 * ksb)
    assert r.max_abs_err == pytest.approx(want["max_err"], rel=1e-12)
    assert r.err_sumsq == pytest.approx(want["err_sumsq"], rel=1e-9)
    assert bool(r.compliant) == want["ok"] and r.failed_elements == 0
    # an element far outside its bound, a non-zero result under a zero bound, a missed NaN
    bad = impf.copy()
    bad[1000] += 1000 * bnd[1000]
    bad[10] = 1.0
    ref2 = ref.copy()
    ref2[2000] = np.nan
    bad_dev = bad.astype(np.float16) if kind == "fp16" else (cases.float_to_bf16_bits(bad.astype(np.float32)) if kind == "bf16"
                                                                else bad.astype(np.float32))
    r = ctx.dot_product_check(dtype, n, ctx.upload(bad_dev, dtype), ctx.upload(ref2, capi.F64), ctx.upload(bnd, capi.F64), ksb)
    assert r.failed_elements == 3 and not r.compliant


@pytest.mark.parametrize("kind", ["fp16", "bf16", "fp32"])
def test_device_dot_product_check_branches(ctx, kind):
    """every branch of validateElement / validateDataDP (verify_dot_product.cpp:34-87, 127-139): a NaN reference met
    and missed, a NaN bound, a bound at which the sum may overflow the output type, and the error-sum rule that only
    the data sets 3..5 carry"""
    rng = np.random.default_rng(11)
    n, ksb = 4096, 5
    frac = dp.NORMAL_FRAC[kind]
    big = {"fp16": 65000.0, "bf16": 3.3e38, "fp32": 3.3e38}[kind]      # bnd * (1 + abs_bound * 2^-(1+frac)) overflows
    dtype = {"fp16": capi.FP16, "bf16": capi.BF16, "fp32": capi.FP32}[kind]

    def to_dev(a64):
        if kind == "fp16":
            return a64.astype(np.float16)
        if kind == "bf16":
            return cases.float_to_bf16_bits(a64.astype(np.float32))
        return a64.astype(np.float32)

    def back(a):
        return cases.bf16_bits_to_float(a).astype(np.float64) if kind == "bf16" else a.astype(np.float64)

    ref = rng.normal(0, 2, n)
    bnd = np.abs(ref) + 1.0
    imp64 = ref + 0.3 * bnd * 2.0 ** (-1 - frac)          # every error +0.3 units: a bias, well inside abs_bound
    ref[5], imp64[5] = np.nan, np.nan                     # NaN reference, matched
    bnd[6] = np.nan                                       # NaN bound: anything goes
    imp64[6] = 12345.0
    with np.errstate(over="ignore"):
        bnd[7] = big                                      # may overflow: anything goes
        imp64[7] = -1.0
    imp = to_dev(imp64)
    for set_number in (-1, 0, 3, 5):
        want = dp.check(back(imp), ref, bnd, kind, ksb, set_number)
        r = ctx.dot_product_check(dtype, n, ctx.upload(imp, dtype), ctx.upload(ref, capi.F64), ctx.upload(bnd, capi.F64), ksb,
                                  set_number)
        assert r.failed_elements == want["failed_elements"] == 0
        assert r.err_sum == pytest.approx(want["err_sum"], rel=1e-9)
        assert r.err_sumsq == pytest.approx(want["err_sumsq"], rel=1e-9)
        assert bool(r.compliant) == want["ok"]
        # 4093 errors of about +0.3 (fp16 / bf16 round them to multiples of a unit): the sum is beyond
        # sqrt(10 * 1.6 ksb * T) = 572, which only sets 3..5 hold against
        assert want["ok"] == (set_number not in (3, 5)) and abs(want["err_sum"]) > 600
    # the NaN reference missed
    imp2 = back(imp).copy()
    imp2[5] = 0.0
    want = dp.check(imp2, ref, bnd, kind, ksb)
    r = ctx.dot_product_check(dtype, n, ctx.upload(to_dev(imp2), dtype), ctx.upload(ref, capi.F64), ctx.upload(bnd, capi.F64), ksb)
    assert r.failed_elements == want["failed_elements"] == 1 and not r.compliant and not want["ok"]


@pytest.mark.parametrize("data_set", range(6))
def test_config5_bf16_matmul_compliance_on_the_device(ctx, data_set):
    """[4,2048,4096] x [4,4096,2048] bf16 -> fp32 on the specification's data set, every pass on the GPU:
    the GEMM kernel, the fp64 precise pass, the bounds pass and the DOT_PRODUCT check with ksb = C."""
    n, h, c, w = 4, 2048, 4096, 2048
    a_s, _, dtype = narrow(oracle.dot_product_data("matmul", data_set, 0, c, (n, h, c), kind="bf16"), "bf16")
    b_s, _, _ = narrow(oracle.dot_product_data("matmul", data_set, 1, c, (n, c, w), kind="bf16"), "bf16")
    ta, tb = ctx.upload(a_s, dtype), ctx.upload(b_s, dtype)
    imp, ref, bnd = ctx.empty((n, h, w), capi.FP32), ctx.empty((n, h, w), capi.F64), ctx.empty((n, h, w), capi.F64)
    try:
        ctx.matmul(dtype, n, h, c, w, ta, tb, 0, 0, imp)
        assert ctx.last_kernel == "matmul_gemm_bf16"
        ctx.matmul_precise(dtype, n, h, c, w, ta, tb, False, ref)
        ctx.matmul_precise(dtype, n, h, c, w, ta, tb, True, bnd)
        r = ctx.dot_product_check(capi.FP32, n * h * w, imp, ref, bnd, dp.kernel_size_bound(c, "fp32", has_bias=False), data_set)
        assert r.compliant and r.failed_elements == 0, (r.max_abs_err, r.err_sum, r.err_sumsq)
    finally:
        for t in list(ctx._owned):
            ctx._free(t)


@pytest.mark.parametrize("data_set", range(6))
def test_config5_fp16_conv_compliance_on_the_device(ctx, data_set):
    """fp16 CONV2D 3x3 [16,28,28,256] -> 256 (fp32 accumulate, fp16 result) on the specification's data set."""
    n, hw, ic, oc = 16, 28, 256, 256
    ks = 9 * ic
    xs, _, dtype = narrow(oracle.dot_product_data("conv2d", data_set, 0, ks, (n, hw, hw, ic), kind="fp16", kernel=(3, 3)), "fp16")
    ws, _, _ = narrow(oracle.dot_product_data("conv2d", data_set, 1, ks, (oc, 3, 3, ic), kind="fp16"), "fp16")
    bs, _, _ = narrow(oracle.dot_product_data("conv2d", data_set, 2, ks, (oc,), kind="fp16"), "fp16")
    d = ctx.conv_desc(dtype, dtype, xs.shape, oc, 3, 3, (hw, hw), (1, 1, 1, 1), (1, 1), (1, 1), oc)
    tx, tw, tb = ctx.upload(xs, dtype), ctx.upload(ws, dtype), ctx.upload(bs, dtype)
    shape = (n, hw, hw, oc)
    imp, ref, bnd = ctx.empty(shape, capi.FP16), ctx.empty(shape, capi.F64), ctx.empty(shape, capi.F64)
    try:
        ctx.conv2d(d, tx, tw, tb, 0, 0, imp)
        ctx.conv2d_precise(d, tx, tw, tb, False, ref)
        ctx.conv2d_precise(d, tx, tw, tb, True, bnd)
        r = ctx.dot_product_check(capi.FP16, int(np.prod(shape)), imp, ref, bnd, dp.kernel_size_bound(ks, "fp16"), data_set)
        assert r.compliant and r.failed_elements == 0, (r.max_abs_err, r.err_sum, r.err_sumsq)
    finally:
        for t in list(ctx._owned):
            ctx._free(t)


@pytest.mark.parametrize("data_set", range(6))
def test_fp32_conv_and_matmul_compliance_on_the_device(ctx, data_set):
    """FP32 operators (fp32 accumulation in the reference's order) on the specification's data sets, whose fp32
    generator output is pinned bit for bit by the reference's goldens: implementation, fp64 precise pass, bounds
    pass and DOT_PRODUCT check (ksb = KS + 1 with a bias, fp32 accumulator and result) on the GPU."""
    n, hw, ic, oc = 2, 14, 48, 24
    ks = 9 * ic
    xs = oracle.dot_product_data("conv2d", data_set, 0, ks, (n, hw, hw, ic), kind="fp32", kernel=(3, 3))
    ws = oracle.dot_product_data("conv2d", data_set, 1, ks, (oc, 3, 3, ic), kind="fp32")
    bs = oracle.dot_product_data("conv2d", data_set, 2, ks, (oc,), kind="fp32")
    d = ctx.conv_desc(capi.FP32, capi.FP32, xs.shape, oc, 3, 3, (hw, hw), (1, 1, 1, 1), (1, 1), (1, 1), oc)
    shape = (n, hw, hw, oc)
    try:
        tx, tw, tb = ctx.upload(xs, capi.FP32), ctx.upload(ws, capi.FP32), ctx.upload(bs, capi.FP32)
        imp, ref, bnd = ctx.empty(shape, capi.FP32), ctx.empty(shape, capi.F64), ctx.empty(shape, capi.F64)
        ctx.conv2d(d, tx, tw, tb, 0, 0, imp)
        assert ctx.last_kernel == "conv2d_direct_f32"
        ctx.conv2d_precise(d, tx, tw, tb, False, ref)
        ctx.conv2d_precise(d, tx, tw, tb, True, bnd)
        r = ctx.dot_product_check(capi.FP32, int(np.prod(shape)), imp, ref, bnd, dp.kernel_size_bound(ks, "fp32"), data_set)
        assert r.compliant and r.failed_elements == 0, (r.max_abs_err, r.err_sum, r.err_sumsq)
        assert np.array_equal(ref.numpy(), oracle.conv2d("f64", xs.astype(np.float64), ws.astype(np.float64),
                                                         bs.astype(np.float64), (1, 1, 1, 1), (1, 1), (1, 1)))
        nb, h, c, w = 2, 24, 200, 16
        a_s = oracle.dot_product_data("matmul", data_set, 0, c, (nb, h, c), kind="fp32")
        b_s = oracle.dot_product_data("matmul", data_set, 1, c, (nb, c, w), kind="fp32")
        ta, tb2 = ctx.upload(a_s, capi.FP32), ctx.upload(b_s, capi.FP32)
        imp, ref, bnd = ctx.empty((nb, h, w), capi.FP32), ctx.empty((nb, h, w), capi.F64), ctx.empty((nb, h, w), capi.F64)
        ctx.matmul(capi.FP32, nb, h, c, w, ta, tb2, 0, 0, imp)
        assert ctx.last_kernel == "matmul_direct_f32"
        ctx.matmul_precise(capi.FP32, nb, h, c, w, ta, tb2, False, ref)
        ctx.matmul_precise(capi.FP32, nb, h, c, w, ta, tb2, True, bnd)
        r = ctx.dot_product_check(capi.FP32, nb * h * w, imp, ref, bnd, dp.kernel_size_bound(c, "fp32", has_bias=False), data_set)
        assert r.compliant and r.failed_elements == 0, (r.max_abs_err, r.err_sum, r.err_sumsq)
    finally:
        for t in list(ctx._owned):
            ctx._free(t)


def test_benchmark_fp16_conv_and_bf16_matmul_errors_at_full_size(ctx):
    """The two floating-point benchmark configurations on the benchmark's own operands, at full size, against the
    library's fp64 pass over the same operands (itself bit-equal to the fp64 oracle on the small cases above):
    the DOT_PRODUCT check, the largest error in ULPs of the output type as the reference's ULP verifier defines
    the unit (verify_ulp.cpp:27-47), the largest relative error, and the largest error relative to the sum of the
    absolute products.  Measured on MI355X: fp16 CONV2D 14.7 ULP over all elements, 0.50 ULP where the result is
    at least an eighth of that sum (the rounding of the fp32 sum to fp16 and nothing else), 7.3e-5 of the sum; bf16
    MATMUL to fp32 3.8 ULP on those elements and 1.5e-7 of the sum (over all elements 2.3e8 ULP and a relative error of
    16: results of 1e-7 against a sum of absolute products of 50).  An element whose products
    cancel has an error of many ULPs of its small result whatever the accumulation order, so the asserted limits
    are on the well-conditioned elements and on the error relative to the sum, with headroom of about two."""
    c = cases.c5_conv()
    n, ih, iw, ic = c["x"].shape
    oc, kh, kw, _ = c["w"].shape
    d = ctx.conv_desc(capi.FP16, capi.FP16, c["x"].shape, oc, kh, kw, (ih, iw), c["pad"], c["stride"], c["dilation"], oc)
    try:
        tx, tw, tb = ctx.upload(c["x"], capi.FP16), ctx.upload(c["w"], capi.FP16), ctx.upload(c["bias"], capi.FP16)
        shape = (n, ih, iw, oc)
        imp, ref, bnd = ctx.empty(shape, capi.FP16), ctx.empty(shape, capi.F64), ctx.empty(shape, capi.F64)
        ctx.conv2d(d, tx, tw, tb, 0, 0, imp)
        assert ctx.last_kernel == "gemm_mfma_f16_patch"
        ctx.conv2d_precise(d, tx, tw, tb, False, ref)
        ctx.conv2d_precise(d, tx, tw, tb, True, bnd)
        ksb = dp.kernel_size_bound(kh * kw * ic, "fp16")
        r = ctx.dot_product_check(capi.FP16, int(np.prod(shape)), imp, ref, bnd, ksb)
        assert ctx.sync() == capi.VALID and r.compliant
        ref_h, bnd_h = ref.numpy(), bnd.numpy()
        # one whole image of the fp64 reference and of the bound against the oracle's own loop nest (its OpenMP build:
        # the same C source on all host cores), element for element: the reference the check above divides by is the
        # oracle's, not only the library's
        img = 11
        x64, w64, b64 = (c[k].astype(np.float64) for k in ("x", "w", "bias"))
        oracle.set_parallel(True)
        try:
            ref_o = oracle.conv2d("f64", x64[img:img + 1], w64, b64, c["pad"], c["stride"], c["dilation"])
            bnd_o = oracle.conv2d("f64", x64[img:img + 1], w64, b64, c["pad"], c["stride"], c["dilation"], abs_mode=True)
        finally:
            oracle.set_parallel(False)
        assert np.array_equal(ref_h[img:img + 1], ref_o) and np.array_equal(bnd_h[img:img + 1], bnd_o)
        one = dp.check(imp.numpy()[img:img + 1], ref_o, bnd_o, "fp16", ksb)
        assert one["ok"], one
        st = dp.check(imp.numpy(), ref_h, bnd_h, "fp16", ksb)
        print("fp16 CONV2D [16,28,28,256]x[256,3,3,256]:", st)
        assert st["ok"] and st["max_ulp"] <= 32 and st["max_ulp_conditioned"] <= 1.0
        assert st["max_rel_to_bound"] <= 2.0 ** -12          # half an fp16 ULP of the sum of absolute products
    finally:
        for t in list(ctx._owned):
            ctx._free(t)

    m = cases.c5_matmul()
    nb, h, k = m["a"].shape
    w = m["b"].shape[2]
    try:
        ta, tb = ctx.upload(m["a"], capi.BF16), ctx.upload(m["b"], capi.BF16)
        imp, ref, bnd = ctx.empty((nb, h, w), capi.FP32), ctx.empty((nb, h, w), capi.F64), ctx.empty((nb, h, w), capi.F64)
        ctx.matmul(capi.BF16, nb, h, k, w, ta, tb, 0, 0, imp)
        assert ctx.last_kernel == "matmul_gemm_bf16"
        ctx.matmul_precise(capi.BF16, nb, h, k, w, ta, tb, False, ref)
        ctx.matmul_precise(capi.BF16, nb, h, k, w, ta, tb, True, bnd)
        ksb = dp.kernel_size_bound(k, "fp32", has_bias=False)
        r = ctx.dot_product_check(capi.FP32, nb * h * w, imp, ref, bnd, ksb)
        assert ctx.sync() == capi.VALID and r.compliant
        st = dp.check(imp.numpy(), ref.numpy(), bnd.numpy(), "fp32", ksb)
        print("bf16 MATMUL [4,2048,4096]x[4,4096,2048]:", st)
        assert st["ok"] and st["max_ulp_conditioned"] <= 8
        assert st["max_rel_to_bound"] <= 2.0 ** -21           # four fp32 ULPs of the sum of absolute products
    finally:
        for t in list(ctx._owned):
            ctx._free(t)
