"""Seeded random layers through the automatic kernel choice, as a caller of the C ABI gets it: every operator of the
path with random geometry (kernel, stride, dilation, padding), channel counts on both sides of the kernels'
eligibility rules (multiples of 16 / 64 and odd ones), random zero points, fused and separate RESCALE + CLAMP.
Integer work: bit for bit against the CPU oracle.  The hand-picked shape lists of the other files exercise named
corner cases; this one looks for what nobody thought of."""
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


def _axis(rng, k, max_out):
    """(extent, pad_lo, pad_hi, stride, dilation, out) with (extent - 1 + pads - (k - 1) * dilation) % stride == 0"""
    while True:
        stride, dil = int(rng.integers(1, 4)), int(rng.integers(1, 3))
        lo, hi = int(rng.integers(0, k + 1)), int(rng.integers(0, k + 1))
        out = int(rng.integers(1, max_out + 1))
        extent = (out - 1) * stride + (k - 1) * dil + 1 - lo - hi
        if extent >= 1:
            return extent, lo, hi, stride, dil, out


CHANNELS = [1, 3, 8, 13, 16, 24, 32, 48, 64, 80, 96, 128, 144, 256]


@pytest.mark.parametrize("seed", range(120))
def test_conv2d_random_layer(ctx, seed):
    rng = np.random.default_rng(7000 + seed)
    kh, kw = (int(rng.integers(1, 6)), int(rng.integers(1, 6))) if seed % 3 else ((3, 3) if seed % 2 else (1, 1))
    ih, pt, pb, sy, dy, oh = _axis(rng, kh, 24)
    iw, pl, pr, sx, dx, ow = _axis(rng, kw, 24)
    n = int(rng.integers(1, 4))
    ic, oc = int(rng.choice(CHANNELS)), int(rng.choice(CHANNELS))
    in_zp = int(rng.integers(-128, 128)) if seed % 4 else 0
    w_zp = int(rng.integers(-128, 128)) if seed % 5 == 0 else 0
    x = rng.integers(-128, 128, (n, ih, iw, ic)).astype(np.int8)
    w = rng.integers(-128, 128, (oc, kh, kw, ic)).astype(np.int8)
    bias = rng.integers(-(1 << 18), 1 << 18, oc if seed % 7 else 1).astype(np.int32)
    pad, stride, dil = (pt, pb, pl, pr), (sy, sx), (dy, dx)
    acc = oracle.conv2d("i8", x, w, bias, pad, stride, dil, in_zp=in_zp, w_zp=w_zp)
    got, st = gpu_ops.conv2d(ctx, x, w, bias, pad, stride, dil, in_zp=in_zp, w_zp=w_zp)
    assert st == capi.VALID and np.array_equal(got, acc), (ctx.last_kernel, x.shape, w.shape, pad, stride, dil)
    mult = rng.integers(1 << 30, 1 << 31, oc).astype(np.int32)
    shift = rng.integers(30, 46, oc).astype(np.int8) if seed % 3 else np.full(oc, 40, np.int8)
    mode = capi.ROUND_DOUBLE if seed % 2 else capi.ROUND_SINGLE
    out_dt = np.int8 if seed % 6 else np.int16
    out_zp = int(rng.integers(-30, 30)) if out_dt == np.int8 else 0
    clamp = None if seed % 4 == 1 else ((0, 100) if seed % 4 == 2 else (-90, 77))
    got, st = gpu_ops.conv2d(ctx, x, w, bias, pad, stride, dil, in_zp=in_zp, w_zp=w_zp,
                             rescale=dict(mult=mult, shift=shift, out_zp=out_zp, out_dtype=out_dt, rounding_mode=mode),
                             clamp=clamp)
    want, wst = oracle.rescale(acc, mult, shift, out_zp=out_zp, out_dtype=out_dt, rounding_mode=mode)
    if clamp is not None:
        want = oracle.clamp(want, *clamp)
    assert st == wst and np.array_equal(got, want), (ctx.last_kernel, x.shape, w.shape, pad, stride, dil, shift[:4])


@pytest.mark.parametrize("seed", range(80))
def test_depthwise_conv2d_random_layer(ctx, seed):
    rng = np.random.default_rng(8000 + seed)
    kh, kw = (int(rng.integers(1, 5)), int(rng.integers(1, 5))) if seed % 2 else (3, 3)
    ih, pt, pb, sy, dy, oh = _axis(rng, kh, 24)
    iw, pl, pr, sx, dx, ow = _axis(rng, kw, 24)
    n = int(rng.integers(1, 4))
    c = int(rng.choice(CHANNELS))
    m = 1 if seed % 3 else int(rng.integers(1, 4))
    in_zp = int(rng.integers(-128, 128)) if seed % 4 else 0
    w_zp = int(rng.integers(-128, 128)) if seed % 5 == 0 else 0
    x = rng.integers(-128, 128, (n, ih, iw, c)).astype(np.int8)
    w = rng.integers(-128, 128, (kh, kw, c, m)).astype(np.int8)
    bias = rng.integers(-(1 << 16), 1 << 16, c * m).astype(np.int32)
    pad, stride, dil = (pt, pb, pl, pr), (sy, sx), (dy, dx)
    acc = oracle.depthwise_conv2d("i8", x, w, bias, pad, stride, dil, in_zp=in_zp, w_zp=w_zp)
    got, st = gpu_ops.conv2d(ctx, x, w, bias, pad, stride, dil, in_zp=in_zp, w_zp=w_zp, depthwise=True)
    assert st == capi.VALID and np.array_equal(got, acc), (ctx.last_kernel, x.shape, w.shape, pad, stride, dil)
    mult = rng.integers(1 << 30, 1 << 31, c * m).astype(np.int32)
    shift = rng.integers(26, 42, c * m).astype(np.int8)
    mode = capi.ROUND_DOUBLE if seed % 2 else capi.ROUND_SINGLE
    got, st = gpu_ops.conv2d(ctx, x, w, bias, pad, stride, dil, in_zp=in_zp, w_zp=w_zp, depthwise=True,
                             rescale=dict(mult=mult, shift=shift, out_zp=-7, rounding_mode=mode))
    want, wst = oracle.rescale(acc, mult, shift, out_zp=-7, rounding_mode=mode)
    assert st == wst and np.array_equal(got, want), (ctx.last_kernel, x.shape, w.shape, pad, stride, dil)


@pytest.mark.parametrize("seed", range(60))
def test_matmul_random_shape(ctx, seed):
    rng = np.random.default_rng(9000 + seed)
    n = int(rng.integers(1, 5))
    h, k, w = (int(rng.choice([1, 7, 31, 64, 100, 128, 257, 384])) for _ in range(3))
    if seed % 10 == 0:
        h, k, w = 512, 256, 640            # large enough for the matrix-core GEMM kernel
    a = rng.integers(-128, 128, (n, h, k)).astype(np.int8)
    b = rng.integers(-128, 128, (n, k, w)).astype(np.int8)
    a_zp = int(rng.integers(-128, 128)) if seed % 3 else 0
    b_zp = int(rng.integers(-128, 128)) if seed % 4 else 0
    got, st = gpu_ops.matmul(ctx, a, b, a_zp, b_zp)
    assert st == capi.VALID and np.array_equal(got, oracle.matmul("i8", a, b, a_zp, b_zp)), (ctx.last_kernel, a.shape, b.shape)


@pytest.mark.parametrize("seed", range(40))
def test_transpose_conv2d_and_conv3d_random_layer(ctx, seed):
    rng = np.random.default_rng(9500 + seed)
    ic, oc = int(rng.choice([1, 5, 16, 32, 64, 128])), int(rng.choice([1, 6, 16, 48, 64]))
    in_zp = int(rng.integers(-128, 128))
    w_zp = int(rng.integers(-128, 128)) if seed % 3 == 0 else 0
    if seed % 2:
        kh, kw = int(rng.integers(1, 5)), int(rng.integers(1, 5))
        stride = (int(rng.integers(1, 4)), int(rng.integers(1, 4)))
        out_pad = tuple(int(v) for v in rng.integers(-min(kh, kw) + 1 if min(kh, kw) > 1 else 0, 3, 4))
        x = rng.integers(-128, 128, (int(rng.integers(1, 3)), int(rng.integers(1, 12)), int(rng.integers(1, 12)), ic)).astype(np.int8)
        w = rng.integers(-128, 128, (oc, kh, kw, ic)).astype(np.int8)
        bias = rng.integers(-(1 << 18), 1 << 18, oc).astype(np.int32)
        try:
            want = oracle.transpose_conv2d("i8", x, w, bias, out_pad, stride, in_zp, w_zp)
        except oracle.OracleStatus:
            pytest.skip("the drawn out_pad leaves no output")
        got, st = gpu_ops.transpose_conv2d(ctx, x, w, bias, out_pad, stride, in_zp, w_zp)
        assert st == capi.VALID and np.array_equal(got, want), (ctx.last_kernel, x.shape, w.shape, out_pad, stride)
    else:
        kd, kh, kw = (int(rng.integers(1, 4)) for _ in range(3))
        dims, pads, strides, dils = [], [], [], []
        for k in (kd, kh, kw):
            e, lo, hi, s, d, _ = _axis(rng, k, 8)
            dims.append(e), pads.extend([lo, hi]), strides.append(s), dils.append(d)
        ic = min(ic, 32)
        x = rng.integers(-128, 128, (int(rng.integers(1, 3)), *dims, ic)).astype(np.int8)
        w = rng.integers(-128, 128, (oc, kd, kh, kw, ic)).astype(np.int8)
        bias = rng.integers(-(1 << 18), 1 << 18, oc).astype(np.int32)
        want = oracle.conv3d("i8", x, w, bias, tuple(pads), tuple(strides), tuple(dils), in_zp, w_zp)
        got, st = gpu_ops.conv3d(ctx, x, w, bias, tuple(pads), tuple(strides), tuple(dils), in_zp, w_zp)
        assert st == capi.VALID and np.array_equal(got, want), (ctx.last_kernel, x.shape, w.shape, pads, strides, dils)


@pytest.mark.parametrize("block", range(12))
def test_rescale_random_configurations(ctx, block):
    """stand-alone RESCALE with every attribute drawn at random - element types, signedness, scale width, rounding
    mode (INEXACT_ROUND included), per-channel or not, rank, zero points inside and outside their rules, shifts over
    the whole 2..62, values over the whole input range: the status always agrees with the oracle's (ERROR as an
    exception), and every element does whenever the status is VALID.  50 configurations per test."""
    from reference_model_amd import TmiError
    seen = {oracle.VALID: 0, oracle.UNPREDICTABLE: 0, oracle.ERROR: 0}
    for seed in range(block * 50, block * 50 + 50):
        rng = np.random.default_rng(31000 + seed)
        in_dt = [np.int8, np.int16, np.int32][int(rng.integers(0, 3))]
        out_dt = [np.int8, np.int16, np.int32][int(rng.integers(0, 3))]
        in_u, out_u = bool(rng.random() < 0.15), bool(rng.random() < 0.15)
        scale32 = bool(rng.random() < 0.7)
        mode = [capi.ROUND_SINGLE, capi.ROUND_DOUBLE, capi.ROUND_INEXACT][int(rng.integers(0, 3))]
        per_channel = bool(rng.random() < 0.7)
        rank = int(rng.integers(1, 6))
        C = int(rng.choice([1, 2, 3, 4, 7, 8, 12, 16, 31, 32, 60, 64, 96, 128, 130]))
        lead = [int(rng.integers(1, 9)) for _ in range(rank - 1)]
        if rng.random() < 0.2 and rank > 1:
            lead[0] = int(rng.integers(100, 3000))
        shape = tuple(lead + [C])
        nm = C if per_channel else 1
        top = 31 if scale32 else 15
        mult = rng.integers(1 << (top - 1), 1 << top, nm) if rng.random() < 0.7 else rng.integers(0, 1 << top, nm)
        s_lo, s_hi = [(2, 63), (30, 47), (32, 35), (20, 32), (40, 63)][int(rng.integers(0, 5))]
        shift = rng.integers(s_lo, s_hi, nm)
        info = np.iinfo(in_dt)
        if rng.random() < 0.5:
            x = rng.integers(info.min, info.max + 1, shape, dtype=np.int64)
        else:
            mag = max(1, min(int(shift.min()) - 2, 8 * np.dtype(in_dt).itemsize - 1))
            x = rng.integers(-(1 << mag), 1 << mag, shape, dtype=np.int64)
        x = np.clip(x, info.min, info.max).astype(in_dt)

        def zero_point(dt, unsigned):
            if rng.random() < 0.05:
                return int(rng.integers(-200, 40000))
            if np.dtype(dt) == np.int8:
                return int(rng.integers(0, 256)) if unsigned else int(rng.integers(-128, 128))
            if np.dtype(dt) == np.int16 and unsigned:
                return int(rng.choice([0, 32768]))
            return 0

        kw = dict(in_zp=zero_point(in_dt, in_u), out_zp=zero_point(out_dt, out_u), out_dtype=out_dt, scale32=scale32,
                  rounding_mode=mode, per_channel=per_channel, input_unsigned=in_u, output_unsigned=out_u)
        want, wst = oracle.rescale(x, mult, shift, **kw)
        try:
            got, st = gpu_ops.rescale(ctx, x, mult, shift, **kw)
        except TmiError:
            got, st = None, capi.ERROR
        assert st == wst, (seed, ctx.last_kernel, shape, in_dt, kw)
        if wst == oracle.VALID:
            got = got.view(want.dtype)
            if mode == capi.ROUND_INEXACT:
                # Where float(value) * float(multiplier) * 2^-shift leaves int32 the reference's cast is undefined
                # (type_conversion.cpp:323); device and oracle share the x86-64 convention there, which is an agreement
                # between the two and not parity with the reference: those elements are kept out of the parity claim.
                bits = 8 * np.dtype(in_dt).itemsize
                v = x.astype(np.int64)
                if in_u:
                    v = v & ((1 << bits) - 1)
                v = v - kw["in_zp"]
                m = np.broadcast_to(np.asarray(mult, np.int64), (nm,)) if nm > 1 else np.full(C, int(mult[0]), np.int64)
                sh = np.broadcast_to(np.asarray(shift, np.int64), (nm,)) if nm > 1 else np.full(C, int(shift[0]), np.int64)
                t = np.rint(v.astype(np.float32) * m.astype(np.float32) * np.exp2(-sh.astype(np.float32)))
                defined = (t >= -2147483648.0) & (t < 2147483648.0)
                assert np.array_equal(got[defined], want[defined]), (seed, ctx.last_kernel, shape, in_dt, kw)
                assert np.array_equal(got[~defined], want[~defined]), ("x86-64 convention", seed, shape, in_dt, kw)
            else:
                assert np.array_equal(got, want), (seed, ctx.last_kernel, shape, in_dt, kw)
        seen[wst] += 1
    assert seen[oracle.VALID] >= 20 and seen[oracle.ERROR] >= 5


@pytest.mark.parametrize("seed", range(60))
def test_floating_point_random_layer_within_the_dot_product_bound(ctx, seed):
    """fp16 / bf16 / fp32 CONV2D, DEPTHWISE_CONV2D and MATMUL with random geometry: the result against the fp64 oracle
    with the reference's DOT_PRODUCT rule (verify_dot_product.cpp:30-139; the tolerance is abs_bound = 2 ksb units of
    max(bound * 2^-(1 + fraction bits), normal_min), ksb from the kernel size and the accumulator / output types)."""
    import cases
    import dot_product_check as dp
    from test_gpu_compliance_passes import narrow
    rng = np.random.default_rng(9900 + seed)
    kind = ["fp16", "bf16", "fp32"][seed % 3]
    op = ["conv2d", "depthwise", "matmul"][(seed // 3) % 3]
    if op == "matmul":
        n = int(rng.integers(1, 4))
        h, k, w = (int(rng.choice([1, 9, 32, 64, 100, 128, 256])) for _ in range(3))
        if seed % 9 == 8:
            h, k, w = 384, 256, 512
        a_s, af, dtype = narrow(rng.normal(0, 1, (n, h, k)).astype(np.float32), kind)
        b_s, bf, _ = narrow(rng.normal(0, 1, (n, k, w)).astype(np.float32), kind)
        out = ctx.empty((n, h, w), capi.FP32)
        try:
            ctx.matmul(dtype, n, h, k, w, ctx.upload(a_s, dtype), ctx.upload(b_s, dtype), 0, 0, out)
            assert ctx.sync() == capi.VALID
            got = out.numpy().astype(np.float64)
        finally:
            for t in list(ctx._owned):
                ctx._free(t)
        ref, bnd = oracle.matmul("f64", af, bf), oracle.matmul("f64", af, bf, abs_mode=True)
        st = dp.check(got, ref, bnd, "fp32", dp.kernel_size_bound(k, "fp32", has_bias=False))
        assert st["ok"], (ctx.last_kernel, kind, (n, h, k, w), st)
        return
    kh, kw = (int(rng.integers(1, 5)), int(rng.integers(1, 5))) if seed % 2 else (3, 3)
    ih, pt, pb, sy, dy, oh = _axis(rng, kh, 16)
    iw, pl, pr, sx, dx, ow = _axis(rng, kw, 16)
    n = int(rng.integers(1, 3))
    pad, stride, dil = (pt, pb, pl, pr), (sy, sx), (dy, dx)
    if op == "conv2d":
        ic, oc = int(rng.choice([1, 7, 16, 32, 64, 96, 256])), int(rng.choice([1, 5, 16, 64, 128]))
        xs, xf, dtype = narrow(rng.normal(0, 1, (n, ih, iw, ic)).astype(np.float32), kind)
        ws, wf, _ = narrow(rng.normal(0, 1, (oc, kh, kw, ic)).astype(np.float32), kind)
        bs, bf, _ = narrow(rng.normal(0, 1, oc).astype(np.float32), kind)
        ref = oracle.conv2d("f64", xf, wf, bf, pad, stride, dil)
        bnd = oracle.conv2d("f64", xf, wf, bf, pad, stride, dil, abs_mode=True)
        ks = kh * kw * ic
    else:
        c, m = int(rng.choice([1, 6, 16, 48, 96])), int(rng.integers(1, 3))
        oc = c * m
        xs, xf, dtype = narrow(rng.normal(0, 1, (n, ih, iw, c)).astype(np.float32), kind)
        ws, wf, _ = narrow(rng.normal(0, 1, (kh, kw, c, m)).astype(np.float32), kind)
        bs, bf, _ = narrow(rng.normal(0, 1, oc).astype(np.float32), kind)
        ref = oracle.depthwise_conv2d("f64", xf, wf, bf, pad, stride, dil)
        bnd = oracle.depthwise_conv2d("f64", xf, wf, bf, pad, stride, dil, abs_mode=True)
        ks = kh * kw
    d = ctx.conv_desc(dtype, dtype, xs.shape, oc, kh, kw, (oh, ow), pad, stride, dil, oc)
    out = ctx.empty((n, oh, ow, oc), dtype, xs.dtype)
    try:
        fn = ctx.depthwise_conv2d if op == "depthwise" else ctx.conv2d
        fn(d, ctx.upload(xs, dtype), ctx.upload(ws, dtype), ctx.upload(bs, dtype), 0, 0, out)
        assert ctx.sync() == capi.VALID
        got = out.numpy()
    finally:
        for t in list(ctx._owned):
            ctx._free(t)
    got = cases.bf16_bits_to_float(got).astype(np.float64) if kind == "bf16" else got.astype(np.float64)
    st = dp.check(got, ref, bnd, kind, dp.kernel_size_bound(ks, kind))
    assert st["ok"], (ctx.last_kernel, kind, op, xs.shape, ws.shape, pad, stride, dil, st)
