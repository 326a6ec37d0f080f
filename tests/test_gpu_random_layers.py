"""Random layers under the library's own kernel choice against the CPU oracle, through the C ABI: seeded draws of int8
CONV2D / DEPTHWISE_CONV2D (int32 results, or the fused RESCALE with an optional CLAMP) and MATMUL, of fp16 / bf16 CONV2D /
DEPTHWISE_CONV2D / MATMUL, and of int8 TRANSPOSE_CONV2D, CONV3D, pooling and stand-alone RESCALE.  Half of the convolutions
are drawn from the shapes the specialised kernels take (zero weight zero point, channel counts that are multiples of 8,
1x1 / 3x3 / 7x7 taps), the rest from everything legal (CONV2D: tensor_ops.cpp:828-882; RESCALE: type_conversion.cpp:224-421).
Integer results are compared bit for bit; floating-point results with the reference's DOT_PRODUCT check
(verify_dot_product.cpp:30-139) plus at most 2 ulp of the output type where the result is not a cancellation.
The hand-picked cases of the other files pin each kernel's corners; this one looks for what nobody thought of (it found a
layer whose tile search overran the LDS)."""
import numpy as np
import pytest

import cases
import dot_product_check as dp
import gpu_ops
import oracle
from reference_model_amd import Context, capi

pytestmark = pytest.mark.gpu

ICS = [1, 2, 3, 4, 5, 8, 12, 16, 24, 32, 40, 48, 64, 72, 96, 104, 128, 160, 168, 192, 256, 320, 512]
OCS = [1, 3, 8, 16, 24, 32, 40, 56, 64, 72, 96, 104, 128, 136, 256]
NICE_ICS = [3, 4, 8, 16, 24, 32, 40, 64, 96, 128, 144, 160, 192, 256, 384, 512, 576, 960, 1024]
NICE_OCS = [8, 16, 24, 32, 48, 64, 96, 128, 160, 256, 320, 512]


@pytest.fixture(scope="module")
def ctx():
    c = Context(0)
    yield c
    c.close()


def _int8_layer(ctx, rng):
    """one int8 CONV2D / DEPTHWISE_CONV2D / MATMUL; returns (description, ok) or None when the draw has no legal geometry"""
    kind = str(rng.choice(["conv", "conv", "conv", "dw", "mm"]))
    fused = bool(rng.integers(0, 2))
    in_zp = int(rng.choice([0, 0, -128, 127, int(rng.integers(-128, 128))]))
    if kind == "mm":
        n, h, c, w_ = int(rng.integers(1, 4)), int(rng.integers(1, 200)), int(rng.choice(ICS)), int(rng.choice(OCS + [33, 100, 200]))
        a = rng.integers(-128, 128, (n, h, c)).astype(np.int8)
        b = rng.integers(-128, 128, (n, c, w_)).astype(np.int8)
        b_zp = int(rng.choice([0, 0, 5, -7]))
        got, st = gpu_ops.matmul(ctx, a, b, in_zp, b_zp)
        return ("mm", n, h, c, w_, in_zp, b_zp), st == capi.VALID and np.array_equal(got, oracle.matmul("i8", a, b, in_zp, b_zp))
    nice = bool(rng.integers(0, 2))
    if nice:    # shapes the specialised kernels take
        kh = kw = 3 if kind == "dw" else int(rng.choice([1, 3, 3, 7]))
        sy = sx = int(rng.choice([1, 1, 2]))
        dy = dx = 1
        pad = [kh // 2] * 4 if rng.integers(0, 2) else [int(rng.integers(0, kh)) for _ in range(4)]
        oh, ow, n = int(rng.integers(1, 40)), int(rng.integers(1, 40)), int(rng.integers(1, 9))
        ic, w_zp = int(rng.choice(NICE_ICS)), 0
    else:
        kh = int(rng.choice([1, 1, 2, 3, 3, 5, 7]))
        kw = kh if rng.integers(0, 3) else int(rng.choice([1, 1, 2, 3, 3, 5, 7]))
        sy, sx = int(rng.choice([1, 1, 2, 3])), int(rng.choice([1, 1, 2, 3]))
        dy, dx = int(rng.choice([1, 1, 1, 2])), int(rng.choice([1, 1, 1, 2]))
        pad = [int(rng.integers(0, kh)), int(rng.integers(0, kh)), int(rng.integers(0, kw)), int(rng.integers(0, kw))]
        oh, ow, n = int(rng.integers(1, 24)), int(rng.integers(1, 24)), int(rng.integers(1, 4))
        ic, w_zp = int(rng.choice(ICS)), int(rng.choice([0, 0, 0, 0, 3, -11]))
    ih = (oh - 1) * sy + (kh - 1) * dy + 1 - pad[0] - pad[1]
    iw = (ow - 1) * sx + (kw - 1) * dx + 1 - pad[2] - pad[3]
    if ih < 1 or iw < 1:
        return None
    if kind == "dw":
        m = 1 if nice else int(rng.choice([1, 1, 1, 2]))
        oc, wshape = ic * m, (kh, kw, ic, m)
    else:
        oc = int(rng.choice(NICE_OCS if nice else OCS))
        wshape = (oc, kh, kw, ic)
    if n * ih * iw * ic > 8_000_000 or n * oh * ow * oc * kh * kw * (1 if kind == "dw" else ic) > 400_000_000:
        return None
    small = fused and bool(rng.integers(0, 2))    # small sums, so that shifts below 32 stay inside apply_scale_32's value range
    x = rng.integers(-128, 128, (n, ih, iw, ic)).astype(np.int8)
    w = (rng.integers(-1, 2, wshape) if small else rng.integers(-128, 128, wshape)).astype(np.int8)
    bias = rng.integers(-3000, 3000, 1 if rng.integers(0, 5) == 0 else oc).astype(np.int32)
    desc = (kind, n, ih, iw, ic, oc, kh, kw, tuple(pad), (sy, sx), (dy, dx), in_zp, w_zp, fused, small, bias.size)
    conv = oracle.depthwise_conv2d if kind == "dw" else oracle.conv2d
    acc = conv("i8", x, w, bias, pad, (sy, sx), (dy, dx), in_zp=in_zp, w_zp=w_zp)
    if not fused:
        got, st = gpu_ops.conv2d(ctx, x, w, bias, pad, (sy, sx), (dy, dx), in_zp=in_zp, w_zp=w_zp, depthwise=kind == "dw")
        return desc, st == capi.VALID and np.array_equal(got, acc)
    od = np.int8 if rng.integers(0, 3) else np.int16
    out_zp = 0 if od == np.int16 else int(rng.integers(-128, 128))
    mode = int(rng.choice([capi.ROUND_SINGLE, capi.ROUND_DOUBLE]))
    per_channel = bool(rng.integers(0, 4))
    nc = oc if per_channel else 1
    mult = rng.integers(1 << 30, 1 << 31, nc).astype(np.int64).astype(np.int32)
    if small:
        shift = np.where(rng.integers(0, 3, nc) > 0, rng.integers(33, 40, nc), rng.integers(20, 33, nc)).astype(np.int8)
    else:
        shift = rng.integers(34, 48, nc).astype(np.int8)
    want, wst = oracle.rescale(acc, mult, shift, out_zp=out_zp, out_dtype=od, rounding_mode=mode, per_channel=per_channel)
    clamp = None
    if rng.integers(0, 2):
        clamp = (int(rng.integers(-128, 0)), int(rng.integers(0, 128)))
        want = oracle.clamp(want, *clamp)
    got, st = gpu_ops.conv2d(ctx, x, w, bias, pad, (sy, sx), (dy, dx), in_zp=in_zp, w_zp=w_zp, depthwise=kind == "dw", clamp=clamp,
                             rescale=dict(mult=mult, shift=shift, out_zp=out_zp, out_dtype=od, rounding_mode=mode, per_channel=per_channel))
    desc = desc + (np.dtype(od).name, out_zp, mode, per_channel, clamp, int(wst))
    return desc, st == wst and (wst != capi.VALID or np.array_equal(got, want))


@pytest.mark.parametrize("seed", [101, 102, 103, 104])
def test_random_int8_layers(ctx, seed):
    rng = np.random.default_rng(seed)
    kernels, ran = set(), 0
    for case in range(700):
        r = _int8_layer(ctx, rng)
        if r is None:
            continue
        desc, ok = r
        ran += 1
        kernels.add(ctx.last_kernel)
        assert ok, (seed, case, desc, ctx.last_kernel)
    assert ran > 500 and len(kernels) >= 18, sorted(kernels)    # the draw reaches most kernels


def _narrow(kind, *arrs):
    if kind == "fp16":
        s = [a.astype(np.float16) for a in arrs]
        return s, [v.astype(np.float64) for v in s], capi.FP16
    s = [cases.float_to_bf16_bits(a) for a in arrs]
    return s, [cases.bf16_bits_to_float(v).astype(np.float64) for v in s], capi.BF16


def _widen(kind, got):
    return got.astype(np.float64) if kind == "fp16" else cases.bf16_bits_to_float(got).astype(np.float64)


def _other_layer(ctx, rng):
    kind = str(rng.choice(["fconv", "fconv", "fdw", "fmm", "tconv", "conv3d", "pool", "rescale"]))
    if kind in ("fconv", "fdw"):
        fk = str(rng.choice(["fp16", "bf16"]))
        kh = int(rng.choice([1, 1, 2, 3, 3, 5, 7]))
        kw = kh if rng.integers(0, 3) else int(rng.choice([1, 2, 3, 5]))
        stride = (int(rng.choice([1, 1, 2, 3])), int(rng.choice([1, 1, 2, 3])))
        n, ic = int(rng.integers(1, 5)), int(rng.choice(ICS[:-1]))
        dil = (int(rng.choice([1, 1, 1, 2])), int(rng.choice([1, 1, 1, 2])))
        if rng.integers(0, 2):
            ic, dil = int(rng.choice([16, 32, 64, 128, 256])), (1, 1)
        pad = [int(rng.integers(0, kh)), int(rng.integers(0, kh)), int(rng.integers(0, kw)), int(rng.integers(0, kw))]
        oh, ow = int(rng.integers(1, 24)), int(rng.integers(1, 24))
        ih = (oh - 1) * stride[0] + (kh - 1) * dil[0] + 1 - pad[0] - pad[1]
        iw = (ow - 1) * stride[1] + (kw - 1) * dil[1] + 1 - pad[2] - pad[3]
        if ih < 1 or iw < 1:
            return None
        if kind == "fdw":
            m = int(rng.choice([1, 1, 2]))
            oc, wshape, ks = ic * m, (kh, kw, ic, m), kh * kw
        else:
            oc = int(rng.choice(OCS))
            wshape, ks = (oc, kh, kw, ic), kh * kw * ic
        if n * oh * ow * oc * ks > 200_000_000:
            return None
        x = rng.normal(0, 1, (n, ih, iw, ic)).astype(np.float32)
        w = rng.normal(0, 1 / np.sqrt(ks), wshape).astype(np.float32)
        b = rng.normal(0, 0.1, 1 if rng.integers(0, 5) == 0 else oc).astype(np.float32)
        (xs, ws, bs), (xf, wf, bf), dtype = _narrow(fk, x, w, b)
        conv = oracle.depthwise_conv2d if kind == "fdw" else oracle.conv2d
        ref = conv("f64", xf, wf, bf, pad, stride, dil)
        bnd = conv("f64", xf, wf, bf, pad, stride, dil, abs_mode=True)
        got, st = gpu_ops.conv2d(ctx, xs, ws, bs, pad, stride, dil, dtype=dtype, depthwise=kind == "fdw")
        res = dp.check(_widen(fk, got), ref, bnd, fk, dp.kernel_size_bound(ks, fk))
        # tolerance: the DOT_PRODUCT bound, and 2 ulp of the output type on results that are no cancellation
        return (kind, fk, n, ih, iw, ic, oc, kh, kw, tuple(pad), stride, dil, b.size, res), \
            st == capi.VALID and res["ok"] and res["max_ulp_conditioned"] <= 2.0
    if kind == "fmm":
        fk = str(rng.choice(["fp16", "bf16"]))
        n, h = int(rng.integers(1, 4)), int(rng.integers(1, 300))
        c, w_ = int(rng.choice(ICS + [33, 100, 200, 1000])), int(rng.choice(OCS + [33, 100, 200]))
        a = rng.normal(0, 1, (n, h, c)).astype(np.float32)
        b = rng.normal(0, 1 / np.sqrt(c), (n, c, w_)).astype(np.float32)
        (as_, bs), (af, bf), dtype = _narrow(fk, a, b)
        ref, bnd = oracle.matmul("f64", af, bf), oracle.matmul("f64", af, bf, abs_mode=True)
        got, st = gpu_ops.matmul(ctx, as_, bs, dtype=dtype)
        res = dp.check(got.astype(np.float64), ref, bnd, "fp32", dp.kernel_size_bound(c, "fp32", has_bias=False))
        return (kind, fk, n, h, c, w_, res), st == capi.VALID and res["ok"]    # tolerance: the DOT_PRODUCT bound for fp32 results
    if kind == "tconv":
        kh, kw = int(rng.choice([1, 2, 3, 3, 4, 5])), int(rng.choice([1, 2, 3, 3, 4, 5]))
        sy, sx = int(rng.choice([1, 2, 2, 3])), int(rng.choice([1, 2, 2, 3]))
        n, ih, iw = int(rng.integers(1, 4)), int(rng.integers(1, 16)), int(rng.integers(1, 16))
        ic, oc = int(rng.choice(ICS)), int(rng.choice(OCS))
        if rng.integers(0, 3) == 0:
            ic, oc, kh, kw = int(rng.choice([64, 96, 128])), int(rng.choice([48, 64, 96, 128])), 3, 3
        out_pad = [int(rng.integers(-((kh - 1) // 2), 3)), int(rng.integers(-((kh - 1) // 2), 3)),
                   int(rng.integers(-((kw - 1) // 2), 3)), int(rng.integers(-((kw - 1) // 2), 3))]
        oh = (ih - 1) * sy + out_pad[0] + out_pad[1] + kh
        ow = (iw - 1) * sx + out_pad[2] + out_pad[3] + kw
        if oh < 1 or ow < 1 or n * oh * ow * oc * kh * kw * ic > 200_000_000:
            return None
        in_zp, w_zp = int(rng.choice([0, -128, 127, 5])), int(rng.choice([0, 0, 0, 3]))
        x = rng.integers(-128, 128, (n, ih, iw, ic)).astype(np.int8)
        w = rng.integers(-128, 128, (oc, kh, kw, ic)).astype(np.int8)
        b = rng.integers(-3000, 3000, 1 if rng.integers(0, 5) == 0 else oc).astype(np.int32)
        want = oracle.transpose_conv2d("i8", x, w, b, out_pad, (sy, sx), in_zp, w_zp)
        got, st = gpu_ops.transpose_conv2d(ctx, x, w, b, out_pad, (sy, sx), in_zp, w_zp)
        return (kind, n, ih, iw, ic, oc, kh, kw, tuple(out_pad), (sy, sx), in_zp, w_zp, b.size), st == capi.VALID and np.array_equal(got, want)
    if kind == "conv3d":
        k3 = [int(rng.choice([1, 2, 3])) for _ in range(3)]
        st3 = [int(rng.choice([1, 1, 2])) for _ in range(3)]
        dl3 = [int(rng.choice([1, 1, 2])) for _ in range(3)]
        pad = [int(rng.integers(0, k)) for k in (k3[0], k3[0], k3[1], k3[1], k3[2], k3[2])]
        o3 = [int(rng.integers(1, 6)), int(rng.integers(1, 12)), int(rng.integers(1, 12))]
        i3 = [(o3[i] - 1) * st3[i] + (k3[i] - 1) * dl3[i] + 1 - pad[2 * i] - pad[2 * i + 1] for i in range(3)]
        if min(i3) < 1:
            return None
        n, ic, oc = int(rng.integers(1, 3)), int(rng.choice([1, 3, 8, 16, 32, 32, 64, 40])), int(rng.choice([1, 8, 16, 48, 64, 72]))
        in_zp, w_zp = int(rng.choice([0, -128, 127, 5])), int(rng.choice([0, 0, 0, 3]))
        x = rng.integers(-128, 128, (n, *i3, ic)).astype(np.int8)
        w = rng.integers(-128, 128, (oc, *k3, ic)).astype(np.int8)
        b = rng.integers(-3000, 3000, 1 if rng.integers(0, 5) == 0 else oc).astype(np.int32)
        want = oracle.conv3d("i8", x, w, b, pad, st3, dl3, in_zp, w_zp)
        got, st = gpu_ops.conv3d(ctx, x, w, b, pad, st3, dl3, in_zp, w_zp)
        return (kind, n, tuple(i3), ic, oc, tuple(k3), tuple(pad), tuple(st3), tuple(dl3), in_zp, w_zp, b.size), st == capi.VALID and np.array_equal(got, want)
    if kind == "pool":
        kh, kw = int(rng.integers(1, 6)), int(rng.integers(1, 6))
        sy, sx = int(rng.integers(1, 4)), int(rng.integers(1, 4))
        pad = [int(rng.integers(0, kh)), int(rng.integers(0, kh)), int(rng.integers(0, kw)), int(rng.integers(0, kw))]
        oh, ow = int(rng.integers(1, 30)), int(rng.integers(1, 30))
        ih, iw = (oh - 1) * sy + kh - pad[0] - pad[1], (ow - 1) * sx + kw - pad[2] - pad[3]
        if ih < 1 or iw < 1:
            return None
        n, c = int(rng.integers(1, 5)), int(rng.choice([1, 3, 4, 8, 16, 24, 32, 64, 100, 128, 256]))
        avg, wide = bool(rng.integers(0, 2)), bool(rng.integers(0, 2))
        x = (rng.integers(-32768, 32768, (n, ih, iw, c)).astype(np.int16) if wide else rng.integers(-128, 128, (n, ih, iw, c)).astype(np.int8))
        in_zp = int(rng.integers(-128, 128)) if (avg and not wide) else 0
        out_zp = int(rng.integers(-128, 128)) if (avg and not wide) else 0
        want = oracle.avg_pool2d(x, (kh, kw), (sy, sx), pad, in_zp, out_zp) if avg else oracle.max_pool2d(x, (kh, kw), (sy, sx), pad)
        got, st = gpu_ops.pool2d(ctx, x, (kh, kw), (sy, sx), pad, avg=avg, in_zp=in_zp, out_zp=out_zp)
        return (kind, avg, wide, n, ih, iw, c, kh, kw, (sy, sx), tuple(pad), in_zp, out_zp), st == capi.VALID and np.array_equal(got, want)
    rank = int(rng.integers(1, 5))
    shape = tuple(int(rng.integers(1, 40)) for _ in range(rank))
    idt, odt = rng.choice([np.int8, np.int16, np.int32]), rng.choice([np.int8, np.int16, np.int32])
    per_channel, scale32 = bool(rng.integers(0, 2)), bool(rng.integers(0, 2))
    nc = shape[-1] if per_channel else 1
    mode = int(rng.choice([capi.ROUND_SINGLE, capi.ROUND_DOUBLE])) if scale32 else capi.ROUND_SINGLE
    info = np.iinfo(idt)
    x = rng.integers(max(info.min, -(1 << 20)), min(info.max, 1 << 20) + 1, shape).astype(idt)
    mult = (rng.integers(1 << 29, 1 << 31, nc) if scale32 else rng.integers(1 << 13, 1 << 15, nc)).astype(np.int64)
    shift = rng.integers(30, 50, nc) if scale32 else rng.integers(14, 30, nc)
    in_zp = int(rng.integers(-128, 128)) if idt == np.int8 else 0
    out_zp = int(rng.integers(-128, 128)) if odt == np.int8 else 0
    want, wst = oracle.rescale(x, mult.astype(np.int32 if scale32 else np.int16), shift.astype(np.int8), in_zp, out_zp, odt,
                               scale32, mode, per_channel)
    got, st = gpu_ops.rescale(ctx, x, mult, shift, in_zp, out_zp, odt, scale32, mode, per_channel)
    return (kind, shape, np.dtype(idt).name, np.dtype(odt).name, per_channel, scale32, mode, in_zp, out_zp), \
        st == wst and (wst != capi.VALID or np.array_equal(got, want))


@pytest.mark.parametrize("seed", [201, 202])
def test_random_other_operators(ctx, seed):
    rng = np.random.default_rng(seed)
    kernels, ran = set(), 0
    for case in range(700):
        r = _other_layer(ctx, rng)
        if r is None:
            continue
        desc, ok = r
        ran += 1
        kernels.add(ctx.last_kernel)
        assert ok, (seed, case, desc, ctx.last_kernel)
    assert ran > 500 and len(kernels) >= 20, sorted(kernels)
