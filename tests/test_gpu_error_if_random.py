"""Seeded random operator descriptors, most of them broken in some attribute (negative or oversized padding, a zero
stride or dilation, an output size that the attribute rule does not give, a bias of the wrong length, zero points on
int16 pooling): the library has to refuse exactly the descriptors the CPU oracle refuses (the reference's ERROR_IF
conditions: check_pool2d_attribute tensor_ops.cpp:29-117 and :568-571 for pooling, check_conv_attribute :120-226 with
its callers :690-740, :901-950, :1139-1190 for the convolutions, :1982-2057 for TRANSPOSE_CONV2D) and agree bit for bit on the ones both accept.  The descriptor carries one channel count for input
and weights and the zero points arrive as int8 values in the reference, so neither is varied here."""
import numpy as np
import pytest

import gpu_ops
import oracle
from reference_model_amd import Context, TmiError, capi

pytestmark = pytest.mark.gpu

OPS = ("conv2d", "depthwise", "tconv", "conv3d", "avg", "max")


@pytest.fixture(scope="module")
def ctx():
    c = Context(0)
    yield c
    c.close()


def _outcome(fn):
    try:
        return "ok", fn()
    except oracle.OracleStatus as e:
        return "refused", e.status
    except TmiError as e:
        return "refused", e.status


def _nudged(rng, v):
    return int(v + rng.integers(-2, 3)) if rng.random() < 0.25 else int(v)


def _claimed(rng, true, rank):
    """The output size handed over: usually the rule's own, sometimes one that is off."""
    if true is None or rng.random() < 0.3:
        return tuple(max(1, _nudged(rng, b)) for b in (true or (1,) * rank))
    return tuple(true)


def _case(rng, op):
    """(description, oracle call, device call) of one random descriptor"""
    n, ih, iw, ic = (int(rng.integers(1, 3)), int(rng.integers(1, 9)), int(rng.integers(1, 9)), int(rng.integers(1, 6)))
    kh, kw, oc = int(rng.integers(1, 4)), int(rng.integers(1, 4)), int(rng.integers(1, 6))
    pad = [int(rng.integers(-1, 3)) if rng.random() < 0.3 else int(rng.integers(0, 2)) for _ in range(4)]
    stride = [int(rng.integers(0, 4)) if rng.random() < 0.2 else int(rng.integers(1, 3)) for _ in range(2)]
    dil = [int(rng.integers(0, 3)) if rng.random() < 0.2 else int(rng.integers(1, 3)) for _ in range(2)]
    zi, zw = int(rng.integers(-128, 128)), int(rng.integers(-128, 128))

    def bias_for(nout):
        length = nout if rng.random() < 0.6 else (1 if rng.random() < 0.6 else nout + 1)
        return rng.integers(-1000, 1000, length).astype(np.int32)

    if op in ("conv2d", "depthwise"):
        x = rng.integers(-128, 128, (n, ih, iw, ic)).astype(np.int8)
        if op == "conv2d":
            w, nout = rng.integers(-128, 128, (oc, kh, kw, ic)).astype(np.int8), oc
        else:
            m = int(rng.integers(1, 3))
            w, nout = rng.integers(-128, 128, (kh, kw, ic, m)).astype(np.int8), ic * m
        bias = bias_for(nout)
        out_hw = _claimed(rng, oracle.conv_out_hw(ih, iw, kh, kw, pad, stride, dil), 2)
        ofn = oracle.conv2d if op == "conv2d" else oracle.depthwise_conv2d
        return (dict(op=op, x=x.shape, w=w.shape, bias=bias.size, pad=pad, stride=stride, dilation=dil, out=out_hw),
                lambda: ofn("i8", x, w, bias, pad, stride, dil, zi, zw, out_hw=out_hw),
                lambda: gpu_ops.conv2d(ctx_, x, w, bias, pad, stride, dil, zi, zw, out_hw=out_hw,
                                       depthwise=(op == "depthwise")))
    if op == "tconv":
        x = rng.integers(-128, 128, (n, ih, iw, ic)).astype(np.int8)
        w = rng.integers(-128, 128, (oc, kh, kw, ic)).astype(np.int8)
        bias = bias_for(oc)
        out_pad = [int(rng.integers(-3, 3)) for _ in range(4)]
        true = ((ih - 1) * stride[0] + out_pad[0] + out_pad[1] + kh, (iw - 1) * stride[1] + out_pad[2] + out_pad[3] + kw)
        out_hw = true if rng.random() < 0.7 else (_nudged(rng, true[0]), _nudged(rng, true[1]))
        if min(out_hw) < 1:
            return None
        return (dict(op=op, x=x.shape, w=w.shape, bias=bias.size, out_pad=out_pad, stride=stride, out=out_hw),
                lambda: oracle.transpose_conv2d("i8", x, w, bias, out_pad, stride, zi, zw, out_hw=out_hw),
                lambda: gpu_ops.transpose_conv2d(ctx_, x, w, bias, out_pad, stride, zi, zw, out_hw=out_hw))
    if op == "conv3d":
        idp, kd = int(rng.integers(1, 5)), int(rng.integers(1, 3))
        x = rng.integers(-128, 128, (n, idp, ih, iw, ic)).astype(np.int8)
        w = rng.integers(-128, 128, (oc, kd, kh, kw, ic)).astype(np.int8)
        bias = bias_for(oc)
        pad6 = [int(rng.integers(-1, 2)) if rng.random() < 0.2 else int(rng.integers(0, 2)) for _ in range(2)] + pad
        stride3, dil3 = [int(rng.integers(1, 3))] + stride, [int(rng.integers(1, 3))] + dil
        out = _claimed(rng, oracle.conv3d_out_dhw((idp, ih, iw), (kd, kh, kw), pad6, stride3, dil3), 3)
        return (dict(op=op, x=x.shape, w=w.shape, bias=bias.size, pad=pad6, stride=stride3, dilation=dil3, out=out),
                lambda: oracle.conv3d("i8", x, w, bias, pad6, stride3, dil3, zi, zw, out_dhw=out),
                lambda: gpu_ops.conv3d(ctx_, x, w, bias, pad6, stride3, dil3, zi, zw, out_dhw=out))
    dt = np.int8 if rng.random() < 0.7 else np.int16
    info = np.iinfo(dt)
    x = rng.integers(info.min, info.max + 1, (n, ih, iw, ic)).astype(dt)
    kernel = [int(rng.integers(0, 4)) if rng.random() < 0.15 else kh, kw]
    out_hw = _claimed(rng, oracle.pool_out_hw(ih, iw, kernel, stride, pad) if min(stride) > 0 else None, 2)
    zi, zo = (zi if rng.random() < 0.5 else 0), (zw if rng.random() < 0.5 else 0)
    desc = dict(op=op, x=x.shape, dtype=dt.__name__, kernel=kernel, pad=pad, stride=stride, zp=(zi, zo), out=out_hw)
    if op == "avg":
        return (desc, lambda: oracle.avg_pool2d(x, kernel, stride, pad, zi, zo, out_hw=out_hw),
                lambda: gpu_ops.pool2d(ctx_, x, kernel, stride, pad, True, zi, zo, out_hw=out_hw))
    return (desc, lambda: oracle.max_pool2d(x, kernel, stride, pad, out_hw=out_hw),
            lambda: gpu_ops.pool2d(ctx_, x, kernel, stride, pad, False, out_hw=out_hw))


ctx_ = None


@pytest.mark.parametrize("op", OPS)
def test_broken_descriptors_are_refused_exactly_where_the_oracle_refuses_them(ctx, op):
    global ctx_
    ctx_ = ctx
    accepted = refused = 0
    for seed in range(400):
        rng = np.random.default_rng(900000 + 7 * seed + OPS.index(op))
        case = _case(rng, op)
        if case is None:
            continue
        desc, on_cpu, on_gpu = case
        want, got = _outcome(on_cpu), _outcome(on_gpu)
        assert want[0] == got[0], (seed, desc, want[:2], got[0])
        if want[0] == "refused":
            assert want[1] == got[1] == capi.ERROR, (seed, desc)
            refused += 1
        else:
            out, status = got[1]
            assert status == capi.VALID and out.shape == want[1].shape and np.array_equal(out, want[1]), (seed, desc)
            accepted += 1
    assert accepted >= 20 and refused >= 100, (accepted, refused)    # the generator must keep producing both kinds
