"""tmi_transpose_conv2d_noalloc: the entry point that allocates nothing (its re-laid-out operands live in the
library's static device array) against tmi_transpose_conv2d on the same operands, bit for bit, on two calls in a
row, the second with a smaller input, and (integers) against the CPU oracle; that it leaves the context's scratch
buffer unallocated; and its refusal of operands beyond the array's size."""
from __future__ import annotations

import numpy as np
import pytest

import oracle
from reference_model_amd import Context, capi

pytestmark = pytest.mark.gpu


def _desc(x, w, bias, out_pad, stride, in_dtype):
    n, ih, iw, ic = x.shape
    oc, kh, kw, _ = w.shape
    d = capi.TconvDesc()
    d.in_dtype, d.out_dtype = in_dtype, capi.INT32 if in_dtype == capi.INT8 else in_dtype
    d.N, d.IH, d.IW, d.IC, d.OC, d.KH, d.KW = n, ih, iw, ic, oc, kh, kw
    d.OH = (ih - 1) * stride[0] + out_pad[0] + out_pad[1] + kh
    d.OW = (iw - 1) * stride[1] + out_pad[2] + out_pad[3] + kw
    d.out_pad[:], d.stride[:] = list(out_pad), list(stride)
    d.bias_len = bias.shape[0]
    return d


def _operands(rng, shape, oc, k, fp):
    n, ih, iw, ic = shape
    if fp:
        x = rng.standard_normal(shape).astype(np.float16)
        w = (rng.standard_normal((oc, k, k, ic)) / np.sqrt(k * k * ic)).astype(np.float16)
        b = rng.standard_normal(oc).astype(np.float16)
        return x, w, b, capi.FP16, 0, 0
    x = rng.integers(-128, 128, shape, dtype=np.int8)
    w = rng.integers(-127, 128, (oc, k, k, ic), dtype=np.int8)
    b = rng.integers(-(1 << 16), 1 << 16, oc, dtype=np.int32)
    return x, w, b, capi.INT8, -9, 3


def _run_both(ctx, x, w, b, dt, in_zp, w_zp, out_pad, stride):
    """the entry point that allocates nothing first, on a context whose scratch buffer must stay unallocated; then the
    ordinary entry point, which allocates one"""
    d = _desc(x, w, b, out_pad, stride, dt)
    tx, tw, tb = ctx.upload(x, dt), ctx.upload(w, dt), ctx.upload(b)
    np_out = np.int32 if dt == capi.INT8 else np.float16
    shape = (d.N, d.OH, d.OW, d.OC)
    want_t, got_t = ctx.empty(shape, d.out_dtype, np_out), ctx.empty(shape, d.out_dtype, np_out)
    before = ctx.workspace_bytes()
    ctx.transpose_conv2d_noalloc(d, tx, tw, tb, in_zp, w_zp, got_t)
    noalloc_kernel = ctx.last_kernel
    assert ctx.sync() == capi.VALID
    assert ctx.workspace_bytes() == before, "the entry point that allocates nothing grew the context's scratch buffer"
    ctx.transpose_conv2d(d, tx, tw, tb, in_zp, w_zp, want_t)
    assert ctx.last_kernel == noalloc_kernel
    assert ctx.sync() == capi.VALID
    want, got = want_t.numpy(), got_t.numpy()
    for t in (tx, tw, tb, want_t, got_t):
        t.free()
    return want, got


@pytest.mark.parametrize("fp", [False, True], ids=["int8", "fp16"])
def test_noalloc_matches_transpose_conv2d_twice(fp):
    """Two calls in a row on one context, the second with a smaller input: the static array still holds the first
    call's operands, and the second call must not read any of them.  48 input channels keep the layer off the
    kernel that reads TRANSPOSE_CONV2D operands in place, so both re-laid-out operands go through scratch memory."""
    rng = np.random.default_rng(20260 + fp)
    ctx = Context(0)
    try:
        assert ctx.workspace_bytes() == (0, 0)
        # the third layer has unit stride: no holes, only the flipped weights go through the static array
        for i, (shape, oc, out_pad, stride) in enumerate((((2, 13, 11, 48), 40, (0, 1, 1, 0), (2, 2)),
                                                          ((1, 5, 7, 48), 24, (1, 0, 0, 0), (2, 3)),
                                                          ((2, 9, 8, 48), 32, (0, 0, 1, 1), (1, 1)))):
            x, w, b, dt, in_zp, w_zp = _operands(rng, shape, oc, 3, fp)
            want, got = _run_both(ctx, x, w, b, dt, in_zp, w_zp, out_pad, stride)
            assert want.shape == got.shape and want.size > 0
            assert np.array_equal(want.view(np.uint8), got.view(np.uint8)), (
                f"{shape}: {int(np.count_nonzero(want != got))} of {want.size} elements differ")
            if not fp:
                ref = oracle.transpose_conv2d("i8", x, w, b, out_pad, stride, in_zp, w_zp)
                assert np.array_equal(got, ref), f"{shape}: differs from the oracle"
            if i == 0:
                assert ctx.workspace_bytes()[0] > 0    # the ordinary entry point did allocate
    finally:
        ctx.close()


@pytest.mark.parametrize("ic", [3, 4])
def test_noalloc_stays_off_the_kernel_that_needs_the_contexts_buffer(ic):
    """At most 4 input channels, 3 x 3 taps, weight zero point 0: as a CONV2D this layer goes to the first-layer
    kernel, whose pre-pass writes the context's scratch buffer (growing it on demand).  Reached from
    TRANSPOSE_CONV2D the convolution must take another kernel: its operands lie in scratch memory already, and the
    entry point that allocates nothing may not grow anything."""
    rng = np.random.default_rng(977 + ic)
    ctx = Context(0)
    try:
        assert ctx.workspace_bytes() == (0, 0)
        for shape, oc, out_pad, stride in (((2, 9, 7, ic), 16, (0, 1, 1, 0), (2, 2)), ((1, 6, 5, ic), 8, (0, 0, 0, 0), (1, 1))):
            x, w, b, dt, in_zp, _ = _operands(rng, shape, oc, 3, False)
            want, got = _run_both(ctx, x, w, b, dt, in_zp, 0, out_pad, stride)
            assert np.array_equal(want, got)
            assert np.array_equal(got, oracle.transpose_conv2d("i8", x, w, b, out_pad, stride, in_zp, 0))
    finally:
        ctx.close()


def test_noalloc_refuses_operands_beyond_the_static_array():
    """The input with its stride holes alone exceeds TMI_NOALLOC_SCRATCH_BYTES: TMI_ERROR, nothing launched (the
    operand pointers are never dereferenced: they are small valid buffers)."""
    ctx = Context(0)
    try:
        d = capi.TconvDesc()
        d.in_dtype, d.out_dtype = capi.INT8, capi.INT32
        d.N, d.IH, d.IW, d.IC, d.OC, d.KH, d.KW = 8, 300, 300, 48, 8, 3, 3
        d.stride[:] = [2, 2]
        d.out_pad[:] = [0, 0, 0, 0]
        d.OH, d.OW = (d.IH - 1) * 2 + 3, (d.IW - 1) * 2 + 3
        d.bias_len = 1
        need = 8 * 599 * 599 * 48
        assert need > capi.NOALLOC_SCRATCH_BYTES
        t = ctx.empty((64,), capi.INT8)
        with pytest.raises(capi.TmiError) as e:
            ctx.transpose_conv2d_noalloc(d, t, t, t, 0, 0, t)
        assert e.value.status == capi.ERROR and "TMI_NOALLOC_SCRATCH_BYTES" in e.value.message
        assert ctx.sync() == capi.VALID
    finally:
        ctx.close()
