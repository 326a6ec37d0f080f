"""numpy-in / numpy-out helpers over the C ABI for the GPU parity tests (upload, run, download)."""
from __future__ import annotations

import numpy as np

import oracle
from reference_model_amd import capi

_TMI = {np.dtype(np.int8): capi.INT8, np.dtype(np.uint8): capi.INT8, np.dtype(np.int16): capi.INT16,
        np.dtype(np.uint16): capi.INT16, np.dtype(np.int32): capi.INT32, np.dtype(np.int64): capi.INT48,
        np.dtype(np.float16): capi.FP16, np.dtype(np.float32): capi.FP32}


def _conv_common(ctx, x, w_shape_khkwoc, bias, pad, stride, dilation, in_dtype, out_hw):
    kh, kw, oc = w_shape_khkwoc
    if out_hw is None:
        out_hw = oracle.conv_out_hw(x.shape[1], x.shape[2], kh, kw, pad, stride, dilation) or (0, 0)
    out_dtype = capi.INT32 if in_dtype == capi.INT8 else (capi.INT48 if in_dtype == capi.INT16 else in_dtype)
    d = ctx.conv_desc(in_dtype, out_dtype, x.shape, oc, kh, kw, out_hw, pad, stride, dilation, bias.shape[0])
    return d, out_hw, out_dtype


def conv2d(ctx, x, w, bias, pad=(0, 0, 0, 0), stride=(1, 1), dilation=(1, 1), in_zp=0, w_zp=0, out_hw=None,
           depthwise=False, dtype=None, rescale=None, clamp=None):
    """Runs CONV2D / DEPTHWISE_CONV2D (optionally fused with RESCALE[/CLAMP]); returns (out, status).

    rescale = dict(mult, shift, out_zp, out_dtype(np), rounding_mode, scale32, per_channel, output_unsigned)."""
    in_dtype = dtype or _TMI[x.dtype]
    if depthwise:
        kh, kw, c, m = w.shape
        oc = c * m
    else:
        oc, kh, kw, _ = w.shape
    d, out_hw, out_dtype = _conv_common(ctx, x, (kh, kw, oc), bias, pad, stride, dilation, in_dtype, out_hw)
    # INT16 inputs come with INT8 weights and an INT48 bias (int64)
    tx, tw = ctx.upload(x, in_dtype), ctx.upload(w, capi.INT8 if in_dtype == capi.INT16 else in_dtype)
    tb = ctx.upload(bias, None if bias.dtype != np.uint16 else in_dtype)
    shape = (x.shape[0], out_hw[0], out_hw[1], oc)
    try:
        if rescale is None:
            np_out = {capi.INT32: np.int32, capi.INT48: np.int64, capi.FP16: np.float16, capi.BF16: np.uint16,
                      capi.FP32: np.float32}[out_dtype]
            to = ctx.empty(shape, out_dtype, np_out)
            fn = ctx.depthwise_conv2d if depthwise else ctx.conv2d
            fn(d, tx, tw, tb, in_zp, w_zp, to)
        else:
            od = np.dtype(rescale.get("out_dtype", np.int8))
            mult, shift = np.atleast_1d(rescale["mult"]), np.atleast_1d(rescale["shift"]).astype(np.int8)
            scale32 = rescale.get("scale32", True)
            tm = ctx.upload(mult.astype(np.int32 if scale32 else np.int16))
            ts = ctx.upload(shift)
            r = ctx.rescale_desc(capi.INT32, _TMI[od], mult.size, shift.size, 0, rescale.get("out_zp", 0), scale32,
                                 rescale.get("rounding_mode", capi.ROUND_DOUBLE), rescale.get("per_channel", True),
                                 False, rescale.get("output_unsigned", False))
            to = ctx.empty(shape, _TMI[od], od)
            fn = ctx.depthwise_conv2d_rescale_clamp if depthwise else ctx.conv2d_rescale_clamp
            fn(d, tx, tw, tb, in_zp, w_zp, r, tm, ts, to, clamp)
        st = ctx.sync()
        return to.numpy(), st
    finally:
        for t in list(ctx._owned):
            ctx._free(t)


def matmul(ctx, a, b, a_zp=0, b_zp=0, dtype=None):
    in_dtype = dtype or _TMI[a.dtype]
    n, h, c = a.shape
    w = b.shape[2]
    ta, tb = ctx.upload(a, in_dtype), ctx.upload(b, in_dtype)
    to = ctx.empty((n, h, w), capi.INT32 if in_dtype == capi.INT8 else (capi.INT48 if in_dtype == capi.INT16 else capi.FP32))
    try:
        ctx.matmul(in_dtype, n, h, c, w, ta, tb, a_zp, b_zp, to)
        st = ctx.sync()
        return to.numpy(), st
    finally:
        for t in list(ctx._owned):
            ctx._free(t)


def rescale(ctx, x, mult, shift, in_zp=0, out_zp=0, out_dtype=np.int8, scale32=True,
            rounding_mode=capi.ROUND_DOUBLE, per_channel=True, input_unsigned=False, output_unsigned=False):
    x = np.asarray(x)
    od = np.dtype(out_dtype)
    mult, shift = np.atleast_1d(mult), np.atleast_1d(shift).astype(np.int8)
    rank = x.ndim
    C = x.shape[-1] if rank else 1
    rows = int(np.prod(x.shape[:-1], dtype=np.int64)) if rank else 1
    try:
        tx = ctx.upload(x)
        tm = ctx.upload(mult.astype(np.int32 if scale32 else np.int16))
        ts = ctx.upload(shift)
        to = ctx.empty(x.shape, _TMI[od], od)
        r = ctx.rescale_desc(_TMI[x.dtype], _TMI[od], mult.size, shift.size, in_zp, out_zp, scale32, rounding_mode,
                             per_channel, input_unsigned, output_unsigned)
        ctx.rescale(r, rank, rows, C, tx, tm, ts, to)
        st = ctx.sync()
        return to.numpy(), st
    finally:
        for t in list(ctx._owned):
            ctx._free(t)


def clamp(ctx, x, lo, hi):
    try:
        tx = ctx.upload(x)
        to = ctx.empty(x.shape, _TMI[x.dtype], x.dtype)
        ctx.clamp(_TMI[x.dtype], x.size, tx, lo, hi, to)
        st = ctx.sync()
        return to.numpy(), st
    finally:
        for t in list(ctx._owned):
            ctx._free(t)


def transpose_conv2d(ctx, x, w, bias, out_pad=(0, 0, 0, 0), stride=(1, 1), in_zp=0, w_zp=0, dtype=None, out_hw=None):
    """TRANSPOSE_CONV2D through the C ABI; returns (out, status)."""
    in_dtype = dtype or _TMI[x.dtype]
    n, ih, iw, ic = x.shape
    oc, kh, kw, _ = w.shape
    if out_hw is None:
        out_hw = ((ih - 1) * stride[0] + out_pad[0] + out_pad[1] + kh, (iw - 1) * stride[1] + out_pad[2] + out_pad[3] + kw)
    d = capi.TconvDesc()
    d.in_dtype = in_dtype
    d.out_dtype = capi.INT32 if in_dtype == capi.INT8 else (capi.INT48 if in_dtype == capi.INT16 else in_dtype)
    d.N, d.IH, d.IW, d.IC, d.OC, d.KH, d.KW = n, ih, iw, ic, oc, kh, kw
    d.OH, d.OW = out_hw
    d.out_pad[:], d.stride[:] = list(out_pad), list(stride)
    d.bias_len = bias.shape[0]
    # INT16 inputs come with INT8 weights and an INT48 bias (int64)
    tx, tw = ctx.upload(x, in_dtype), ctx.upload(w, capi.INT8 if in_dtype == capi.INT16 else in_dtype)
    tb = ctx.upload(bias, None if bias.dtype != np.uint16 else in_dtype)
    np_out = {capi.INT32: np.int32, capi.INT48: np.int64, capi.FP16: np.float16, capi.BF16: np.uint16, capi.FP32: np.float32}[d.out_dtype]
    try:
        to = ctx.empty((n, max(out_hw[0], 0), max(out_hw[1], 0), oc), d.out_dtype, np_out)
        ctx.transpose_conv2d(d, tx, tw, tb, in_zp, w_zp, to)
        st = ctx.sync()
        return to.numpy(), st
    finally:
        for t in list(ctx._owned):
            ctx._free(t)


def conv3d(ctx, x, w, bias, pad=(0,) * 6, stride=(1, 1, 1), dilation=(1, 1, 1), in_zp=0, w_zp=0, dtype=None,
           out_dhw=None):
    """CONV3D through the C ABI; returns (out, status)."""
    in_dtype = dtype or _TMI[x.dtype]
    n, idp, ih, iw, ic = x.shape
    oc, kd, kh, kw, _ = w.shape
    if out_dhw is None:
        out_dhw = oracle.conv3d_out_dhw((idp, ih, iw), (kd, kh, kw), pad, stride, dilation) or (0, 0, 0)
    d = capi.Conv3dDesc()
    d.in_dtype = in_dtype
    d.out_dtype = capi.INT32 if in_dtype == capi.INT8 else (capi.INT48 if in_dtype == capi.INT16 else in_dtype)
    d.N, d.ID, d.IH, d.IW, d.IC, d.OC, d.KD, d.KH, d.KW = n, idp, ih, iw, ic, oc, kd, kh, kw
    d.OD, d.OH, d.OW = out_dhw
    d.pad[:], d.stride[:], d.dilation[:] = list(pad), list(stride), list(dilation)
    d.bias_len = bias.shape[0]
    # INT16 inputs come with INT8 weights and an INT48 bias (int64)
    tx, tw = ctx.upload(x, in_dtype), ctx.upload(w, capi.INT8 if in_dtype == capi.INT16 else in_dtype)
    tb = ctx.upload(bias, None if bias.dtype != np.uint16 else in_dtype)
    np_out = {capi.INT32: np.int32, capi.INT48: np.int64, capi.FP16: np.float16, capi.BF16: np.uint16, capi.FP32: np.float32}[d.out_dtype]
    try:
        to = ctx.empty((n,) + tuple(out_dhw) + (oc,), d.out_dtype, np_out)
        ctx.conv3d(d, tx, tw, tb, in_zp, w_zp, to)
        st = ctx.sync()
        return to.numpy(), st
    finally:
        for t in list(ctx._owned):
            ctx._free(t)


def pool2d(ctx, x, kernel, stride=(1, 1), pad=(0, 0, 0, 0), avg=True, in_zp=0, out_zp=0, nan_mode=1, dtype=None,
           out_hw=None, acc_dtype=None):
    """AVG_POOL2D / MAX_POOL2D through the C ABI; returns (out, status).  bf16 travels as uint16 bit patterns."""
    np_to_tmi = {np.dtype(np.int8): capi.INT8, np.dtype(np.int16): capi.INT16, np.dtype(np.float16): capi.FP16,
                 np.dtype(np.float32): capi.FP32}
    tmi_dtype = dtype or np_to_tmi[x.dtype]
    n, ih, iw, c = x.shape
    if out_hw is None:
        out_hw = oracle.pool_out_hw(ih, iw, kernel, stride, pad) or (0, 0)
    d = capi.PoolDesc()
    d.dtype = tmi_dtype
    d.acc_dtype = acc_dtype if acc_dtype is not None else (capi.INT32 if tmi_dtype in (capi.INT8, capi.INT16) else capi.FP32)
    d.N, d.IH, d.IW, d.C = n, ih, iw, c
    d.OH, d.OW = out_hw
    d.kernel[:], d.stride[:], d.pad[:] = list(kernel), list(stride), list(pad)
    d.nan_mode = nan_mode
    tx = ctx.upload(x, tmi_dtype)
    try:
        to = ctx.empty((n, max(out_hw[0], 0), max(out_hw[1], 0), c), tmi_dtype, x.dtype)
        if avg:
            ctx.avg_pool2d(d, tx, in_zp, out_zp, to)
        else:
            ctx.max_pool2d(d, tx, to)
        st = ctx.sync()
        return to.numpy(), st
    finally:
        for t in list(ctx._owned):
            ctx._free(t)
