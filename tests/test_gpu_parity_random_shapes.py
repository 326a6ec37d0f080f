"""Seeded random geometries through the two kernels that load their operands straight into LDS (the CONV2D slab
kernel, with its TRANSPOSE_CONV2D and CONV3D addressing, and the matrix-core DEPTHWISE_CONV2D kernel): the tile search, the padded LDS pitches and the incremental
source walks depend on the geometry in ways a hand-picked list does not exhaust.  Integer work: bit for bit against
the CPU oracle."""
import numpy as np
import pytest

import gpu_ops
import oracle
from reference_model_amd import Context, capi

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def ctx():
    c = Context(0)
    c.set_kernel_choice(capi.KERNEL_SLAB)
    yield c
    c.close()


def _geometry(rng):
    """a legal (ih, iw, pad, stride, dilation) for 3x3 taps: (ih - 1 + pad - 2 * dilation) % stride == 0"""
    while True:
        stride = (int(rng.integers(1, 4)), int(rng.integers(1, 4)))
        dil = (int(rng.integers(1, 3)), int(rng.integers(1, 3)))
        pad = tuple(int(v) for v in rng.integers(0, 3, 4))
        oh, ow = int(rng.integers(1, 40)), int(rng.integers(1, 40))
        ih = (oh - 1) * stride[0] + 2 * dil[0] + 1 - pad[0] - pad[1]
        iw = (ow - 1) * stride[1] + 2 * dil[1] + 1 - pad[2] - pad[3]
        if ih >= 1 and iw >= 1:
            return ih, iw, pad, stride, dil


@pytest.mark.parametrize("seed", range(24))
def test_conv2d_slab_random_geometry(ctx, seed):
    rng = np.random.default_rng(1000 + seed)
    ih, iw, pad, stride, dil = _geometry(rng)
    n, ic = int(rng.integers(1, 5)), int(rng.choice([64, 96, 128]))
    oc = 16 * int(rng.integers(3, 11))
    in_zp = int(rng.integers(-128, 128))
    x = rng.integers(-128, 128, (n, ih, iw, ic)).astype(np.int8)
    w = rng.integers(-128, 128, (oc, 3, 3, ic)).astype(np.int8)
    bias = rng.integers(-(1 << 18), 1 << 18, oc).astype(np.int32)
    acc = oracle.conv2d("i8", x, w, bias, pad, stride, dil, in_zp=in_zp, w_zp=0)
    got, st = gpu_ops.conv2d(ctx, x, w, bias, pad, stride, dil, in_zp=in_zp, w_zp=0)
    assert st == capi.VALID and ctx.last_kernel == "conv2d_slab_i8"
    assert np.array_equal(got, acc), (ih, iw, ic, oc, pad, stride, dil)
    mult = rng.integers(1 << 30, 1 << 31, oc).astype(np.int32)
    shift = rng.integers(37, 45, oc).astype(np.int8) if seed % 3 else np.full(oc, 41, np.int8)
    out_zp = int(rng.integers(-20, 20))
    got, st = gpu_ops.conv2d(ctx, x, w, bias, pad, stride, dil, in_zp=in_zp, w_zp=0,
                             rescale=dict(mult=mult, shift=shift, out_zp=out_zp), clamp=(-120, 120))
    want, wst = oracle.rescale(acc, mult, shift, out_zp=out_zp)
    assert st == wst == capi.VALID
    assert ctx.last_kernel == ("conv2d_slab_wreg_i8_rescale" if ic == 64 and stride == (1, 1) else "conv2d_slab_i8_rescale")
    assert np.array_equal(got, oracle.clamp(want, -120, 120)), (ih, iw, ic, oc, pad, stride, dil)


@pytest.mark.parametrize("seed", range(24))
def test_depthwise_mfma_random_geometry(ctx, seed):
    rng = np.random.default_rng(2000 + seed)
    ih, iw, pad, stride, dil = _geometry(rng)
    n, c = int(rng.integers(1, 5)), 16 * int(rng.integers(2, 21))
    in_zp = int(rng.integers(-128, 128))
    x = rng.integers(-128, 128, (n, ih, iw, c)).astype(np.int8)
    w = rng.integers(-128, 128, (3, 3, c, 1)).astype(np.int8)
    bias = rng.integers(-(1 << 16), 1 << 16, c).astype(np.int32)
    acc = oracle.depthwise_conv2d("i8", x, w, bias, pad, stride, dil, in_zp=in_zp, w_zp=0)
    got, st = gpu_ops.conv2d(ctx, x, w, bias, pad, stride, dil, in_zp=in_zp, w_zp=0, depthwise=True)
    assert st == capi.VALID and ctx.last_kernel in ("depthwise_mfma_i8", "depthwise_mfma_pipe_i8")
    assert np.array_equal(got, acc), (ih, iw, c, pad, stride, dil)
    mult = rng.integers(1 << 30, 1 << 31, c).astype(np.int32)
    shift = rng.integers(33, 40, c).astype(np.int8) if seed % 3 else np.full(c, 35, np.int8)
    out_zp = int(rng.integers(-20, 20))
    got, st = gpu_ops.conv2d(ctx, x, w, bias, pad, stride, dil, in_zp=in_zp, w_zp=0, depthwise=True,
                             rescale=dict(mult=mult, shift=shift, out_zp=out_zp))
    want, wst = oracle.rescale(acc, mult, shift, out_zp=out_zp)
    assert st == wst == capi.VALID and ctx.last_kernel in ("depthwise_mfma_i8_rescale", "depthwise_mfma_pipe_i8_rescale")
    assert np.array_equal(got, want), (ih, iw, c, pad, stride, dil)


@pytest.mark.parametrize("seed", range(16))
def test_transpose_conv2d_slab_random_geometry(ctx, seed):
    """holes and flipped taps as part of the kernel's addressing: strides 1..3, out_pad from -2 (cropping) to 2"""
    rng = np.random.default_rng(3000 + seed)
    stride = (int(rng.integers(1, 4)), int(rng.integers(1, 4)))
    n, ih, iw = int(rng.integers(1, 4)), int(rng.integers(2, 17)), int(rng.integers(2, 17))
    ic, oc = int(rng.choice([64, 96, 128])), 16 * int(rng.integers(3, 9))
    out_pad = tuple(int(v) for v in rng.integers(-2, 3, 4))
    in_zp = int(rng.integers(-128, 128))
    x = rng.integers(-128, 128, (n, ih, iw, ic)).astype(np.int8)
    w = rng.integers(-128, 128, (oc, 3, 3, ic)).astype(np.int8)
    bias = rng.integers(-(1 << 18), 1 << 18, oc).astype(np.int32)
    want = oracle.transpose_conv2d("i8", x, w, bias, out_pad, stride, in_zp, 0)
    got, st = gpu_ops.transpose_conv2d(ctx, x, w, bias, out_pad, stride, in_zp, 0)
    assert st == capi.VALID and ctx.last_kernel == "transpose_conv2d_slab_i8"
    assert np.array_equal(got, want), (n, ih, iw, ic, oc, out_pad, stride)


@pytest.mark.parametrize("seed", range(16))
def test_conv3d_slab_random_geometry(ctx, seed):
    """depth taps as part of the kernel's addressing: 2..4 depth taps of 32 channels or 2 of 64, any depth stride,
    dilation and padding"""
    rng = np.random.default_rng(4000 + seed)
    ic, kd = [(32, 2), (32, 3), (32, 4), (64, 2)][int(rng.integers(0, 4))]
    while True:
        stride = tuple(int(v) for v in rng.integers(1, 3, 3))
        dil = (int(rng.integers(1, 3)), 1, 1)
        pad = tuple(int(v) for v in rng.integers(0, 3, 6))
        od, oh, ow = int(rng.integers(1, 7)), int(rng.integers(1, 13)), int(rng.integers(1, 13))
        idp = (od - 1) * stride[0] + (kd - 1) * dil[0] + 1 - pad[0] - pad[1]
        ih = (oh - 1) * stride[1] + 3 - pad[2] - pad[3]
        iw = (ow - 1) * stride[2] + 3 - pad[4] - pad[5]
        if idp >= 1 and ih >= 1 and iw >= 1:
            break
    n, oc = int(rng.integers(1, 3)), 16 * int(rng.integers(3, 9))
    in_zp = int(rng.integers(-128, 128))
    x = rng.integers(-128, 128, (n, idp, ih, iw, ic)).astype(np.int8)
    w = rng.integers(-128, 128, (oc, kd, 3, 3, ic)).astype(np.int8)
    bias = rng.integers(-(1 << 18), 1 << 18, oc).astype(np.int32)
    want = oracle.conv3d("i8", x, w, bias, pad, stride, dil, in_zp, 0)
    got, st = gpu_ops.conv3d(ctx, x, w, bias, pad, stride, dil, in_zp, 0)
    assert st == capi.VALID and ctx.last_kernel == "conv3d_slab_i8"
    assert np.array_equal(got, want), (n, idp, ih, iw, ic, oc, kd, pad, stride, dil)
