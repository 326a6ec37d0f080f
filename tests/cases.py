"""Seeded synthetic operands for the benchmark configurations and for small parity cases.

Values are produced on the host by numpy's PCG64 seeded per configuration, so the oracle and the GPU see
identical bytes.
"""
from __future__ import annotations

import numpy as np

SEED = 0x705A5E75


def rng_for(config_id: int) -> np.random.Generator:
    return np.random.default_rng(SEED ^ config_id)


def c1():
    """INT8 CONV2D 1x1 [1,32,32,8] -> 16, RESCALE per-channel double-round to int8."""
    r = rng_for(1)
    return dict(
        x=r.integers(-128, 128, (1, 32, 32, 8)).astype(np.int8),
        w=r.integers(-127, 128, (16, 1, 1, 8)).astype(np.int8),
        bias=r.integers(-65536, 65537, 16).astype(np.int32),
        in_zp=-3, w_zp=0, pad=(0, 0, 0, 0), stride=(1, 1), dilation=(1, 1),
        mult=r.integers(1 << 30, 1 << 31, 16).astype(np.int32),
        shift=r.integers(36, 41, 16).astype(np.int8), out_zp=5, clamp=None)


def c2(n=8, h=1024, c=1024, w=1024):
    """INT8 batched MATMUL [8,1024,1024] x [8,1024,1024] -> int32, a_zp -5, b_zp 3."""
    r = rng_for(2)
    return dict(a=r.integers(-128, 128, (n, h, c)).astype(np.int8),
                b=r.integers(-128, 128, (n, c, w)).astype(np.int8), a_zp=-5, b_zp=3)


def c3(n=8, hw=56, ic=64, oc=64):
    """INT8 CONV2D ResNet-style 3x3 [8,56,56,64] -> 64, RESCALE shift 38 double-round, CLAMP [0,127]."""
    r = rng_for(3)
    return dict(
        x=r.integers(-128, 128, (n, hw, hw, ic)).astype(np.int8),
        w=np.clip(np.rint(r.normal(0, 30, (oc, 3, 3, ic))), -127, 127).astype(np.int8),
        bias=np.rint(r.normal(0, 2 ** 14, oc)).astype(np.int32),
        in_zp=-7, w_zp=0, pad=(1, 1, 1, 1), stride=(1, 1), dilation=(1, 1),
        mult=r.integers(1 << 30, 1 << 31, oc).astype(np.int32),
        shift=np.full(oc, 38, np.int8), out_zp=0, clamp=(0, 127))


def c4(n=8, hw=112, c=96, stride=2):
    """INT8 DEPTHWISE_CONV2D MobileNetV2-style [8,112,112,96], stride 2, pad [0,1,0,1], per-channel RESCALE
    (stride 1: pad 1 all round, the network's first depthwise layer when c is 32)."""
    r = rng_for(4)
    d = _c4(r, n, hw, c)
    if stride == 1:
        d.update(pad=(1, 1, 1, 1), stride=(1, 1))
    return d


def _c4(r, n, hw, c):
    return dict(
        x=r.integers(-128, 128, (n, hw, hw, c)).astype(np.int8),
        w=r.integers(-127, 128, (3, 3, c, 1)).astype(np.int8),
        bias=r.integers(-(1 << 15), (1 << 15) + 1, c).astype(np.int32),
        in_zp=4, w_zp=0, pad=(0, 1, 0, 1), stride=(2, 2), dilation=(1, 1),
        mult=r.integers(1 << 30, 1 << 31, c).astype(np.int32),
        shift=r.integers(34, 41, c).astype(np.int8), out_zp=0, clamp=None)


def c5_conv(n=16, hw=28, ic=256, oc=256):
    """FP16 CONV2D 3x3 [16,28,28,256] -> 256, fp32 accumulate."""
    r = rng_for(5)
    return dict(
        x=r.normal(0, 1, (n, hw, hw, ic)).astype(np.float16),
        w=r.normal(0, 1 / np.sqrt(9 * ic), (oc, 3, 3, ic)).astype(np.float16),
        bias=r.normal(0, 0.1, oc).astype(np.float16),
        pad=(1, 1, 1, 1), stride=(1, 1), dilation=(1, 1))


def float_to_bf16_bits(a: np.ndarray) -> np.ndarray:
    """Round-to-nearest-even float32 -> bfloat16 bit patterns (uint16)."""
    u = np.ascontiguousarray(a, np.float32).view(np.uint32).astype(np.uint64)
    r = (u + 0x7FFF + ((u >> 16) & 1)) >> 16
    return r.astype(np.uint16)


def bf16_bits_to_float(b: np.ndarray) -> np.ndarray:
    return (b.astype(np.uint32) << 16).view(np.float32)


def c5_matmul(n=4, h=2048, c=4096, w=2048):
    """BF16 MATMUL [4,2048,4096] x [4,4096,2048] -> fp32."""
    r = rng_for(6)
    a = float_to_bf16_bits(r.normal(0, 1 / 64, (n, h, c)).astype(np.float32))
    b = float_to_bf16_bits(r.normal(0, 1 / 64, (n, c, w)).astype(np.float32))
    return dict(a=a, b=b)


def conv2d_exact_blas(x, w, bias, pad, stride, dilation, in_zp=0, w_zp=0):
    """int8 CONV2D (NHWC x OHWI, int32 result) as one float64 BLAS product per kernel tap.  Every partial
    sum is an integer far below 2^53, so the float64 arithmetic is exact; the int32 result wraps like the
    accumulator of the oracle does.  For operands too large for the scalar oracle to finish in seconds;
    the CPU suite checks this helper against the oracle on small shapes."""
    n, ih, iw, ic = x.shape
    oc, kh, kw, _ = w.shape
    pt, pb, pl, pr = pad
    sy, sx = stride
    dy, dx = dilation
    oh = (ih - 1 + pt + pb - (kh - 1) * dy) // sy + 1
    ow = (iw - 1 + pl + pr - (kw - 1) * dx) // sx + 1
    xp = np.zeros((n, ih + pt + pb, iw + pl + pr, ic), np.float64)       # (x - in_zp), zero outside the image
    xp[:, pt:pt + ih, pl:pl + iw, :] = x.astype(np.float64) - in_zp
    wf = w.astype(np.float64) - w_zp
    acc = np.zeros((n * oh * ow, oc), np.float64)
    for ky in range(kh):
        for kx in range(kw):
            win = xp[:, ky * dy: ky * dy + (oh - 1) * sy + 1: sy, kx * dx: kx * dx + (ow - 1) * sx + 1: sx, :]
            acc += win.reshape(-1, ic) @ wf[:, ky, kx, :].T
    acc += (bias.astype(np.float64) if bias.shape[0] == oc else float(bias[0]))
    return acc.astype(np.int64).astype(np.int32).reshape(n, oh, ow, oc)
