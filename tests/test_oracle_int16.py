"""The INT16 -> INT48 functions of the oracle, pinned without the reference's own vectors (its unit tests hold none for these
instantiations): independent numpy int64 formulations written per tap, the INT8 literal vectors of
tensor_ops_tests.cpp re-read as INT16 (the same numbers must come out wherever the input zero point is 0), and the
48-bit clip (tensor_ops.cpp:875-879, 1325-1329, 1485-1489) at both limits."""
import numpy as np
import pytest

import oracle


def _conv_numpy(x, w, bias, pad, stride, dil, w_zp):
    n, h, w_, ic = x.shape
    oc, kh, kw, _ = w.shape
    oh, ow = oracle.conv_out_hw(h, w_, kh, kw, pad, stride, dil)
    xp = np.pad(x.astype(np.int64), ((0, 0), (pad[0], pad[1]), (pad[2], pad[3]), (0, 0)))
    out = np.zeros((n, oh, ow, oc), np.int64)
    for ky in range(kh):
        for kx in range(kw):
            v = xp[:, ky * dil[0]: ky * dil[0] + (oh - 1) * stride[0] + 1: stride[0],
                   kx * dil[1]: kx * dil[1] + (ow - 1) * stride[1] + 1: stride[1], :]
            out += np.einsum("nhwc,oc->nhwo", v, w[:, ky, kx, :].astype(np.int64) - w_zp)
    return np.clip(out + bias.astype(np.int64), -(1 << 47), (1 << 47) - 1)


@pytest.mark.parametrize("geom", [(9, 10, (1, 1, 1, 1), (1, 1), (1, 1)), (10, 10, (0, 1, 2, 0), (2, 1), (1, 2)),
                                  (9, 11, (2, 2, 0, 0), (1, 3), (2, 1))])
def test_conv2d_i16_against_per_tap_numpy(geom):
    ih, iw, pad, stride, dil = geom
    rng = np.random.default_rng(sum(pad) + stride[0])
    x = rng.integers(-32768, 32768, (2, ih, iw, 6)).astype(np.int16)
    w = rng.integers(-128, 128, (5, 3, 2, 6)).astype(np.int8)
    bias = rng.integers(-(1 << 45), 1 << 45, 5).astype(np.int64)
    assert oracle.conv_out_hw(ih, iw, 3, 2, pad, stride, dil) is not None
    for w_zp in (0, 11):
        assert np.array_equal(oracle.conv2d("i16", x, w, bias, pad, stride, dil, w_zp=w_zp),
                              _conv_numpy(x, w, bias, pad, stride, dil, w_zp))


def test_depthwise_i16_against_per_tap_numpy():
    rng = np.random.default_rng(8)
    x = rng.integers(-32768, 32768, (2, 7, 8, 5)).astype(np.int16)
    w = rng.integers(-128, 128, (3, 3, 5, 2)).astype(np.int8)
    bias = rng.integers(-(1 << 30), 1 << 30, 10).astype(np.int64)
    xp = np.pad(x.astype(np.int64), ((0, 0), (1, 1), (1, 1), (0, 0)))
    want = np.zeros((2, 7, 8, 10), np.int64)
    for ky in range(3):
        for kx in range(3):
            prod = xp[:, ky:ky + 7, kx:kx + 8, :, None] * (w[ky, kx].astype(np.int64) - 4)[None, None, None]
            want += prod.reshape(2, 7, 8, 10)
    want += bias
    assert np.array_equal(oracle.depthwise_conv2d("i16", x, w, bias, (1, 1, 1, 1), w_zp=4), want)


def test_matmul_i16_against_numpy_and_the_transpose_identity():
    rng = np.random.default_rng(9)
    a = rng.integers(-32768, 32768, (3, 6, 50)).astype(np.int16)
    b = rng.integers(-32768, 32768, (3, 50, 4)).astype(np.int16)
    got = oracle.matmul("i16", a, b)
    assert np.array_equal(got, np.einsum("nhc,ncw->nhw", a.astype(np.int64), b.astype(np.int64)))
    assert np.array_equal(got.transpose(0, 2, 1), oracle.matmul("i16", b.transpose(0, 2, 1).copy(), a.transpose(0, 2, 1).copy()))


def test_int16_functions_give_the_int8_results_on_int8_numbers():
    """operands inside the INT8 range and a zero input zero point: the INT16 instantiation is the INT8 one with wider
    types (the INT8 one is pinned by the reference's literal vectors and its stored golden)"""
    rng = np.random.default_rng(10)
    x = rng.integers(-128, 128, (1, 6, 6, 8)).astype(np.int8)
    w = rng.integers(-128, 128, (4, 3, 3, 8)).astype(np.int8)
    bias = rng.integers(-1000, 1000, 4).astype(np.int32)
    assert np.array_equal(oracle.conv2d("i16", x.astype(np.int16), w, bias.astype(np.int64), (1, 1, 1, 1), w_zp=3),
                          oracle.conv2d("i8", x, w, bias, (1, 1, 1, 1), w_zp=3).astype(np.int64))
    wd = rng.integers(-128, 128, (3, 3, 8, 1)).astype(np.int8)
    bd = rng.integers(-1000, 1000, 8).astype(np.int32)
    assert np.array_equal(oracle.depthwise_conv2d("i16", x.astype(np.int16), wd, bd.astype(np.int64), (1, 1, 1, 1)),
                          oracle.depthwise_conv2d("i8", x, wd, bd, (1, 1, 1, 1)).astype(np.int64))
    a = rng.integers(-128, 128, (2, 5, 7)).astype(np.int8)
    b = rng.integers(-128, 128, (2, 7, 3)).astype(np.int8)
    assert np.array_equal(oracle.matmul("i16", a.astype(np.int16), b.astype(np.int16)),
                          oracle.matmul("i8", a, b).astype(np.int64))


def test_int48_clip_and_zero_point_rules():
    lim = (1 << 47) - 1
    x = np.full((1, 1, 1, 4096), -32768, np.int16)
    w = np.stack([np.full((1, 1, 4096), -128, np.int8), np.full((1, 1, 4096), 127, np.int8)])
    out = oracle.conv2d("i16", x, w, np.array([lim, -lim - 1], np.int64))
    assert out.ravel().tolist() == [lim, -lim - 1]
    out = oracle.conv2d("i16", x, w, np.array([0, 0], np.int64))    # 2^34 and -2^34 + ...: inside the range, untouched
    assert out.ravel().tolist() == [4096 * 32768 * 128, -4096 * 32768 * 127]
    with pytest.raises(oracle.OracleStatus):
        oracle.conv2d("i16", x, w, np.zeros(2, np.int64), in_zp=1)
    a = np.zeros((1, 2, 2), np.int16)
    with pytest.raises(oracle.OracleStatus):
        oracle.matmul("i16", a, a, b_zp=2)


def test_transpose_conv2d_and_conv3d_i16_against_independent_sums():
    """the INT16 forms of TRANSPOSE_CONV2D and CONV3D (tensor_ops.cpp:2237, 2291): the same loop-nest templates as the INT8
    functions at 64 bits.  Pins: the INT8 functions on operands that fit 8 bits; an independent scatter formulation of
    TRANSPOSE_CONV2D and a per-tap formulation of CONV3D in Python integers on full-range INT16 values; the 48-bit clip
    and the zero-point rule"""
    rng = np.random.default_rng(33)
    x = rng.integers(-32768, 32768, (2, 4, 5, 6)).astype(np.int16)
    w = rng.integers(-128, 128, (3, 3, 2, 6)).astype(np.int8)
    bias = rng.integers(-(1 << 40), 1 << 40, 3).astype(np.int64)
    out_pad, stride, w_zp = (1, 0, -1, 2), (2, 3), -5
    got = oracle.transpose_conv2d("i16", x, w, bias, out_pad, stride, w_zp=w_zp)
    n, ih, iw, ic = x.shape
    oc, kh, kw, _ = w.shape
    oh, ow = got.shape[1:3]
    want = np.zeros(got.shape, object)
    want[...] = [int(b) for b in bias]
    for b in range(n):
        for iy in range(ih):
            for ix in range(iw):
                for ky in range(kh):
                    for kx in range(kw):
                        oy, ox = iy * stride[0] + out_pad[0] + ky, ix * stride[1] + out_pad[2] + kx
                        if 0 <= oy < oh and 0 <= ox < ow:
                            for o in range(oc):
                                want[b, oy, ox, o] += sum(int(x[b, iy, ix, c]) * (int(w[o, ky, kx, c]) - w_zp) for c in range(ic))
    assert np.array_equal(got, want.astype(np.int64))
    x8 = rng.integers(-128, 128, x.shape).astype(np.int8)
    b32 = rng.integers(-999, 999, 3).astype(np.int32)
    assert np.array_equal(oracle.transpose_conv2d("i16", x8.astype(np.int16), w, b32.astype(np.int64), out_pad, stride, w_zp=w_zp),
                          oracle.transpose_conv2d("i8", x8, w, b32, out_pad, stride, w_zp=w_zp).astype(np.int64))

    x3 = rng.integers(-32768, 32768, (1, 4, 5, 4, 3)).astype(np.int16)
    w3 = rng.integers(-128, 128, (2, 2, 3, 2, 3)).astype(np.int8)
    b3 = rng.integers(-(1 << 40), 1 << 40, 2).astype(np.int64)
    pad, st3, dil = (1, 0, 1, 1, 0, 1), (1, 2, 1), (2, 1, 1)
    got3 = oracle.conv3d("i16", x3, w3, b3, pad, st3, dil, w_zp=4)
    _, idp, ih, iw, ic = x3.shape
    want3 = np.zeros(got3.shape, object)
    for od in range(got3.shape[1]):
        for oy in range(got3.shape[2]):
            for ox in range(got3.shape[3]):
                for o in range(2):
                    acc = int(b3[o])
                    for kd in range(2):
                        for ky in range(3):
                            for kx in range(2):
                                dd, yy, xx = od * st3[0] + kd * dil[0] - pad[0], oy * st3[1] + ky * dil[1] - pad[2], ox * st3[2] + kx * dil[2] - pad[4]
                                if 0 <= dd < idp and 0 <= yy < ih and 0 <= xx < iw:
                                    acc += sum(int(x3[0, dd, yy, xx, c]) * (int(w3[o, kd, ky, kx, c]) - 4) for c in range(ic))
                    want3[0, od, oy, ox, o] = acc
    assert np.array_equal(got3, want3.astype(np.int64))
    x38 = rng.integers(-128, 128, x3.shape).astype(np.int8)
    assert np.array_equal(oracle.conv3d("i16", x38.astype(np.int16), w3, b32[:2].astype(np.int64), pad, st3, dil, w_zp=4),
                          oracle.conv3d("i8", x38, w3, b32[:2], pad, st3, dil, w_zp=4).astype(np.int64))
    # the 48-bit clip (:1113-1117, :2190-2194) and the input zero point rule (:1031, :2115)
    lim = (1 << 47) - 1
    one = np.full((1, 1, 1, 8), 32767, np.int16)
    wt = np.full((1, 1, 1, 8), 127, np.int8)
    assert oracle.transpose_conv2d("i16", one, wt, np.array([lim], np.int64)).ravel().tolist() == [lim]
    assert oracle.conv3d("i16", one[None], wt[None], np.array([-lim - 1], np.int64), w_zp=127).ravel().tolist() == [-lim - 1]
    assert oracle.conv3d("i16", -one[None], wt[None], np.array([-lim - 1], np.int64)).ravel().tolist() == [-lim - 1]
    with pytest.raises(oracle.OracleStatus):
        oracle.transpose_conv2d("i16", one, wt, np.zeros(1, np.int64), in_zp=1)
    with pytest.raises(oracle.OracleStatus):
        oracle.conv3d("i16", one[None], wt[None], np.zeros(1, np.int64), in_zp=-1)
