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
