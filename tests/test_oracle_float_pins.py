"""CPU pins of the oracle's floating-point MATMUL and DEPTHWISE_CONV2D (fp32 / fp64, ordinary and bounds pass) and of
the bounds pass without local_bound, against what the mathematics fixes: operands of small integers, for which every
product and sum is exact in fp32 and the result must equal the integer computation; random operands against an
independent numpy fp64 formulation; the bounds pass as the same operator on absolute values; the bounds pass of an
operator without local_bound as max|input| times the sum of |weights| over the taps inside the image."""
import numpy as np
import pytest

import oracle


def _dw_numpy(x, w, bias, pad, stride, dilation):
    """DEPTHWISE_CONV2D in fp64 by windows of a zero-padded copy (taps outside the image contribute nothing)"""
    n, ih, iw, c = x.shape
    kh, kw, _, m = w.shape
    pt, pb, pl, pr = pad
    oh = (ih - 1 + pt + pb - (kh - 1) * dilation[0]) // stride[0] + 1
    ow = (iw - 1 + pl + pr - (kw - 1) * dilation[1]) // stride[1] + 1
    xp = np.zeros((n, ih + pt + pb, iw + pl + pr, c))
    xp[:, pt:pt + ih, pl:pl + iw] = x
    out = np.zeros((n, oh, ow, c, m))
    for ky in range(kh):
        for kx in range(kw):
            win = xp[:, ky * dilation[0]: ky * dilation[0] + (oh - 1) * stride[0] + 1: stride[0],
                     kx * dilation[1]: kx * dilation[1] + (ow - 1) * stride[1] + 1: stride[1]]
            out += win[..., None] * w[ky, kx][None, None, None]
    b = bias if bias.shape[0] == c * m else np.full(c * m, bias[0])
    return out.reshape(n, oh, ow, c * m) + b


GEOMS = [((1, 1, 1, 1), (1, 1), (1, 1)), ((0, 1, 0, 1), (2, 2), (1, 1)), ((2, 2, 2, 2), (1, 1), (2, 2)),
         ((1, 0, 2, 1), (2, 1), (1, 1))]


@pytest.mark.parametrize("kind", ["f32", "f64"])
def test_matmul_float_exact_on_small_integers(kind):
    rng = np.random.default_rng(3)
    a = rng.integers(-9, 10, (3, 11, 37)).astype(np.float64)
    b = rng.integers(-9, 10, (3, 37, 13)).astype(np.float64)
    want = np.einsum("nhc,ncw->nhw", a.astype(np.int64), b.astype(np.int64))
    got = oracle.matmul(kind, a, b)
    assert got.dtype == (np.float32 if kind == "f32" else np.float64)
    assert np.array_equal(got.astype(np.int64), want) and np.array_equal(got, want.astype(got.dtype))
    # a transposed operand or a dropped term would show
    assert not np.array_equal(oracle.matmul(kind, a, b[:, ::-1]), got)


@pytest.mark.parametrize("kind,tol", [("f32", 2e-5), ("f64", 1e-13)])
def test_matmul_float_against_numpy_and_its_bounds_pass(kind, tol):
    rng = np.random.default_rng(4)
    a, b = rng.normal(0, 1, (2, 9, 64)), rng.normal(0, 1, (2, 64, 17))
    if kind == "f32":
        a, b = a.astype(np.float32).astype(np.float64), b.astype(np.float32).astype(np.float64)
    want = a @ b
    bound = np.abs(a) @ np.abs(b)
    got = oracle.matmul(kind, a, b).astype(np.float64)
    assert np.all(np.abs(got - want) <= tol * bound)
    if kind == "f64":
        got_b = oracle.matmul("f64", a, b, abs_mode=True)
        assert np.all(np.abs(got_b - bound) <= tol * bound) and np.all(got_b >= np.abs(want) * (1 - 1e-12))
        assert np.array_equal(got_b, oracle.matmul("f64", np.abs(a), np.abs(b)))


@pytest.mark.parametrize("kind", ["f32", "f64"])
@pytest.mark.parametrize("pad,stride,dilation", GEOMS)
def test_depthwise_float_exact_on_small_integers(kind, pad, stride, dilation):
    rng = np.random.default_rng(5)
    ih, iw = 9 + (stride[0] > 1), 8 + (stride[1] > 1)
    # shapes for which (I - 1 + pads - (K - 1) d) divides by the stride
    while (ih - 1 + pad[0] + pad[1] - 2 * dilation[0]) % stride[0]:
        ih += 1
    while (iw - 1 + pad[2] + pad[3] - 2 * dilation[1]) % stride[1]:
        iw += 1
    x = rng.integers(-9, 10, (2, ih, iw, 5)).astype(np.float64)
    w = rng.integers(-9, 10, (3, 3, 5, 2)).astype(np.float64)
    bias = rng.integers(-50, 50, 10).astype(np.float64)
    want = _dw_numpy(x, w, bias, pad, stride, dilation)
    got = oracle.depthwise_conv2d(kind, x, w, bias, pad, stride, dilation)
    assert np.array_equal(got.astype(np.float64), want)
    assert np.array_equal(oracle.depthwise_conv2d(kind, x, w, bias[:1], pad, stride, dilation).astype(np.float64),
                          _dw_numpy(x, w, bias[:1], pad, stride, dilation))


@pytest.mark.parametrize("pad,stride,dilation", GEOMS)
def test_depthwise_f64_random_and_bounds_passes(pad, stride, dilation):
    rng = np.random.default_rng(6)
    ih, iw = 10, 9
    while (ih - 1 + pad[0] + pad[1] - 2 * dilation[0]) % stride[0]:
        ih += 1
    while (iw - 1 + pad[2] + pad[3] - 2 * dilation[1]) % stride[1]:
        iw += 1
    x, w, bias = rng.normal(0, 1, (2, ih, iw, 6)), rng.normal(0, 1, (3, 3, 6, 1)), rng.normal(0, 1, 6)
    want = _dw_numpy(x, w, bias, pad, stride, dilation)
    assert np.allclose(oracle.depthwise_conv2d("f64", x, w, bias, pad, stride, dilation), want, rtol=0, atol=1e-12)
    assert np.allclose(oracle.depthwise_conv2d("f32", x, w, bias, pad, stride, dilation), want, rtol=0, atol=2e-5)
    # bounds pass: the operator on absolute values (tensor_ops.cpp:1245-1251)
    bnd = oracle.depthwise_conv2d("f64", x, w, bias, pad, stride, dilation, abs_mode=True)
    assert np.allclose(bnd, _dw_numpy(np.abs(x), np.abs(w), np.abs(bias), pad, stride, dilation), rtol=0, atol=1e-12)
    # without local_bound the input is one constant, its largest magnitude (:1252-1256): every output is that constant
    # times the sum of |w| over the taps inside the image, plus |bias|
    flat = oracle.depthwise_conv2d("f64", x, w, bias, pad, stride, dilation, abs_mode=True, local_bound=False)
    closed = _dw_numpy(np.full_like(x, np.abs(x).max()), np.abs(w), np.abs(bias), pad, stride, dilation)
    assert np.allclose(flat, closed, rtol=0, atol=1e-12) and np.all(flat >= bnd - 1e-12) and not np.allclose(flat, bnd)
    # the ordinary pass ignores the attribute
    assert np.array_equal(oracle.depthwise_conv2d("f64", x, w, bias, pad, stride, dilation, local_bound=False),
                          oracle.depthwise_conv2d("f64", x, w, bias, pad, stride, dilation))


@pytest.mark.parametrize("pad,stride,dilation", GEOMS)
def test_conv2d_f64_bounds_pass_without_local_bound(pad, stride, dilation):
    """tensor_ops.cpp:790-802: |w|, |bias|, and the input replaced by max|input| inside the image (the padding stays
    zero): out = max|x| * sum over the in-image taps of sum_ic |w| + |bias|"""
    rng = np.random.default_rng(7)
    ih, iw = 8, 11
    while (ih - 1 + pad[0] + pad[1] - 2 * dilation[0]) % stride[0]:
        ih += 1
    while (iw - 1 + pad[2] + pad[3] - 2 * dilation[1]) % stride[1]:
        iw += 1
    x, w, bias = rng.normal(0, 1, (2, ih, iw, 7)), rng.normal(0, 1, (4, 3, 3, 7)), rng.normal(0, 1, 4)
    flat = oracle.conv2d("f64", x, w, bias, pad, stride, dilation, abs_mode=True, local_bound=False)
    ones = np.ones((2, ih, iw, 1))
    taps = np.abs(w).sum(axis=3)[..., None]                      # [OC, KH, KW, 1]: sum over ic of |w|
    closed = np.abs(x).max() * (oracle.conv2d("f64", ones, taps, np.zeros(4), pad, stride, dilation)) + np.abs(bias)
    assert np.allclose(flat, closed, rtol=0, atol=1e-12)
    local = oracle.conv2d("f64", x, w, bias, pad, stride, dilation, abs_mode=True)
    assert np.all(flat >= local - 1e-12) and not np.allclose(flat, local)
    # an independent einsum for the local bound at an interior pixel
    if pad == (1, 1, 1, 1) and stride == (1, 1):
        patch = np.abs(x[0, 2:5, 3:6, :])
        assert abs(local[0, 3, 4, 1] - (np.einsum("yxc,yxc->", patch, np.abs(w[1])) + abs(bias[1]))) < 1e-12


def test_float_clamp_against_numpy_and_the_nan_rules():
    """activation_funcs.cpp:97-106 over applyClip (arith_util.h:390-413): max with min_val, then min with max_val;
    a NaN input stays NaN under PROPAGATE (1) and becomes min_val under IGNORE (2): applyMax(NaN, min) = min, and
    applyMin(min, max) = min"""
    rng = np.random.default_rng(3)
    x = np.concatenate([rng.normal(0, 3, 1000), [np.inf, -np.inf, 0.0, -0.0, 1.0, -1.0]]).astype(np.float32)
    for lo, hi in ((-1.0, 1.0), (0.0, 6.0), (-np.inf, np.inf), (2.5, 2.5)):
        for mode in (1, 2):
            assert np.array_equal(oracle.clamp(x, lo, hi, mode), np.clip(x, np.float32(lo), np.float32(hi)))
    xn = np.array([np.nan, 0.5, -7.0, np.nan, 9.0], np.float32)
    got = oracle.clamp(xn, -1.0, 2.0, 1)
    assert np.isnan(got[[0, 3]]).all() and np.array_equal(got[[1, 2, 4]], np.array([0.5, -1.0, 2.0], np.float32))
    assert np.array_equal(oracle.clamp(xn, -1.0, 2.0, 2), np.array([-1.0, 0.5, -1.0, -1.0, 2.0], np.float32))
    # the comparisons are (a >= min) ? a : min and (a < max) ? a : max: an input zero of either sign is kept when it
    # equals min, and replaced by max's own zero when it equals max
    z = oracle.clamp(np.array([-0.0, 0.0], np.float32), 0.0, 1.0, 1)
    assert np.signbit(z[0]) and not np.signbit(z[1])
    z = oracle.clamp(np.array([-0.0, 0.0], np.float32), -1.0, 0.0, 1)
    assert not np.signbit(z[0]) and not np.signbit(z[1])
    # half-precision storage: the result of clamping representable values to representable limits is representable
    h = rng.normal(0, 3, 500).astype(np.float16)
    assert np.array_equal(oracle.clamp(h, -1.5, 2.25, 1), np.clip(h, np.float16(-1.5), np.float16(2.25)))
    for bad in ((1.0, 0.0), (np.nan, 1.0), (0.0, np.nan)):
        with pytest.raises(oracle.OracleStatus):
            oracle.clamp(x, bad[0], bad[1], 1)
