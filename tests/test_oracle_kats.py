"""Known-answer and closed-form pins for the CPU oracle (no GPU).

Sources of the expected values:
  * the literal vectors of reference_model/test/ref_model_tests/tensor_ops_tests.cpp:622-683 (zero
    points) and :736-798 (bias broadcast, literal expected numbers);
  * reference_model/test/ref_model_tests/type_conversion_tests.cpp:324-405 (RESCALE literals and the
    four shape negatives);
  * Python arbitrary-precision integers for apply_scale_32 / apply_scale_16 (floor shift), which do not
    share the oracle's int64 code;
  * independent numpy formulations (int64 einsum over an explicitly gathered patch tensor) for shapes
    with padding, stride and dilation.
"""
import numpy as np
import pytest

import oracle

ZP_CASES = [  # (inVals, weightVals, inZp, weightZp, expected): tensor_ops_tests.cpp:622-683
    ([126, -126, -120, 0], [2, 1, 4, -7], 4, 15, 122 * -13 + -130 * -14 + -124 * -11 + -4 * -22),
    ([122, -7, -120, 121], [2, 1, 4, -7], -10, -5, 132 * 7 + 3 * 6 + -110 * 9 + 131 * -2),
    ([3, -12, 5, 70], [-120, -12, 0, -7], 55, 15, -52 * -135 + -67 * -27 + -50 * -15 + 15 * -22),
    ([-5, 65, -1, 32], [-2, 125, 4, -1], -10, -5, 5 * 3 + 75 * 130 + 9 * 9 + 42 * 4),
]


@pytest.mark.parametrize("inv,wv,izp,wzp,want", ZP_CASES)
def test_conv2d_zero_points(inv, wv, izp, wzp, want):
    x = np.array(inv, np.int8).reshape(1, 2, 2, 1)
    w = np.array(wv, np.int8).reshape(1, 2, 2, 1)
    out = oracle.conv2d("i8", x, w, np.zeros(1, np.int32), stride=(2, 2), in_zp=izp, w_zp=wzp)
    assert out.shape == (1, 1, 1, 1) and int(out.ravel()[0]) == want


@pytest.mark.parametrize("inv,wv,izp,wzp,want", ZP_CASES)
def test_depthwise_zero_points(inv, wv, izp, wzp, want):
    x = np.array(inv, np.int8).reshape(1, 2, 2, 1)
    w = np.array(wv, np.int8).reshape(2, 2, 1, 1)
    out = oracle.depthwise_conv2d("i8", x, w, np.zeros(1, np.int32), stride=(2, 2), in_zp=izp, w_zp=wzp)
    assert int(out.ravel()[0]) == want


@pytest.mark.parametrize("inv,wv,izp,wzp,_", ZP_CASES)
def test_matmul_zero_points(inv, wv, izp, wzp, _):
    a = np.array(inv, np.int8).reshape(1, 2, 2)
    b = np.array(wv, np.int8).reshape(1, 2, 2)
    want = (a.astype(np.int64) - izp) @ (b.astype(np.int64) - wzp)
    assert np.array_equal(oracle.matmul("i8", a, b, izp, wzp), want)


def test_conv2d_bias_broadcast_literals():  # tensor_ops_tests.cpp:736-766
    x = np.array([5, 9], np.int8).reshape(1, 1, 1, 2)
    w = np.array([3, -7, -1, 4], np.int8).reshape(2, 1, 1, 2)
    assert oracle.conv2d("i8", x, w, np.array([-5], np.int32)).ravel().tolist() == [-53, 26]
    assert oracle.conv2d("i8", x, w, np.array([-5, 14], np.int32)).ravel().tolist() == [-53, 45]


def test_depthwise_bias_broadcast_literals():  # tensor_ops_tests.cpp:768-798
    x = np.array([5, 9], np.int8).reshape(1, 1, 1, 2)
    w = np.array([3, -7], np.int8).reshape(1, 1, 2, 1)
    assert oracle.depthwise_conv2d("i8", x, w, np.array([-5], np.int32)).ravel().tolist() == [10, -68]
    assert oracle.depthwise_conv2d("i8", x, w, np.array([-5, 14], np.int32)).ravel().tolist() == [10, -49]


def test_conv_shape_rule_rejects_inexact_and_mismatched_outputs():
    x = np.zeros((1, 5, 5, 1), np.int8)
    w = np.zeros((1, 2, 2, 1), np.int8)
    with pytest.raises(oracle.OracleStatus) as e:  # (5-1-1) % 2 != 0
        oracle.conv2d("i8", x, w, np.zeros(1, np.int32), stride=(2, 2))
    assert e.value.status == oracle.ERROR
    with pytest.raises(oracle.OracleStatus):
        oracle.conv2d("i8", x, w, np.zeros(1, np.int32), out_hw=(3, 4))
    with pytest.raises(oracle.OracleStatus):  # bias neither 1 nor OC
        oracle.conv2d("i8", x, np.zeros((3, 2, 2, 1), np.int8), np.zeros(2, np.int32))
    with pytest.raises(oracle.OracleStatus):  # negative pad
        oracle.conv2d("i8", x, w, np.zeros(1, np.int32), pad=(-1, 1, 0, 0))


# ---------------------------------------------------------------------------------------------
# apply_scale_32 / apply_scale_16 against arbitrary-precision integers
# ---------------------------------------------------------------------------------------------
def _scale32_bigint(v, m, s, dr):
    if m < 0 or s < 2 or s > 62 or not (-(1 << (s - 1)) <= v < (1 << (s - 1))):
        return None
    rnd = 1 << (s - 1)
    if dr and s > 31:
        rnd += (1 << 30) if v >= 0 else -(1 << 30)
    r = (v * m + rnd) >> s  # Python's >> floors, like an arithmetic shift
    return r if -(1 << 31) <= r < (1 << 31) else None


def test_apply_scale_32_brute_force():
    rng = np.random.default_rng(1234)
    cases = []
    for s in (2, 3, 15, 30, 31, 32, 33, 38, 40, 47, 61, 62):
        lim = min(1 << 31, 1 << (s - 1))
        vs = [0, 1, -1, 2, -2, lim - 1, -lim, lim, -lim - 1, 12345, -12345]
        vs += rng.integers(-lim, lim, 40).tolist()
        ms = [0, 1, (1 << 30), (1 << 30) + 1, (1 << 31) - 1, -1] + rng.integers(1 << 30, 1 << 31, 8).tolist()
        for v in vs:
            if not -(1 << 31) <= v < (1 << 31):
                continue
            for m in ms:
                for dr in (False, True):
                    cases.append((v, m, s, dr))
    bad = 0
    for v, m, s, dr in cases:
        want = _scale32_bigint(v, m, s, dr)
        got, st = oracle.apply_scale_32(v, m, s, dr)
        if want is None:
            bad += st != oracle.UNPREDICTABLE
        else:
            bad += not (st == oracle.VALID and got == want)
    assert bad == 0 and len(cases) > 5000


def test_apply_scale_32_rejects_bad_shift():
    for s in (-1, 0, 1, 63, 64):
        assert oracle.apply_scale_32(1, 1 << 30, s, True)[1] == oracle.UNPREDICTABLE


def test_apply_scale_32_reference_hand_expansion():
    # tensor_ops_tests.cpp:552-564: multiplier 2^30+1, shift 32, single round, written out by hand there
    for total in (-7, 0, 5, 493, -511):
        want = (total * ((1 << 30) + 1) + (1 << 31)) >> 32
        assert oracle.apply_scale_32(total, (1 << 30) + 1, 32, False) == (want, oracle.VALID)


def test_apply_scale_32_special_operands():
    # generate_int_special.cpp:119-131: value {-2, 1, lowest, max} x multiplier {0, max} x shift {2, 62}
    i32max, i32min = (1 << 31) - 1, -(1 << 31)
    for v, m, s in [(-2, 0, 2), (-2, i32max, 2), (1, 0, 2), (1, i32max, 2), (i32min, 0, 62), (i32min, i32max, 62),
                    (i32max, 0, 62), (i32max, i32max, 62)]:
        for dr in (False, True):
            want = _scale32_bigint(v, m, s, dr)
            got, st = oracle.apply_scale_32(v, m, s, dr)
            assert (st, got) == ((oracle.VALID, want) if want is not None else (oracle.UNPREDICTABLE, 0))


def test_apply_scale_16_brute_force():
    rng = np.random.default_rng(7)
    for _ in range(3000):
        s = int(rng.integers(2, 63))
        v = int(rng.integers(-(1 << 47), 1 << 47))
        m = int(rng.integers(0, 1 << 15))
        r = (v * m + (1 << (s - 1))) >> s
        got, st = oracle.apply_scale_16(v, m, s)
        if -(1 << 31) <= r < (1 << 31):
            assert (got, st) == (r, oracle.VALID)
        else:
            assert st == oracle.UNPREDICTABLE


# ---------------------------------------------------------------------------------------------
# RESCALE operator
# ---------------------------------------------------------------------------------------------
def test_rescale_output_zp_extension():  # type_conversion_tests.cpp:324-335
    out, st = oracle.rescale(np.array([65], np.int8), [4], [2], in_zp=1, out_zp=32768, out_dtype=np.uint16,
                             scale32=False, rounding_mode=oracle.ROUND_SINGLE, per_channel=False,
                             output_unsigned=True)
    assert st == oracle.VALID and out.tolist() == [32832]


def test_rescale_inexact_round_literals():  # type_conversion_tests.cpp:385-405
    out, st = oracle.rescale(np.array([65], np.int8), [4], [2], in_zp=1, out_zp=32768, out_dtype=np.uint16,
                             scale32=False, rounding_mode=oracle.ROUND_INEXACT, per_channel=False,
                             output_unsigned=True)
    assert st == oracle.VALID and out.tolist() == [32832]
    out, st = oracle.rescale(np.array([103], np.int8), [147], [8], in_zp=-95, out_zp=0, out_dtype=np.uint8,
                             scale32=False, rounding_mode=oracle.ROUND_INEXACT, per_channel=False,
                             output_unsigned=True)
    assert st == oracle.VALID and out.tolist() == [114]


def test_rescale_inexact_round_is_float_arithmetic_and_beyond_int32_reference_undefined_x86_64_convention():
    """INEXACT_ROUND is float(value) * float(multiplier) * 2^-shift rounded to nearest even (type_conversion.cpp:320-323),
    checked against numpy float32; a product outside int32 makes the reference's cast undefined, and the value its
    x86-64 builds return, INT32_MIN, is what the oracle states"""
    rng = np.random.default_rng(5)
    x = rng.integers(-(1 << 20), 1 << 20, (50, 8)).astype(np.int32)
    mult = rng.integers(1 << 30, 1 << 31, 8).astype(np.int32)
    shift = rng.integers(30, 45, 8).astype(np.int32)
    out, st = oracle.rescale(x, mult, shift, out_dtype=np.int32, rounding_mode=oracle.ROUND_INEXACT)
    want = np.rint((x.astype(np.float32) * mult.astype(np.float32)) * np.exp2(-shift.astype(np.float32)))
    assert st == oracle.VALID and np.array_equal(out, want.astype(np.int64))
    big = np.array([[(1 << 31) - 1, -(1 << 31), 100000, -100000, 8192, 3]], np.int32)
    out, st = oracle.rescale(big, [1803664250], [12], out_dtype=np.int32, rounding_mode=oracle.ROUND_INEXACT,
                             per_channel=False)
    assert st == oracle.VALID and out.tolist() == [[-(1 << 31)] * 5 + [1321043]]


@pytest.mark.parametrize("inp,mult,shift,kw", [  # type_conversion_tests.cpp:337-383
    (np.array([20, -5, -16], np.int8), [4, 2], [16, 5, 9], dict(scale32=True, per_channel=True, in_zp=-19,
                                                                  out_dtype=np.int32)),
    (np.array([0, -12, 0, 12], np.int32), [4, 1024, 2048, 115], [12], dict(scale32=False, per_channel=True,
                                                                            out_zp=-12, out_dtype=np.int8)),
    (np.array([20, -5, -16], np.int8), [4, 519], [12], dict(scale32=True, per_channel=False, in_zp=-19,
                                                             out_dtype=np.int32)),
    (np.array([0, -12, 0, 12], np.int32), [4], [6, 16], dict(scale32=False, per_channel=False, out_zp=-12,
                                                              out_dtype=np.int8)),
])
def test_rescale_shape_negatives_are_errors(inp, mult, shift, kw):
    _, st = oracle.rescale(inp, mult, shift, rounding_mode=oracle.ROUND_SINGLE, **kw)
    assert st == oracle.ERROR


def test_rescale_attribute_negatives():
    x = np.array([1, 2], np.int32)
    assert oracle.rescale(x, [1 << 30], [31], per_channel=False, scale32=False,
                          rounding_mode=oracle.ROUND_DOUBLE)[1] == oracle.ERROR
    assert oracle.rescale(x, [1 << 30], [31], per_channel=False, output_unsigned=True)[1] == oracle.ERROR
    assert oracle.rescale(x, [1 << 30], [31], per_channel=False, in_zp=3)[1] == oracle.ERROR  # int32 in_zp != 0
    assert oracle.rescale(x, [1 << 30], [31], per_channel=False, rounding_mode=7)[1] == oracle.ERROR
    x8 = np.array([1, 2], np.int8)
    assert oracle.rescale(x8, [1 << 30], [31], per_channel=False, input_unsigned=True,
                          output_unsigned=True)[1] == oracle.ERROR


def test_rescale_per_channel_random_vs_bigint():
    rng = np.random.default_rng(99)
    C = 7
    x = rng.integers(-(1 << 24), 1 << 24, (5, 3, C)).astype(np.int32)
    mult = rng.integers(1 << 30, 1 << 31, C)
    shift = rng.integers(33, 45, C)
    for mode in (oracle.ROUND_SINGLE, oracle.ROUND_DOUBLE):
        out, st = oracle.rescale(x, mult, shift, out_zp=5, out_dtype=np.int8, rounding_mode=mode)
        want = np.empty_like(x)
        for idx in np.ndindex(x.shape):
            c = idx[-1]
            r = _scale32_bigint(int(x[idx]), int(mult[c]), int(shift[c]), mode == oracle.ROUND_DOUBLE)
            want[idx] = min(127, max(-128, r + 5))
        assert st == oracle.VALID and np.array_equal(out, want.astype(np.int8))


def test_rescale_value_out_of_range_is_unpredictable():
    # shift 20 admits |v| < 2^19 only (quant_util.h:59-67)
    x = np.array([1 << 19], np.int32)
    assert oracle.rescale(x, [1 << 30], [20], per_channel=False, out_dtype=np.int32)[1] == oracle.UNPREDICTABLE
    x = np.array([(1 << 19) - 1], np.int32)
    assert oracle.rescale(x, [1 << 30], [20], per_channel=False, out_dtype=np.int32)[1] == oracle.VALID


def test_rescale_unsigned_input_and_rank0():
    out, st = oracle.rescale(np.array(200, np.uint8), [1 << 30], [30], in_zp=128, out_dtype=np.int8,
                             rounding_mode=oracle.ROUND_SINGLE, per_channel=False, input_unsigned=True)
    assert st == oracle.VALID and out.shape == () and int(out) == 72


def test_rescale_int48_vs_bigint():
    """INT48 input: int64 storage, 16-bit multipliers, apply_scale_16 (quant_util.h:86-108): with Python's
    unbounded integers ((v * m + 2^(s-1)) >> s), results beyond int32 being REQUIRE failures"""
    rng = np.random.default_rng(48)
    C = 5
    x = rng.integers(-(1 << 47), 1 << 47, (4, 6, C)).astype(np.int64)
    x[0, 0, :] = [(1 << 47) - 1, -(1 << 47), 0, -1, 1]                 # the extremes of the type
    mult = rng.integers(1, 1 << 15, C)
    shift = rng.integers(40, 63, C)
    for out_dtype, lo, hi in ((np.int8, -128, 127), (np.int16, -32768, 32767), (np.int32, -(1 << 31), (1 << 31) - 1)):
        out, st = oracle.rescale(x, mult, shift, out_dtype=out_dtype, scale32=False, rounding_mode=oracle.ROUND_SINGLE)
        want = np.empty(x.shape, np.int64)
        for idx in np.ndindex(x.shape):
            c = idx[-1]
            r = (int(x[idx]) * int(mult[c]) + (1 << (int(shift[c]) - 1))) >> int(shift[c])
            assert -(1 << 31) <= r < (1 << 31)
            want[idx] = min(hi, max(lo, r))
        assert st == oracle.VALID and np.array_equal(out, want.astype(out_dtype))
    assert len(np.unique(out)) > 40


def test_rescale_int48_boundary_operands():
    """rescaleTestVals (generate_int_special.cpp:119-131) for INT48: value x multiplier x shift extremes"""
    lowest, top, mmax = -(1 << 47), (1 << 47) - 1, (1 << 15) - 1
    for v, m, s in [(-2, 0, 2), (-2, mmax, 2), (1, 0, 2), (1, mmax, 2), (lowest, 0, 62), (lowest, mmax, 62),
                    (top, 0, 62), (top, mmax, 62)]:
        out, st = oracle.rescale(np.array([v], np.int64), [m], [s], out_dtype=np.int32, scale32=False,
                                 rounding_mode=oracle.ROUND_SINGLE, per_channel=False)
        assert st == oracle.VALID and int(out[0]) == (v * m + (1 << (s - 1))) >> s, (v, m, s)
    # a result beyond int32 is a REQUIRE failure (quant_util.h:102-106)
    _, st = oracle.rescale(np.array([top], np.int64), [mmax], [20], out_dtype=np.int32, scale32=False,
                           rounding_mode=oracle.ROUND_SINGLE, per_channel=False)
    assert st == oracle.UNPREDICTABLE


def test_rescale_int48_attribute_negatives():
    """type_conversion.cpp:122 (scale32), :129 (output_unsigned), :132 (input_unsigned), :242 (input_zp)"""
    x = np.array([1, 2], np.int64)
    kw = dict(per_channel=False, rounding_mode=oracle.ROUND_SINGLE, out_dtype=np.int16)
    assert oracle.rescale(x, [1 << 14], [20], scale32=False, **kw)[1] == oracle.VALID
    assert oracle.rescale(x, [1 << 30], [40], scale32=True, **kw)[1] == oracle.ERROR
    assert oracle.rescale(x, [1 << 14], [20], scale32=False, input_unsigned=True, **kw)[1] == oracle.ERROR
    assert oracle.rescale(x, [1 << 14], [20], scale32=False, in_zp=3, **kw)[1] == oracle.ERROR
    kw["out_dtype"] = np.uint16
    assert oracle.rescale(x, [1 << 14], [20], scale32=False, output_unsigned=True, **kw)[1] == oracle.ERROR


def test_clamp_int8():
    x = np.arange(-128, 128).astype(np.int8)
    assert np.array_equal(oracle.clamp(x, 0, 127), np.clip(x, 0, 127))
    with pytest.raises(oracle.OracleStatus):
        oracle.clamp(x, 5, 4)


# ---------------------------------------------------------------------------------------------
# Independent numpy formulation for general shapes
# ---------------------------------------------------------------------------------------------
def _np_conv(x, w, bias, pad, stride, dil, izp, wzp):
    n, ih, iw, ic = x.shape
    oc, kh, kw, _ = w.shape
    oh, ow = oracle.conv_out_hw(ih, iw, kh, kw, pad, stride, dil)
    xp = np.full((n, ih + pad[0] + pad[1], iw + pad[2] + pad[3], ic), izp, np.int64)
    xp[:, pad[0]:pad[0] + ih, pad[2]:pad[2] + iw] = x
    patches = np.empty((n, oh, ow, kh, kw, ic), np.int64)
    for ky in range(kh):
        for kx in range(kw):
            patches[:, :, :, ky, kx] = xp[:, ky * dil[0]:ky * dil[0] + (oh - 1) * stride[0] + 1:stride[0],
                                          kx * dil[1]:kx * dil[1] + (ow - 1) * stride[1] + 1:stride[1]]
    out = np.einsum("nhwyxc,oyxc->nhwo", patches - izp, w.astype(np.int64) - wzp)
    return out + (bias.astype(np.int64) if bias.size > 1 else int(bias[0]))


CONV_SHAPES = [  # n, ih, iw, ic, oc, kh, kw, pad, stride, dilation
    (1, 8, 8, 3, 5, 3, 3, (1, 1, 1, 1), (1, 1), (1, 1)),
    (2, 10, 11, 4, 6, 3, 2, (0, 1, 2, 0), (2, 1), (1, 1)),
    (1, 12, 10, 2, 3, 3, 3, (2, 2, 2, 2), (1, 1), (2, 2)),
    (3, 7, 7, 16, 8, 1, 1, (0, 0, 0, 0), (2, 2), (1, 1)),
    (1, 11, 44, 13, 7, 2, 4, (1, 0, 0, 2), (1, 3), (1, 1)),
]


@pytest.mark.parametrize("shape", CONV_SHAPES)
def test_conv2d_i8_vs_numpy_einsum(shape):
    n, ih, iw, ic, oc, kh, kw, pad, stride, dil = shape
    rng = np.random.default_rng(sum(shape[:7]))
    x = rng.integers(-128, 128, (n, ih, iw, ic)).astype(np.int8)
    w = rng.integers(-127, 128, (oc, kh, kw, ic)).astype(np.int8)
    for bias in (rng.integers(-65536, 65536, oc).astype(np.int32), np.array([77], np.int32)):
        got = oracle.conv2d("i8", x, w, bias, pad, stride, dil, in_zp=-7, w_zp=3)
        assert np.array_equal(got, _np_conv(x, w, bias, pad, stride, dil, -7, 3))


def test_conv2d_int32_accumulator_wraps():
    # 2^31 / (255*255) ~ 33026 products saturate int32; the reference's accumulator wraps (-fno-strict-overflow)
    ic = 40000
    x = np.full((1, 1, 1, ic), 127, np.int8)
    w = np.full((1, 1, 1, ic), 127, np.int8)
    got = oracle.conv2d("i8", x, w, np.zeros(1, np.int32), in_zp=-128, w_zp=-128)
    want = (ic * 255 * 255 + (1 << 31)) % (1 << 32) - (1 << 31)
    assert int(got.ravel()[0]) == want and want < 0


@pytest.mark.parametrize("m", [1, 2])
def test_depthwise_i8_vs_numpy(m):
    rng = np.random.default_rng(5 + m)
    n, ih, iw, c, kh, kw = 2, 10, 8, 6, 3, 3
    pad, stride, dil = (0, 1, 0, 1), (2, 2), (1, 1)
    oh, ow = oracle.conv_out_hw(ih, iw, kh, kw, pad, stride, dil)
    x = rng.integers(-128, 128, (n, ih, iw, c)).astype(np.int8)
    w = rng.integers(-127, 128, (kh, kw, c, m)).astype(np.int8)
    bias = rng.integers(-1000, 1000, c * m).astype(np.int32)
    izp, wzp = 4, -2
    xp = np.full((n, ih + 1, iw + 1, c), izp, np.int64)
    xp[:, :ih, :iw] = x
    want = np.zeros((n, oh, ow, c, m), np.int64)
    for ky in range(kh):
        for kx in range(kw):
            sl = xp[:, ky:ky + (oh - 1) * 2 + 1:2, kx:kx + (ow - 1) * 2 + 1:2] - izp
            want += sl[..., None] * (w[ky, kx].astype(np.int64) - wzp)
    want = want.reshape(n, oh, ow, c * m) + bias
    assert np.array_equal(oracle.depthwise_conv2d("i8", x, w, bias, pad, stride, dil, izp, wzp), want)


def test_matmul_i8_vs_numpy():
    rng = np.random.default_rng(3)
    a = rng.integers(-128, 128, (3, 17, 29)).astype(np.int8)
    b = rng.integers(-128, 128, (3, 29, 11)).astype(np.int8)
    want = np.matmul(a.astype(np.int64) + 5, b.astype(np.int64) - 3)
    assert np.array_equal(oracle.matmul("i8", a, b, -5, 3), want)


def test_zero_point_folding_identity():
    """sum((a-za)(w-zw)) == sum(a*w) - zw*sum(a) - za*sum(w) + K*za*zw on the padded input: the identity the
    GPU kernels rely on, checked on the oracle with padding present."""
    rng = np.random.default_rng(11)
    x = rng.integers(-128, 128, (1, 6, 6, 5)).astype(np.int8)
    w = rng.integers(-127, 128, (4, 3, 3, 5)).astype(np.int8)
    za, zw, pad = -9, 6, (1, 1, 1, 1)
    direct = oracle.conv2d("i8", x, w, np.zeros(1, np.int32), pad, in_zp=za, w_zp=zw)
    xp = np.full((1, 8, 8, 5), za, np.int8)
    xp[:, 1:7, 1:7] = x
    raw = oracle.conv2d("i8", xp, w, np.zeros(1, np.int32))
    ones = np.ones_like(w)
    suma = oracle.conv2d("i8", xp, ones, np.zeros(1, np.int32))
    sumw = w.astype(np.int64).sum(axis=(1, 2, 3))
    K = 3 * 3 * 5
    assert np.array_equal(direct, raw - zw * suma - za * sumw + K * za * zw)


def test_fp_variants_agree_and_bounds_pass_dominates():
    rng = np.random.default_rng(21)
    x = rng.standard_normal((1, 6, 7, 8)).astype(np.float16)
    w = (rng.standard_normal((4, 3, 3, 8)) / 8).astype(np.float16)
    b = rng.standard_normal(4).astype(np.float16)
    pad = (1, 1, 1, 1)
    f32 = oracle.conv2d("f32", x, w, b, pad)
    f64 = oracle.conv2d("f64", x, w, b, pad)
    bnd = oracle.conv2d("f64", x, w, b, pad, abs_mode=True)
    want = _np_conv_f64(x, w, b)
    assert np.allclose(f64, want, rtol=1e-13, atol=1e-13)
    assert np.all(np.abs(f64) <= bnd * (1 + 1e-12))
    assert np.max(np.abs(f32 - f64)) < 72 * 2.0 ** -24 * np.max(bnd)


def _np_conv_f64(x, w, b):
    xp = np.zeros((1, 8, 9, 8))
    xp[:, 1:7, 1:8] = x
    out = np.zeros((1, 6, 7, 4))
    for ky in range(3):
        for kx in range(3):
            out += np.einsum("nhwc,oc->nhwo", xp[:, ky:ky + 6, kx:kx + 7], w[:, ky, kx].astype(np.float64))
    return out + b.astype(np.float64)


@pytest.mark.parametrize("shape", CONV_SHAPES)
def test_blas_conv_helper_equals_oracle(shape):
    """The float64-BLAS restatement used for GEMM-sized GPU cases gives the oracle's int32 results."""
    import cases
    n, ih, iw, ic, oc, kh, kw, pad, stride, dil = shape
    rng = np.random.default_rng(4242 + sum(shape[:7]))
    x = rng.integers(-128, 128, (n, ih, iw, ic)).astype(np.int8)
    w = rng.integers(-128, 128, (oc, kh, kw, ic)).astype(np.int8)
    bias = rng.integers(-(1 << 30), 1 << 30, oc).astype(np.int32)
    for zps in [(0, 0), (-128, 127), (9, -3)]:
        want = oracle.conv2d("i8", x, w, bias, pad, stride, dil, in_zp=zps[0], w_zp=zps[1])
        assert np.array_equal(cases.conv2d_exact_blas(x, w, bias, pad, stride, dil, *zps), want)
