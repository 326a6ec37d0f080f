"""GPU parity, through the C ABI, of the stand-alone RESCALE / CLAMP kernels and of the direct
(any-shape) CONV2D / DEPTHWISE_CONV2D / MATMUL kernels against the CPU oracle.  Integer results must be
bit exact; the direct fp kernels accumulate in the reference's order, so they are compared bit exactly too
(after the final fp16 / bf16 rounding)."""
import os

import numpy as np
import pytest

import cases
import gpu_ops
import oracle
import tosa_flatbuffer as fb
from reference_model_amd import Context, TmiError, capi
from test_oracle_kats import CONV_SHAPES, ZP_CASES

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def ctx():
    c = Context(0)
    c.set_kernel_choice(capi.KERNEL_DIRECT)
    yield c
    c.close()


# ---- RESCALE ---------------------------------------------------------------------------------------
@pytest.mark.parametrize("shape", [(4, 7, 16), (3, 5, 7), (1, 65539, 1, 1), (64,), (2, 3, 4, 5, 6, 8)])
@pytest.mark.parametrize("mode", [capi.ROUND_SINGLE, capi.ROUND_DOUBLE])
def test_rescale_i32_to_i8_per_channel(ctx, shape, mode):
    rng = np.random.default_rng(hash(shape) & 0xFFFF)
    C = shape[-1]
    x = rng.integers(-(1 << 26), 1 << 26, shape).astype(np.int32)
    mult = rng.integers(1 << 30, 1 << 31, C).astype(np.int32)
    shift = rng.integers(33, 46, C).astype(np.int8)
    want, wst = oracle.rescale(x, mult, shift, out_zp=-3, rounding_mode=mode)
    got, st = gpu_ops.rescale(ctx, x, mult, shift, out_zp=-3, rounding_mode=mode)
    assert st == wst == capi.VALID
    assert np.array_equal(got, want)


@pytest.mark.parametrize("shape", [(3000, 64), (517, 96), (100003, 8), (33, 1024), (70000, 4), (9, 7, 11, 32)])
@pytest.mark.parametrize("mode", [capi.ROUND_SINGLE, capi.ROUND_DOUBLE])
@pytest.mark.parametrize("shifts", ["high", "mixed", "edge32", "low"])
@pytest.mark.parametrize("out_dt,out_zp", [(np.int8, -128), (np.int8, 17), (np.int16, 0), (np.int32, 0)])
def test_rescale_i32_register_resident_kernel_in_every_form(ctx, shape, mode, shifts, out_dt, out_zp):
    """signed int32 -> int8 / int16 / int32 with C a multiple of 4 goes through the kernel that keeps the channel
    constants in registers; it takes the high word of the product when every shift of a wave is at least 32 (33
    with double rounding) and the 64-bit form otherwise.  Values span the whole int32 range where the shift allows
    and sit at the rounding boundaries."""
    rng = np.random.default_rng((hash(shape) ^ len(shifts) ^ mode) & 0xFFFF)
    C = shape[-1]
    lo_s, hi_s = {"high": (33, 47), "mixed": (28, 40), "edge32": (32, 34), "low": (20, 31)}[shifts]
    shift = rng.integers(lo_s, hi_s, C).astype(np.int8)
    mult = rng.integers(1 << 30, 1 << 31, C).astype(np.int32)
    mult[rng.integers(0, C)] = 0
    mag = 31 if lo_s >= 32 else lo_s - 2          # |value| < 2^(shift - 1) keeps the reference's range test quiet
    x = rng.integers(-(1 << mag), 1 << mag, shape, dtype=np.int64)
    x.flat[:4] = [-(1 << mag), (1 << mag) - 1, 0, -1]
    x = x.astype(np.int32)
    want, wst = oracle.rescale(x, mult, shift, out_zp=out_zp, out_dtype=out_dt, rounding_mode=mode)
    got, st = gpu_ops.rescale(ctx, x, mult, shift, out_zp=out_zp, out_dtype=out_dt, rounding_mode=mode)
    assert st == wst == capi.VALID and ctx.last_kernel == "rescale_fast"
    assert np.array_equal(got, want)


def test_rescale_i32_register_resident_kernel_flags_out_of_range_values(ctx):
    """a value at or beyond 2^(shift - 1) in magnitude fails the reference's REQUIRE (quant_util.h:56-60): the graph
    result is UNPREDICTABLE, on the 64-bit form of the kernel (shifts below 32)"""
    rng = np.random.default_rng(8)
    x = rng.integers(-(1 << 20), 1 << 20, (500, 16)).astype(np.int32)
    mult = rng.integers(1 << 30, 1 << 31, 16).astype(np.int32)
    shift = np.full(16, 24, np.int8)
    _, st = gpu_ops.rescale(ctx, x, mult, shift)
    assert st == capi.VALID
    x[321, 5] = 1 << 23
    _, st = gpu_ops.rescale(ctx, x, mult, shift)
    _, wst = oracle.rescale(x, mult, shift)
    assert st == wst == capi.UNPREDICTABLE


@pytest.mark.parametrize("in_dt,out_dt,in_u,out_u,in_zp,out_zp", [
    (np.int8, np.int8, False, False, -5, 9), (np.int8, np.int16, False, False, 3, 0),
    (np.int8, np.int32, False, False, 0, 0), (np.int16, np.int8, False, False, 0, -128),
    (np.int16, np.int16, False, False, 0, 0), (np.int16, np.int32, False, False, 0, 0),
    (np.int32, np.int16, False, False, 0, 0), (np.int32, np.int32, False, False, 0, 0),
    (np.int8, np.int8, True, False, 128, 0), (np.int8, np.int8, False, True, -128, 128),
    (np.int16, np.int16, True, False, 32768, 0), (np.int16, np.int16, False, True, 0, 32768),
    (np.int8, np.int16, False, True, 1, 32768),
])
@pytest.mark.parametrize("scale32", [True, False])
def test_rescale_dtype_matrix(ctx, in_dt, out_dt, in_u, out_u, in_zp, out_zp, scale32):
    rng = np.random.default_rng(17)
    info = np.iinfo(in_dt)
    x = rng.integers(info.min, info.max + 1, (6, 10)).astype(in_dt)
    x.ravel()[:4] = [info.min, info.max, 0, -1]
    if scale32:
        mult, shift = rng.integers(1 << 29, 1 << 31, 10), rng.integers(30, 40, 10)
    else:
        mult, shift = rng.integers(1 << 13, 1 << 15, 10), rng.integers(12, 20, 10)
    if np.dtype(in_dt) == np.int32:
        x = (x >> 8).astype(np.int32)  # keep |v| inside the shift's value range
    for mode in ([capi.ROUND_SINGLE, capi.ROUND_DOUBLE, capi.ROUND_INEXACT] if scale32 else
                 [capi.ROUND_SINGLE, capi.ROUND_INEXACT]):
        kw = dict(in_zp=in_zp, out_zp=out_zp, out_dtype=out_dt, scale32=scale32, rounding_mode=mode,
                  input_unsigned=in_u, output_unsigned=out_u)
        want, wst = oracle.rescale(x, mult, shift, **kw)
        got, st = gpu_ops.rescale(ctx, x, mult, shift, **kw)
        assert st == wst == capi.VALID, (mode, ctx.flags)
        assert np.array_equal(got.view(want.dtype), want), mode


@pytest.mark.parametrize("in_dt", [np.int8, np.int16, np.int32])
@pytest.mark.parametrize("out_dt,out_zp", [(np.int8, 60), (np.int16, 0), (np.int32, 0)])
def test_rescale_inexact_round_beyond_int32_is_reference_undefined_x86_64_convention(ctx, in_dt, out_dt, out_zp):
    """Not a parity test for the elements it is named after: an agreement between device and oracle on a convention.
    INEXACT_ROUND over the whole input range with shifts small enough for float(value) * float(multiplier) * 2^-shift
    to leave int32: the reference's cast is undefined there, its x86-64 builds return INT32_MIN, and the device
    returns the same (not its own saturating conversion), so results and status agree element for element"""
    rng = np.random.default_rng(np.dtype(in_dt).itemsize * 10 + np.dtype(out_dt).itemsize)
    info = np.iinfo(in_dt)
    x = rng.integers(info.min, info.max + 1, (40, 24)).astype(in_dt)
    x.ravel()[:3] = [info.min, info.max, 0]
    mult = rng.integers(1 << 30, 1 << 31, 24).astype(np.int32)
    shift = rng.integers(2, 40, 24).astype(np.int8)
    kw = dict(out_zp=out_zp, out_dtype=out_dt, rounding_mode=capi.ROUND_INEXACT)
    want, wst = oracle.rescale(x, mult, shift, **kw)
    got, st = gpu_ops.rescale(ctx, x, mult, shift, **kw)
    assert st == wst == capi.VALID
    assert np.array_equal(got, want)
    if out_dt == np.int32:
        assert (want == -(1 << 31)).sum() > 20    # the case is there


def test_rescale_reference_literals(ctx):  # type_conversion_tests.cpp:324-335, 385-405
    for mode in (capi.ROUND_SINGLE, capi.ROUND_INEXACT):
        got, st = gpu_ops.rescale(ctx, np.array([65], np.int8), [4], [2], in_zp=1, out_zp=32768, out_dtype=np.uint16,
                                  scale32=False, rounding_mode=mode, per_channel=False, output_unsigned=True)
        assert st == capi.VALID and got.tolist() == [32832]
    got, st = gpu_ops.rescale(ctx, np.array([103], np.int8), [147], [8], in_zp=-95, out_dtype=np.uint8,
                              scale32=False, rounding_mode=capi.ROUND_INEXACT, per_channel=False,
                              output_unsigned=True)
    assert st == capi.VALID and got.tolist() == [114]


def test_rescale_rank0_and_per_tensor(ctx):
    got, st = gpu_ops.rescale(ctx, np.array(200, np.uint8), [1 << 30], [30], in_zp=128, rounding_mode=capi.ROUND_SINGLE,
                              per_channel=False, input_unsigned=True)
    assert st == capi.VALID and got.shape == () and int(got) == 72


@pytest.mark.parametrize("inp,mult,shift,kw", [  # type_conversion_tests.cpp:337-383
    (np.array([20, -5, -16], np.int8), [4, 2], [16, 5, 9], dict(scale32=True, per_channel=True, in_zp=-19,
                                                                  out_dtype=np.int32)),
    (np.array([0, -12, 0, 12], np.int32), [4, 1024, 2048, 115], [12], dict(scale32=False, per_channel=True,
                                                                            out_zp=-12)),
    (np.array([20, -5, -16], np.int8), [4, 519], [12], dict(scale32=True, per_channel=False, in_zp=-19,
                                                             out_dtype=np.int32)),
    (np.array([0, -12, 0, 12], np.int32), [4], [6, 16], dict(scale32=False, per_channel=False, out_zp=-12)),
])
def test_rescale_shape_negatives_are_errors(ctx, inp, mult, shift, kw):
    with pytest.raises(TmiError) as e:
        gpu_ops.rescale(ctx, inp, mult, shift, rounding_mode=capi.ROUND_SINGLE, **kw)
    assert e.value.status == capi.ERROR and "OpRescale" in e.value.message


def test_rescale_require_conditions_raise_unpredictable(ctx):
    x = np.array([1 << 19, 5, 6, 7], np.int32)
    got, st = gpu_ops.rescale(ctx, x, [1 << 30], [20], per_channel=False, out_dtype=np.int32)
    assert st == capi.UNPREDICTABLE and ctx.flags & capi.FLAG_SCALE_VALUE
    assert oracle.rescale(x, [1 << 30], [20], per_channel=False, out_dtype=np.int32)[1] == oracle.UNPREDICTABLE
    # the latch is cleared by the sync that reported it
    got, st = gpu_ops.rescale(ctx, x >> 1, [1 << 30], [20], per_channel=False, out_dtype=np.int32)
    assert st == capi.VALID and ctx.flags == 0
    # apply_scale_32 cannot overflow int32 once the value check passes; apply_scale_16 can (quant_util.h:102-106)
    for mult, shift, scale32, flag in [(-1, 20, True, capi.FLAG_SCALE_MULTIPLIER), (1 << 30, 1, True, capi.FLAG_SCALE_SHIFT),
                                       (1 << 30, 63, True, capi.FLAG_SCALE_SHIFT),
                                       (1 << 14, 2, False, capi.FLAG_SCALE_RESULT)]:
        xs = np.array([1, -2, 1 << 30, 0], np.int32) if not scale32 else np.array([1, -2, 1, 0], np.int32)
        kw = dict(per_channel=False, out_dtype=np.int32, rounding_mode=capi.ROUND_SINGLE, scale32=scale32)
        _, st = gpu_ops.rescale(ctx, xs, [mult], [shift], **kw)
        _, wst = oracle.rescale(xs, [mult], [shift], **kw)
        assert (st, wst) == (capi.UNPREDICTABLE, oracle.UNPREDICTABLE) and ctx.flags & flag, (mult, shift)


@pytest.mark.parametrize("out_dt", [np.int8, np.int16, np.int32])
@pytest.mark.parametrize("shape", [(7, 9, 12), (5, 13), (1 << 16, 8)])      # vector path, scalar path, a larger tensor
@pytest.mark.parametrize("mode", [capi.ROUND_SINGLE, capi.ROUND_INEXACT])
def test_rescale_int48_input(ctx, out_dt, shape, mode):
    """INT48 (int64 storage), 16-bit multipliers: apply_scale_16 on the 64-bit value (type_conversion.cpp:122,
    :200-215, quant_util.h:86-108)"""
    rng = np.random.default_rng(shape[-1] + 48)
    C = shape[-1]
    x = rng.integers(-(1 << 47), 1 << 47, shape).astype(np.int64)
    x.ravel()[:5] = [(1 << 47) - 1, -(1 << 47), 0, -1, 1]
    mult = rng.integers(1, 1 << 15, C)
    shift = rng.integers(40, 63, C)
    if mode == capi.ROUND_INEXACT:      # fp32 arithmetic: keep the scaled values where the cast to int32 is defined
        shift = rng.integers(50, 63, C)
    kw = dict(out_dtype=out_dt, scale32=False, rounding_mode=mode)
    want, wst = oracle.rescale(x, mult, shift, **kw)
    got, st = gpu_ops.rescale(ctx, x, mult, shift, **kw)
    assert st == wst == capi.VALID, ctx.flags
    assert np.array_equal(got, want) and len(np.unique(got)) > 10


def test_rescale_int48_checks(ctx):
    x = np.array([1, 2, (1 << 47) - 1], np.int64)
    kw = dict(per_channel=False, rounding_mode=capi.ROUND_SINGLE, out_dtype=np.int16)
    for bad in (dict(scale32=True), dict(scale32=False, input_unsigned=True), dict(scale32=False, in_zp=3)):
        with pytest.raises(TmiError) as e:
            gpu_ops.rescale(ctx, x, [1 << 14], [40], **{**kw, **bad})
        assert e.value.status == capi.ERROR and "OpRescale" in e.value.message
    with pytest.raises(TmiError):
        gpu_ops.rescale(ctx, x, [1 << 14], [40], scale32=False, output_unsigned=True, per_channel=False,
                        rounding_mode=capi.ROUND_SINGLE, out_dtype=np.uint16)
    # a scaled value beyond int32 is a REQUIRE failure (quant_util.h:102-106)
    _, st = gpu_ops.rescale(ctx, x, [(1 << 15) - 1], [20], scale32=False, **{**kw, "out_dtype": np.int32})
    _, wst = oracle.rescale(x, [(1 << 15) - 1], [20], scale32=False, **{**kw, "out_dtype": np.int32})
    assert (st, wst) == (capi.UNPREDICTABLE, oracle.UNPREDICTABLE) and ctx.flags & capi.FLAG_SCALE_RESULT


def test_clamp(ctx):
    x = np.arange(-128, 128).astype(np.int8)
    got, st = gpu_ops.clamp(ctx, np.tile(x, 33)[:8000], 0, 127)
    assert st == capi.VALID and np.array_equal(got, np.clip(np.tile(x, 33)[:8000], 0, 127))
    x16 = np.arange(-40000, 40000, 7).astype(np.int16)
    got, _ = gpu_ops.clamp(ctx, x16, -300, 1234)
    assert np.array_equal(got, oracle.clamp(x16, -300, 1234))
    with pytest.raises(TmiError):
        gpu_ops.clamp(ctx, x, 5, 4)


# ---- CONV2D / DEPTHWISE / MATMUL, direct kernels ---------------------------------------------------
@pytest.mark.parametrize("inv,wv,izp,wzp,want", ZP_CASES)
def test_zero_point_literals(ctx, inv, wv, izp, wzp, want):
    x = np.array(inv, np.int8).reshape(1, 2, 2, 1)
    z = np.zeros(1, np.int32)
    got, _ = gpu_ops.conv2d(ctx, x, np.array(wv, np.int8).reshape(1, 2, 2, 1), z, stride=(2, 2), in_zp=izp, w_zp=wzp)
    assert int(got.ravel()[0]) == want
    got, _ = gpu_ops.conv2d(ctx, x, np.array(wv, np.int8).reshape(2, 2, 1, 1), z, stride=(2, 2), in_zp=izp, w_zp=wzp,
                            depthwise=True)
    assert int(got.ravel()[0]) == want
    a, b = np.array(inv, np.int8).reshape(1, 2, 2), np.array(wv, np.int8).reshape(1, 2, 2)
    got, _ = gpu_ops.matmul(ctx, a, b, izp, wzp)
    assert np.array_equal(got, oracle.matmul("i8", a, b, izp, wzp))


def test_bias_broadcast_literals(ctx):  # tensor_ops_tests.cpp:736-798
    x = np.array([5, 9], np.int8).reshape(1, 1, 1, 2)
    w = np.array([3, -7, -1, 4], np.int8).reshape(2, 1, 1, 2)
    assert gpu_ops.conv2d(ctx, x, w, np.array([-5], np.int32))[0].ravel().tolist() == [-53, 26]
    assert gpu_ops.conv2d(ctx, x, w, np.array([-5, 14], np.int32))[0].ravel().tolist() == [-53, 45]
    wd = np.array([3, -7], np.int8).reshape(1, 1, 2, 1)
    assert gpu_ops.conv2d(ctx, x, wd, np.array([-5], np.int32), depthwise=True)[0].ravel().tolist() == [10, -68]
    assert gpu_ops.conv2d(ctx, x, wd, np.array([-5, 14], np.int32), depthwise=True)[0].ravel().tolist() == [10, -49]


@pytest.mark.parametrize("shape", CONV_SHAPES)
def test_conv2d_i8_shapes(ctx, shape):
    n, ih, iw, ic, oc, kh, kw, pad, stride, dil = shape
    rng = np.random.default_rng(sum(shape[:7]))
    x = rng.integers(-128, 128, (n, ih, iw, ic)).astype(np.int8)
    w = rng.integers(-127, 128, (oc, kh, kw, ic)).astype(np.int8)
    for bias in (rng.integers(-65536, 65536, oc).astype(np.int32), np.array([77], np.int32)):
        want = oracle.conv2d("i8", x, w, bias, pad, stride, dil, in_zp=-7, w_zp=3)
        got, st = gpu_ops.conv2d(ctx, x, w, bias, pad, stride, dil, in_zp=-7, w_zp=3)
        assert st == capi.VALID and np.array_equal(got, want)
    assert ctx.last_kernel.startswith("conv2d_direct")


def test_conv_validation_errors(ctx):
    x = np.zeros((1, 5, 5, 1), np.int8)
    w = np.zeros((1, 2, 2, 1), np.int8)
    z = np.zeros(1, np.int32)
    for kw, msg in [(dict(stride=(2, 2)), "exact integer"), (dict(out_hw=(3, 4)), "Mismatch between output shape"),
                    (dict(pad=(-1, 1, 0, 0)), "pad is smaller"), (dict(stride=(0, 1)), "stride"),
                    (dict(dilation=(1, 0)), "dilation")]:
        with pytest.raises(TmiError) as e:
            gpu_ops.conv2d(ctx, x, w, z, **kw)
        assert msg in e.value.message
    with pytest.raises(TmiError) as e:
        gpu_ops.conv2d(ctx, x, np.zeros((3, 2, 2, 1), np.int8), np.zeros(2, np.int32))
    assert "bias" in e.value.message
    with pytest.raises(TmiError) as e:
        gpu_ops.conv2d(ctx, x.astype(np.float16), w.astype(np.float16), z.astype(np.float16), in_zp=1)
    assert "zero point" in e.value.message


def test_conv2d_int32_accumulator_wraps(ctx):
    ic = 40000
    x = np.full((1, 1, 1, ic), 127, np.int8)
    w = np.full((1, 1, 1, ic), 127, np.int8)
    got, _ = gpu_ops.conv2d(ctx, x, w, np.zeros(1, np.int32), in_zp=-128, w_zp=-128)
    assert np.array_equal(got, oracle.conv2d("i8", x, w, np.zeros(1, np.int32), in_zp=-128, w_zp=-128))


@pytest.mark.parametrize("m", [1, 2, 3])
def test_depthwise_i8(ctx, m):
    rng = np.random.default_rng(40 + m)
    x = rng.integers(-128, 128, (2, 10, 8, 6)).astype(np.int8)
    w = rng.integers(-127, 128, (3, 3, 6, m)).astype(np.int8)
    bias = rng.integers(-1000, 1000, 6 * m).astype(np.int32)
    args = dict(pad=(0, 1, 0, 1), stride=(2, 2), dilation=(1, 1), in_zp=4, w_zp=-2)
    want = oracle.depthwise_conv2d("i8", x, w, bias, **args)
    got, st = gpu_ops.conv2d(ctx, x, w, bias, depthwise=True, **args)
    assert st == capi.VALID and np.array_equal(got, want)


def test_matmul_i8(ctx):
    rng = np.random.default_rng(3)
    a = rng.integers(-128, 128, (3, 17, 29)).astype(np.int8)
    b = rng.integers(-128, 128, (3, 29, 11)).astype(np.int8)
    got, st = gpu_ops.matmul(ctx, a, b, -5, 3)
    assert st == capi.VALID and np.array_equal(got, oracle.matmul("i8", a, b, -5, 3))


def test_fused_conv_rescale_clamp_equals_separate_ops(ctx):
    c = cases.c1()
    acc = oracle.conv2d("i8", c["x"], c["w"], c["bias"], c["pad"], c["stride"], c["dilation"], c["in_zp"], c["w_zp"])
    want, wst = oracle.rescale(acc, c["mult"], c["shift"], out_zp=c["out_zp"])
    resc = dict(mult=c["mult"], shift=c["shift"], out_zp=c["out_zp"])
    got, st = gpu_ops.conv2d(ctx, c["x"], c["w"], c["bias"], c["pad"], c["stride"], c["dilation"], c["in_zp"],
                             c["w_zp"], rescale=resc)
    assert st == wst == capi.VALID and np.array_equal(got, want)
    got, st = gpu_ops.conv2d(ctx, c["x"], c["w"], c["bias"], c["pad"], c["stride"], c["dilation"], c["in_zp"],
                             c["w_zp"], rescale=resc, clamp=(-20, 31))
    assert np.array_equal(got, oracle.clamp(want, -20, 31))


def test_reference_qi8_example_graph(ctx, golden_dir):
    """The reference's own int8 example (CONV2D -> RESCALE double round) reproduces its stored golden."""
    d = os.path.join(golden_dir, "qi8_conv2d_1x1")
    tensors, ops, _, _ = fb.load_main_block(os.path.join(d, "graph.tosa"))
    x = np.load(os.path.join(d, "placeholder_0.npy"))
    want = np.load(os.path.join(d, "tflite_result.npy"))
    conv, resc = ops[-2], ops[-1]
    ca = fb.conv_attr(conv["attr"])
    t = lambda n: tensors[n]["data"]
    acc, st = gpu_ops.conv2d(ctx, x, t(conv["inputs"][1]), t(conv["inputs"][2]), ca["pad"], ca["stride"],
                             ca["dilation"], int(t(conv["inputs"][3])[0]), int(t(conv["inputs"][4])[0]))
    assert st == capi.VALID
    got, st = gpu_ops.rescale(ctx, acc, t(resc["inputs"][1]), t(resc["inputs"][2]), int(t(resc["inputs"][3])[0]),
                              int(t(resc["inputs"][4])[0]))
    assert st == capi.VALID and np.array_equal(got, want)
    fused, st = gpu_ops.conv2d(ctx, x, t(conv["inputs"][1]), t(conv["inputs"][2]), ca["pad"], ca["stride"],
                               ca["dilation"], 0, 0, rescale=dict(mult=t(resc["inputs"][1]), shift=t(resc["inputs"][2]),
                                                                   out_zp=int(t(resc["inputs"][4])[0])))
    assert st == capi.VALID and np.array_equal(fused, want)


def test_fp16_direct_conv_matches_reference_accumulation_order(ctx):
    rng = np.random.default_rng(21)
    x = rng.standard_normal((2, 6, 7, 8)).astype(np.float16)
    w = (rng.standard_normal((4, 3, 3, 8)) / 8).astype(np.float16)
    b = rng.standard_normal(4).astype(np.float16)
    want = oracle.conv2d("f32", x, w, b, (1, 1, 1, 1)).astype(np.float16)
    got, st = gpu_ops.conv2d(ctx, x, w, b, (1, 1, 1, 1))
    assert st == capi.VALID and np.array_equal(got.view(np.uint16), want.view(np.uint16))


def test_bf16_direct_matmul(ctx):
    rng = np.random.default_rng(22)
    a = cases.float_to_bf16_bits(rng.standard_normal((2, 9, 33)).astype(np.float32))
    b = cases.float_to_bf16_bits(rng.standard_normal((2, 33, 5)).astype(np.float32))
    want = oracle.matmul("f32", cases.bf16_bits_to_float(a), cases.bf16_bits_to_float(b))
    got, st = gpu_ops.matmul(ctx, a, b, dtype=capi.BF16)
    assert st == capi.VALID and np.array_equal(got.view(np.uint32), want.view(np.uint32))


# ---- FP32 CONV2D / DEPTHWISE_CONV2D / MATMUL (OpConv2d<FP32,FP32,FP32,FP32> etc., tensor_ops.cpp:2220-2270) ----
@pytest.mark.parametrize("shape", [
    # n, ih, iw, ic, oc, kh, kw, pad, stride, dilation
    (1, 32, 32, 8, 16, 1, 1, (0, 0, 0, 0), (1, 1), (1, 1)),      # the reference's FP32 example geometry
    (2, 9, 11, 5, 7, 3, 3, (1, 1, 1, 1), (1, 1), (1, 1)),
    (1, 12, 10, 6, 4, 3, 2, (0, 1, 1, 0), (2, 1), (1, 2)),
])
def test_conv2d_fp32_reproduces_the_reference_summation_order(ctx, shape):
    """the one-element-per-lane kernel adds the products in the reference's ky -> kx -> ic order with separate
    multiplies and adds, like the oracle's loop nest: equal bit for bit"""
    n, ih, iw, ic, oc, kh, kw, pad, stride, dil = shape
    rng = np.random.default_rng(ic * oc + kh)
    x = rng.normal(0, 1, (n, ih, iw, ic)).astype(np.float32)
    w = rng.normal(0, 0.3, (oc, kh, kw, ic)).astype(np.float32)
    b = rng.normal(0, 1, oc).astype(np.float32)
    got, st = gpu_ops.conv2d(ctx, x, w, b, pad, stride, dil, dtype=capi.FP32)
    assert st == capi.VALID and ctx.last_kernel == "conv2d_direct_f32" and got.dtype == np.float32
    assert np.array_equal(got, oracle.conv2d("f32", x, w, b, pad, stride, dil))
    # and within a few fp32 roundings of the fp64 result
    ref = oracle.conv2d("f64", x.astype(np.float64), w.astype(np.float64), b.astype(np.float64), pad, stride, dil)
    assert np.allclose(got, ref, rtol=1e-5, atol=1e-5)


def test_depthwise_and_matmul_fp32(ctx):
    rng = np.random.default_rng(32)
    x = rng.normal(0, 1, (2, 9, 8, 6)).astype(np.float32)
    w = rng.normal(0, 0.5, (3, 3, 6, 2)).astype(np.float32)
    b = rng.normal(0, 1, 12).astype(np.float32)
    got, st = gpu_ops.conv2d(ctx, x, w, b, (1, 1, 1, 1), depthwise=True, dtype=capi.FP32)
    assert st == capi.VALID and ctx.last_kernel == "depthwise_direct_f32"
    assert np.array_equal(got, oracle.depthwise_conv2d("f32", x, w, b, (1, 1, 1, 1)))
    a = rng.normal(0, 1, (3, 7, 20)).astype(np.float32)
    bm = rng.normal(0, 1, (3, 20, 5)).astype(np.float32)
    got, st = gpu_ops.matmul(ctx, a, bm, dtype=capi.FP32)
    assert st == capi.VALID and ctx.last_kernel == "matmul_direct_f32"
    assert np.array_equal(got, oracle.matmul("f32", a, bm))
    with pytest.raises(TmiError):      # zero points are for INT8 only (tensor_ops.cpp:1433-1434)
        gpu_ops.matmul(ctx, a, bm, a_zp=1, dtype=capi.FP32)
