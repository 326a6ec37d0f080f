"""GPU parity of AVG_POOL2D / MAX_POOL2D against the CPU oracle through the C ABI: bit exact for every type
(the floating-point AVG_POOL2D accumulates in fp32 in tap order like the reference, so it has one right answer)."""
import numpy as np
import pytest

import cases
import gpu_ops
import oracle
from reference_model_amd import Context, TmiError, capi
from test_oracle_pool import POOL_SHAPES

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def ctx():
    c = Context(0)
    yield c
    c.close()


GPU_POOL_SHAPES = POOL_SHAPES + [
    (2, 56, 56, 64, (2, 2), (2, 2), (0, 0, 0, 0)),       # 16-byte pieces for every type
    (1, 112, 112, 32, (3, 3), (2, 2), (0, 1, 0, 1)),
    (4, 7, 7, 1280, (7, 7), (1, 1), (0, 0, 0, 0)),       # global average pooling at a classifier head
    (1, 33, 29, 24, (3, 3), (1, 1), (1, 1, 1, 1)),
]


def random_ints(rng, dtype, shape):
    info = np.iinfo(dtype)
    return rng.integers(info.min, info.max + 1, shape).astype(dtype)


@pytest.mark.parametrize("shape", GPU_POOL_SHAPES)
@pytest.mark.parametrize("dtype,zps", [(np.int8, (0, 0)), (np.int8, (-7, 12)), (np.int8, (127, -128)), (np.int16, (0, 0))])
def test_avg_pool_int_bit_exact(ctx, shape, dtype, zps):
    n, ih, iw, c, kernel, stride, pad = shape
    x = random_ints(np.random.default_rng(ih * 31 + c), dtype, (n, ih, iw, c))
    got, st = gpu_ops.pool2d(ctx, x, kernel, stride, pad, avg=True, in_zp=zps[0], out_zp=zps[1])
    assert st == capi.VALID and ctx.last_kernel.startswith("avg_pool2d")
    assert np.array_equal(got, oracle.avg_pool2d(x, kernel, stride, pad, *zps))


@pytest.mark.parametrize("shape", GPU_POOL_SHAPES)
@pytest.mark.parametrize("dtype", [np.int8, np.int16])
def test_max_pool_int_bit_exact(ctx, shape, dtype):
    n, ih, iw, c, kernel, stride, pad = shape
    x = random_ints(np.random.default_rng(iw + c), dtype, (n, ih, iw, c))
    got, st = gpu_ops.pool2d(ctx, x, kernel, stride, pad, avg=False)
    assert st == capi.VALID and ctx.last_kernel.startswith("max_pool2d")
    assert np.array_equal(got, oracle.max_pool2d(x, kernel, stride, pad))


def float_operand(rng, kind, shape):
    """(array as it travels to the device, the same values as float32, TMI dtype, narrowing function)"""
    x = rng.normal(0, 4, shape).astype(np.float32)
    if kind == "fp16":
        h = x.astype(np.float16)
        return h, h.astype(np.float32), capi.FP16, lambda r: r.astype(np.float16)
    if kind == "bf16":
        b = cases.float_to_bf16_bits(x)
        return b, cases.bf16_bits_to_float(b), capi.BF16, cases.float_to_bf16_bits
    return x, x, capi.FP32, lambda r: r


@pytest.mark.parametrize("shape", GPU_POOL_SHAPES)
@pytest.mark.parametrize("kind", ["fp16", "bf16", "fp32"])
def test_avg_pool_float_bit_exact(ctx, shape, kind):
    n, ih, iw, c, kernel, stride, pad = shape
    dev, as_f32, dtype, narrow = float_operand(np.random.default_rng(ih + c), kind, (n, ih, iw, c))
    got, st = gpu_ops.pool2d(ctx, dev, kernel, stride, pad, avg=True, dtype=dtype)
    want = narrow(oracle.avg_pool2d(as_f32, kernel, stride, pad))     # fp32 accumulate, one narrowing (RNE)
    assert st == capi.VALID and np.array_equal(got.view(np.uint16 if kind != "fp32" else np.uint32),
                                               want.view(np.uint16 if kind != "fp32" else np.uint32))


@pytest.mark.parametrize("shape", GPU_POOL_SHAPES)
@pytest.mark.parametrize("kind", ["fp16", "bf16", "fp32"])
@pytest.mark.parametrize("nan_mode", [1, 2])
def test_max_pool_float_nan_modes_bit_exact(ctx, shape, kind, nan_mode):
    n, ih, iw, c, kernel, stride, pad = shape
    rng = np.random.default_rng(3 * iw + c)
    dev, as_f32, dtype, narrow = float_operand(rng, kind, (n, ih, iw, c))
    nan_at, inf_at = rng.random(dev.shape) < 0.1, rng.random(dev.shape) < 0.02
    as_f32 = as_f32.copy()
    as_f32[nan_at], as_f32[inf_at] = np.nan, -np.inf
    dev = narrow(as_f32)
    got, st = gpu_ops.pool2d(ctx, dev, kernel, stride, pad, avg=False, nan_mode=nan_mode, dtype=dtype)
    want = oracle.max_pool2d(as_f32, kernel, stride, pad, nan_mode=nan_mode)
    got_f32 = cases.bf16_bits_to_float(got) if kind == "bf16" else got.astype(np.float32)
    assert st == capi.VALID
    assert np.array_equal(np.isnan(got_f32), np.isnan(want))
    assert np.array_equal(got_f32[~np.isnan(want)], want[~np.isnan(want)])


def test_pool_errors_carry_the_reference_messages(ctx):
    x = np.zeros((1, 8, 8, 4), np.int8)
    with pytest.raises(TmiError, match="OpAvgPool2d: At least one pad is >= kernel dimension"):
        gpu_ops.pool2d(ctx, x, (2, 2), (2, 2), (2, 0, 0, 0), out_hw=(5, 4))
    with pytest.raises(TmiError, match="OpMaxPool2d: Parameters must yield exact integer output dimensions"):
        gpu_ops.pool2d(ctx, x, (3, 3), (2, 2), avg=False, out_hw=(3, 3))
    with pytest.raises(TmiError, match=r"expected output shape \(4,4\)"):
        gpu_ops.pool2d(ctx, x, (2, 2), (2, 2), out_hw=(4, 5))
    with pytest.raises(TmiError, match="Input zeropoint must be zero for non int8_t data"):
        gpu_ops.pool2d(ctx, x.astype(np.int16), (2, 2), (2, 2), in_zp=1)
    with pytest.raises(TmiError, match="accumulator type not supported"):
        gpu_ops.pool2d(ctx, x.astype(np.float16), (2, 2), (2, 2), acc_dtype=capi.FP16)


def test_pool_of_an_empty_tensor(ctx):
    got, st = gpu_ops.pool2d(ctx, np.zeros((0, 4, 4, 8), np.int8), (2, 2), (2, 2))
    assert st == capi.VALID and got.shape == (0, 2, 2, 8)
