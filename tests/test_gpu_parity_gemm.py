"""GPU parity of the MFMA GEMM kernel (1x1 CONV2D and MATMUL with operands loaded straight into LDS) against
the CPU oracle and exact float64 BLAS products, through the C ABI.  int8 results are compared bit for bit;
fp16 / bf16 results with the reference's DOT_PRODUCT bound against fp64 (tolerance stated at the assert)."""
import numpy as np
import pytest

import cases
import dot_product_check as dp
import gpu_ops
import oracle
from reference_model_amd import Context, TmiError, capi

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def ctx():
    c = Context(0)
    c.set_kernel_choice(capi.KERNEL_GEMM)
    yield c
    c.close()


def exact_matmul_i8(a, b, a_zp, b_zp):
    """float64 BLAS product: exact, every partial sum is an integer below 2^53"""
    want = np.matmul(a.astype(np.float64) - a_zp, b.astype(np.float64) - b_zp)
    return want.astype(np.int64).astype(np.int32)


# n, h, c, w: the three workgroup shapes (256x256, 128x256, 128x128 channels x pixels), ragged edges in both
# directions, channel counts that are not a multiple of 16, one and many 64-byte K blocks
GEMM_SHAPES = [
    (4, 2048, 320, 2048),     # 256 tiles of 256x256
    (8, 1024, 256, 1024),     # 128x256 tiles
    (2, 1024, 1024, 1024),    # 128x128 tiles
    (3, 1000, 448, 1100),     # ragged rows and columns, columns a multiple of 4 only
    (3, 1000, 448, 1104),     # ragged, whole 16-byte pieces per row of B
    (5, 520, 192 * 3, 784),
    (1, 4099, 256, 515),      # odd column count: element-wise stores
    (32, 300, 64 * 5, 200),
    (1, 128, 256, 16384),
    (1, 16384, 256, 64),
    (2, 1024, 64 * 37, 1024),  # deep K on the small shapes: blocks requested in pairs, an odd number of them
    (3, 900, 64 * 40, 1104),   # the same with an even number and ragged tiles
    (8, 1024, 64 * 35, 1024),  # 128x256 tiles, odd
    (4, 2048, 64 * 49, 2048),  # K-major operand, 48 blocks or more: the first operand's rows requested in pairs;
    (8, 1024, 64 * 50, 1024),  # 256x256 and 128x256 tiles, odd and even block counts, ragged edges
    (3, 1000, 64 * 51, 1104),
    (1, 512, 512, 512),       # 16 tiles: small products are this kernel's too
    (8, 256, 256, 256),
    (1, 130, 64 * 5, 200),    # four ragged tiles
    (8, 1024, 64, 1024),      # one block of K
    (3, 500, 128, 392),       # two, ragged
    (1, 4096, 192, 4096),     # three, 256x256 tiles
]


@pytest.mark.parametrize("shape", GEMM_SHAPES)
@pytest.mark.parametrize("zps", [(0, 0), (7, -9), (-128, 0), (0, 127)])
def test_matmul_i8_gemm_bit_exact(ctx, shape, zps):
    n, h, c, w = shape
    rng = np.random.default_rng(n * 1000 + h + c + w)
    a = rng.integers(-128, 128, (n, h, c)).astype(np.int8)
    b = rng.integers(-128, 128, (n, c, w)).astype(np.int8)
    got, st = gpu_ops.matmul(ctx, a, b, *zps)
    # B is read as it lies when its rows are whole 16-byte pieces, else from a transposed copy
    assert st == capi.VALID and ctx.last_kernel == ("matmul_gemm_i8" if w % 16 == 0 else "matmul_tgemm_i8")
    assert np.array_equal(got, exact_matmul_i8(a, b, *zps))
    # a corner of the last batch against the scalar oracle (the BLAS product is a second, independent witness)
    assert np.array_equal(got[-1, -24:], oracle.matmul("i8", a[-1:, -24:], b[-1:], *zps)[0])


def random_matmul_shapes(count, seed):
    """seeded shapes around the block counts where the kernel changes how it requests its operands (32 and 48
    blocks of 64 bytes), odd and even counts, ragged tiles in both directions"""
    rng = np.random.default_rng(seed)
    shapes = []
    while len(shapes) < count:
        n = int(rng.integers(1, 5))
        h = int(rng.integers(128, 1400))
        w = 16 * int(rng.integers(8, 90))
        blocks = int(rng.choice([4, 7, 16, 31, 32, 33, 34, 47, 48, 49, 50, 63, 64, 65]))
        if ((h + 127) // 128) * ((w + 127) // 128) * n >= 128:    # enough work for the kernel to take it
            shapes.append((n, h, blocks, w))
    return shapes


@pytest.mark.parametrize("shape", random_matmul_shapes(28, 20240607))
def test_matmul_i8_gemm_random_shapes_bit_exact(ctx, shape):
    n, h, blocks, w = shape
    c = 64 * blocks
    rng = np.random.default_rng(h * 7 + w + blocks)
    a = rng.integers(-128, 128, (n, h, c)).astype(np.int8)
    b = rng.integers(-128, 128, (n, c, w)).astype(np.int8)
    zps = (int(rng.integers(-128, 128)), int(rng.integers(-128, 128))) if blocks % 2 else (0, 0)
    got, st = gpu_ops.matmul(ctx, a, b, *zps)
    assert st == capi.VALID and ctx.last_kernel == "matmul_gemm_i8"
    assert np.array_equal(got, exact_matmul_i8(a, b, *zps))


@pytest.mark.parametrize("shape", random_matmul_shapes(10, 77))
def test_matmul_bf16_gemm_random_shapes_within_dot_product_bound(ctx, shape):
    n, h, blocks, w = shape
    c = 32 * blocks
    rng = np.random.default_rng(h + w + blocks)
    a_s = cases.float_to_bf16_bits(rng.normal(0, 1 / 8, (n, h, c)).astype(np.float32))
    b_s = cases.float_to_bf16_bits(rng.normal(0, 1 / 8, (n, c, w)).astype(np.float32))
    af, bf = cases.bf16_bits_to_float(a_s).astype(np.float64), cases.bf16_bits_to_float(b_s).astype(np.float64)
    got, st = gpu_ops.matmul(ctx, a_s, b_s, dtype=capi.BF16)
    assert st == capi.VALID and ctx.last_kernel == "matmul_gemm_bf16"
    ref, bnd = np.matmul(af, bf), np.matmul(np.abs(af), np.abs(bf))
    # tolerance: |imp-ref| <= 2*C * max(bnd*2^-24, 2^-126) per element and sum err^2 <= 1.6*C*T
    res = dp.check(got, ref, bnd, "fp32", dp.kernel_size_bound(c, "fp32", has_bias=False))
    assert res["ok"], res


def test_matmul_i8_gemm_extreme_values(ctx):
    """all operands at -128 with zero points at +127: the largest products the operator can form"""
    n, h, c, w = 8, 512, 4096, 512
    a = np.full((n, h, c), -128, np.int8)
    b = np.full((n, c, w), -128, np.int8)
    got, st = gpu_ops.matmul(ctx, a, b, 127, 127)
    assert st == capi.VALID and ctx.last_kernel == "matmul_gemm_i8"
    assert np.all(got == 255 * 255 * c)


def test_gemm_kernel_refuses_what_it_cannot_take(ctx):
    rng = np.random.default_rng(1)
    a = rng.integers(-128, 128, (1, 512, 100)).astype(np.int8)     # K bytes not a multiple of 64
    b = rng.integers(-128, 128, (1, 100, 512)).astype(np.int8)
    with pytest.raises(TmiError):
        gpu_ops.matmul(ctx, a, b)
    a = rng.integers(-128, 128, (1, 64, 256)).astype(np.int8)      # too little work
    b = rng.integers(-128, 128, (1, 256, 64)).astype(np.int8)
    with pytest.raises(TmiError):
        gpu_ops.matmul(ctx, a, b)


@pytest.mark.parametrize("kind", ["fp16", "bf16"])
@pytest.mark.parametrize("shape", [(2, 2048, 512, 2048), (8, 1024, 256, 1024), (3, 1000, 448, 1100), (3, 1000, 448, 1104),
                                   (1, 4099, 128, 515), (5, 520, 96 * 3, 784),
                                   (3, 1000, 32 * 37, 1104), (8, 1024, 32 * 42, 1024),   # deep K: blocks in pairs
                                   (4, 2048, 32 * 49, 2048), (3, 1000, 32 * 52, 1104),   # ... the first operand's rows
                                   (8, 1024, 32, 1024), (3, 500, 64, 392), (16, 512, 96, 512)])  # one to three blocks of K
def test_matmul_fp_gemm_within_dot_product_bound(ctx, kind, shape):
    n, h, c, w = shape
    rng = np.random.default_rng(8 + h)
    a = rng.normal(0, 1 / 8, (n, h, c)).astype(np.float32)
    b = rng.normal(0, 1 / 8, (n, c, w)).astype(np.float32)
    if kind == "fp16":
        a_s, b_s, dtype = a.astype(np.float16), b.astype(np.float16), capi.FP16
        af, bf = a_s.astype(np.float64), b_s.astype(np.float64)
    else:
        a_s, b_s, dtype = cases.float_to_bf16_bits(a), cases.float_to_bf16_bits(b), capi.BF16
        af, bf = cases.bf16_bits_to_float(a_s).astype(np.float64), cases.bf16_bits_to_float(b_s).astype(np.float64)
    got, st = gpu_ops.matmul(ctx, a_s, b_s, dtype=dtype)
    assert st == capi.VALID and got.dtype == np.float32
    assert ctx.last_kernel == ("matmul_" + ("gemm" if w % 8 == 0 else "tgemm") + ("_f16" if kind == "fp16" else "_bf16"))
    ref, bnd = np.matmul(af, bf), np.matmul(np.abs(af), np.abs(bf))
    res = dp.check(got, ref, bnd, "fp32", dp.kernel_size_bound(c, "fp32", has_bias=False))
    # tolerance: |imp-ref| <= 2*C * max(bnd*2^-24, 2^-126) per element and sum err^2 <= 1.6*C*T
    assert res["ok"], res


# ---- 1x1 CONV2D: all images are rows of one GEMM, bias per channel ---------------------------------------------
@pytest.mark.parametrize("shape", [  # n, ih, iw, ic, oc
    (8, 56, 56, 256, 64),
    (4, 28, 28, 512, 648),
    (1, 97, 131, 256, 130),
    (8, 32, 33, 2944, 200),    # 46 blocks of K: whole trips round the ring of stages, then the general form
    (8, 30, 34, 3520, 136),    # 55 blocks: an odd count behind the trips
    (1, 14, 14, 1024, 200),    # four tiles: a pointwise layer is this kernel's from there on
    (8, 56, 56, 64, 256),      # one block of K
    (4, 40, 40, 128, 136),     # two
    (3, 7, 7, 2048, 520),      # ragged in both directions, 10 tiles
])
@pytest.mark.parametrize("zps", [(0, 0), (-6, 11)])
def test_conv2d_1x1_i8_gemm_bit_exact(ctx, shape, zps):
    n, ih, iw, ic, oc = shape
    rng = np.random.default_rng(ih * iw + oc)
    x = rng.integers(-128, 128, (n, ih, iw, ic)).astype(np.int8)
    w = rng.integers(-128, 128, (oc, 1, 1, ic)).astype(np.int8)
    bias = rng.integers(-(1 << 20), 1 << 20, oc).astype(np.int32)
    got, st = gpu_ops.conv2d(ctx, x, w, bias, in_zp=zps[0], w_zp=zps[1])
    assert st == capi.VALID and ctx.last_kernel == "gemm_mfma_i8"
    want = exact_matmul_i8(x.reshape(1, -1, ic), w.reshape(1, oc, ic).transpose(0, 2, 1), *zps)[0] + bias
    assert np.array_equal(got.reshape(-1, oc), want)
    sub = oracle.conv2d("i8", x[-1:, -2:], w, bias, in_zp=zps[0], w_zp=zps[1])
    assert np.array_equal(got[-1:, -2:], sub)


@pytest.mark.parametrize("kind", ["fp16", "bf16"])
@pytest.mark.parametrize("shape", [(8, 40, 40, 256, 208), (2, 61, 67, 128, 203), (8, 32, 33, 1472, 200), (1, 14, 14, 1024, 200),
                                   (8, 56, 56, 64, 256), (4, 40, 40, 32, 136)])
def test_conv2d_1x1_fp_gemm_within_dot_product_bound(ctx, kind, shape):
    n, ih, iw, ic, oc = shape
    rng = np.random.default_rng(ic + oc)
    x = rng.normal(0, 1, (n, ih, iw, ic)).astype(np.float32)
    w = rng.normal(0, 1 / np.sqrt(ic), (oc, 1, 1, ic)).astype(np.float32)
    b = rng.normal(0, 0.1, oc).astype(np.float32)
    if kind == "fp16":
        xs, ws, bs = x.astype(np.float16), w.astype(np.float16), b.astype(np.float16)
        xf, wf, bf = (v.astype(np.float64) for v in (xs, ws, bs))
        dtype = capi.FP16
    else:
        xs, ws, bs = (cases.float_to_bf16_bits(v) for v in (x, w, b))
        xf, wf, bf = (cases.bf16_bits_to_float(v).astype(np.float64) for v in (xs, ws, bs))
        dtype = capi.BF16
    got, st = gpu_ops.conv2d(ctx, xs, ws, bs, dtype=dtype)
    assert st == capi.VALID and ctx.last_kernel == ("gemm_mfma_f16" if kind == "fp16" else "gemm_mfma_bf16")
    imp = got.astype(np.float64) if kind == "fp16" else cases.bf16_bits_to_float(got).astype(np.float64)
    ref = np.matmul(xf.reshape(-1, ic), wf.reshape(oc, ic).T) + bf
    bnd = np.matmul(np.abs(xf.reshape(-1, ic)), np.abs(wf.reshape(oc, ic).T)) + np.abs(bf)
    res = dp.check(imp.reshape(-1, oc), ref, bnd, kind, dp.kernel_size_bound(ic, kind))
    # tolerance: |imp-ref| <= 2*ksb * max(bnd*2^-(1+frac), normal_min) per element, sum err^2 <= 1.6*ksb*T
    assert res["ok"], res
    # a corner against the oracle's own loop nest
    sub = oracle.conv2d("f64", xf[-1:, -2:], wf, bf, (0, 0, 0, 0), (1, 1), (1, 1))
    assert np.allclose(imp[-1:, -2:], sub, rtol=2.0 ** -7, atol=2.0 ** -10)


# ---- the benchmark configurations at full size ----------------------------------------------------------------
def test_config2_matmul_full_size_gemm(ctx):
    """[8,1024,1024] x [8,1024,1024] -> int32, a_zp -5, b_zp 3: every element against a float64 BLAS product
    (exact: |sum| < 2^53), one batch corner against the scalar oracle, plus the transposition property
    (A.B)^T = B^T.A^T computed by the same kernel."""
    c = cases.c2()
    got, st = gpu_ops.matmul(ctx, c["a"], c["b"], c["a_zp"], c["b_zp"])
    assert st == capi.VALID and ctx.last_kernel == "matmul_gemm_i8"
    assert np.array_equal(got, exact_matmul_i8(c["a"], c["b"], c["a_zp"], c["b_zp"]))
    assert np.array_equal(got[5, :16], oracle.matmul("i8", c["a"][5:6, :16], c["b"][5:6], c["a_zp"], c["b_zp"])[0])
    at = np.ascontiguousarray(c["a"].transpose(0, 2, 1))
    bt = np.ascontiguousarray(c["b"].transpose(0, 2, 1))
    got_t, _ = gpu_ops.matmul(ctx, bt, at, c["b_zp"], c["a_zp"])
    assert np.array_equal(got_t, got.transpose(0, 2, 1))


def test_config5_bf16_matmul_full_size_gemm(ctx):
    """[4,2048,4096] x [4,4096,2048] bf16 -> fp32.  256 rows of every batch against fp64 with the DOT_PRODUCT
    bound; the whole result through a property that needs no reference: scaling A by 2 (exact in bf16) must
    scale every fp32 partial sum, hence every result, by exactly 2."""
    c = cases.c5_matmul()
    got, st = gpu_ops.matmul(ctx, c["a"], c["b"], dtype=capi.BF16)
    assert st == capi.VALID and ctx.last_kernel == "matmul_gemm_bf16"
    rows = slice(1000, 1256)
    af = cases.bf16_bits_to_float(c["a"][:, rows]).astype(np.float64)
    bf = cases.bf16_bits_to_float(c["b"]).astype(np.float64)
    ref, bnd = np.matmul(af, bf), np.matmul(np.abs(af), np.abs(bf))
    res = dp.check(got[:, rows], ref, bnd, "fp32", dp.kernel_size_bound(c["a"].shape[2], "fp32", has_bias=False))
    # tolerance: |imp-ref| <= 2*C * max(bnd*2^-24, 2^-126) per element and sum err^2 <= 1.6*C*T
    assert res["ok"], res
    a2 = cases.float_to_bf16_bits(cases.bf16_bits_to_float(c["a"]) * 2.0)
    got2, _ = gpu_ops.matmul(ctx, a2, c["b"], dtype=capi.BF16)
    assert np.array_equal(got2, got * np.float32(2.0))


# ---- convolutions with taps through the GEMM kernel (K axis = (ky, kx, ic), taps outside the image read zeros) ----
def patch_form(oh, ow, ic_bytes, oc, kh, kw, stride, dil):
    """"_patch" where the GEMM kernel keeps the input patch of a tile in LDS: stride 1, tiles of whole output rows that
    use at least 96 of their 128 pixel rows and 3/4 of an image's last tile, and a patch of (rows + (kh-1) dil) x
    (ow + (kw-1) dil) pixels that fits behind the ring of weight stages (64 KB) and the tables"""
    if tuple(stride) != (1, 1) or ow > 128 or oc < 128 or kh * kw * ic_bytes // 64 < 8:
        return ""
    rows = min(128 // ow, oh)
    patch_bytes = (rows - 1 + (kh - 1) * dil[0] + 1) * (ow - 1 + (kw - 1) * dil[1] + 1) * ic_bytes
    fits = 65536 + 4608 + -(-patch_bytes // 1024) * 1024 <= 160 * 1024
    return "_patch" if rows * ow >= 96 and oh * 4 >= -(-oh // rows) * rows * 3 and fits else ""


TAP_SHAPES = [  # n, ih, iw, ic, oc, kh, kw, pad, stride, dilation
    (16, 28, 28, 256, 256, 3, 3, (1, 1, 1, 1), (1, 1), (1, 1)),     # the named fp16 configuration
    (40, 31, 29, 64, 136, 3, 3, (1, 1, 1, 1), (2, 2), (1, 1)),      # stride 2, ragged tiles
    (6, 40, 40, 128, 200, 5, 3, (2, 2, 1, 1), (1, 1), (1, 1)),      # 15 taps
    (32, 24, 24, 64, 64, 3, 3, (2, 2, 2, 2), (1, 1), (2, 2)),       # dilation 2
    (16, 64, 64, 192, 96, 2, 2, (0, 0, 0, 0), (2, 2), (1, 1)),      # no padding
    (2, 130, 100, 64, 72, 1, 7, (0, 0, 3, 3), (1, 1), (1, 1)),
    (16, 28, 28, 320, 256, 3, 3, (1, 1, 1, 1), (1, 1), (1, 1)),     # 5 blocks per tap: pairs of blocks straddle taps
    # floating point, stride 1, a patch that fits the LDS: the patch form (tiles of whole output rows)
    (24, 29, 20, 256, 160, 3, 3, (1, 1, 1, 1), (1, 1), (1, 1)),     # last tile of an image and of the channels ragged
    (20, 30, 30, 128, 128, 3, 3, (2, 2, 2, 2), (1, 1), (2, 2)),     # dilation 2, 4 blocks per tap
    (20, 26, 21, 192, 136, 2, 3, (0, 1, 2, 0), (1, 1), (1, 1)),     # uneven padding, 6 blocks per tap
    (24, 20, 36, 256, 128, 1, 3, (0, 0, 1, 1), (1, 1), (1, 1)),     # one row of taps, tiles of 3 rows
    (3, 30, 26, 128, 200, 3, 3, (1, 1, 1, 1), (1, 1), (1, 1)),      # 48 tiles of whole rows where 128-pixel tiles would be 38
    (12, 30, 28, 64, 136, 3, 3, (1, 1, 1, 1), (1, 1), (1, 1)),      # few channels: one (int8) or two (fp) blocks per tap
]
FP_TAP_SHAPES = [  # rows of K that are whole 64-byte blocks for two-byte elements only
    (12, 28, 30, 32, 128, 3, 3, (1, 1, 1, 1), (1, 1), (1, 1)),      # one block per tap
    (10, 33, 25, 96, 160, 3, 3, (1, 1, 1, 1), (1, 1), (1, 1)),      # three
]


@pytest.mark.parametrize("shape", TAP_SHAPES)
@pytest.mark.parametrize("w_zp", [0, -11])
def test_conv2d_taps_i8_gemm_bit_exact(ctx, shape, w_zp):
    n, ih, iw, ic, oc, kh, kw, pad, stride, dil = shape
    rng = np.random.default_rng(ih * iw + oc + kh)
    x = rng.integers(-128, 128, (n, ih, iw, ic)).astype(np.int8)
    w = rng.integers(-128, 128, (oc, kh, kw, ic)).astype(np.int8)
    bias = rng.integers(-(1 << 20), 1 << 20, oc).astype(np.int32)
    got, st = gpu_ops.conv2d(ctx, x, w, bias, pad, stride, dil, in_zp=0, w_zp=w_zp)
    assert st == capi.VALID
    assert ctx.last_kernel == "gemm_mfma_i8" + patch_form(got.shape[1], got.shape[2], ic, oc, kh, kw, stride, dil)
    assert np.array_equal(got, cases.conv2d_exact_blas(x, w, bias, pad, stride, dil, 0, w_zp))
    sub = oracle.conv2d("i8", x[-1:], w[:3], bias[:3], pad, stride, dil, in_zp=0, w_zp=w_zp)
    assert np.array_equal(got[-1:, :, :, :3], sub)


@pytest.mark.parametrize("in_zp", [5, -128, 127])
def test_conv2d_taps_i8_gemm_pads_with_the_input_zero_point(ctx, in_zp):
    """taps outside the image read a page of input_zp bytes, so they contribute (zp - zp) * (w - w_zp) = 0"""
    rng = np.random.default_rng(in_zp + 500)
    x = rng.integers(-128, 128, (32, 28, 28, 64)).astype(np.int8)
    w = rng.integers(-128, 128, (72, 3, 3, 64)).astype(np.int8)
    bias = rng.integers(-999, 999, 72).astype(np.int32)
    got, st = gpu_ops.conv2d(ctx, x, w, bias, (1, 1, 1, 1), in_zp=in_zp, w_zp=-4)
    assert st == capi.VALID and ctx.last_kernel == "gemm_mfma_i8"
    assert np.array_equal(got, cases.conv2d_exact_blas(x, w, bias, (1, 1, 1, 1), (1, 1), (1, 1), in_zp, -4))


@pytest.mark.parametrize("shape", TAP_SHAPES + FP_TAP_SHAPES)
@pytest.mark.parametrize("kind", ["fp16", "bf16"])
def test_conv2d_taps_fp_gemm_within_dot_product_bound(ctx, shape, kind):
    n, ih, iw, ic, oc, kh, kw, pad, stride, dil = shape
    rng = np.random.default_rng(31 + ic + kh)
    x = rng.normal(0, 1, (n, ih, iw, ic)).astype(np.float32)
    w = rng.normal(0, 1 / np.sqrt(kh * kw * ic), (oc, kh, kw, ic)).astype(np.float32)
    b = rng.normal(0, 0.1, oc).astype(np.float32)
    if kind == "fp16":
        xs, ws, bs = x.astype(np.float16), w.astype(np.float16), b.astype(np.float16)
        xf, wf, bf = (v.astype(np.float64) for v in (xs, ws, bs))
        dtype = capi.FP16
    else:
        xs, ws, bs = (cases.float_to_bf16_bits(v) for v in (x, w, b))
        xf, wf, bf = (cases.bf16_bits_to_float(v).astype(np.float64) for v in (xs, ws, bs))
        dtype = capi.BF16
    got, st = gpu_ops.conv2d(ctx, xs, ws, bs, pad, stride, dil, dtype=dtype)
    oh, ow = got.shape[1], got.shape[2]
    assert st == capi.VALID and ctx.last_kernel == ("gemm_mfma_f16" if kind == "fp16" else "gemm_mfma_bf16") + patch_form(
        oh, ow, ic * 2, oc, kh, kw, stride, dil)
    imp = got.astype(np.float64) if kind == "fp16" else cases.bf16_bits_to_float(got).astype(np.float64)
    # reference and bound from the device's fp64 precise / bounds passes, which the fp64 oracle pins bit for bit
    oh, ow = got.shape[1], got.shape[2]
    d = ctx.conv_desc(dtype, dtype, xs.shape, oc, kh, kw, (oh, ow), pad, stride, dil, oc)
    tx, tw, tb = ctx.upload(xs, dtype), ctx.upload(ws, dtype), ctx.upload(bs, dtype)
    ref, bnd = ctx.empty(got.shape, capi.F64), ctx.empty(got.shape, capi.F64)
    try:
        ctx.conv2d_precise(d, tx, tw, tb, False, ref)
        ctx.conv2d_precise(d, tx, tw, tb, True, bnd)
        assert ctx.sync() == capi.VALID
        ref_h, bnd_h = ref.numpy(), bnd.numpy()
    finally:
        for t in list(ctx._owned):
            ctx._free(t)
    res = dp.check(imp, ref_h, bnd_h, kind, dp.kernel_size_bound(kh * kw * ic, kind))
    # tolerance: |imp-ref| <= 2*ksb * max(bnd*2^-(1+frac), normal_min) per element, sum err^2 <= 1.6*ksb*T
    assert res["ok"], res
    sub = oracle.conv2d("f64", xf[-1:, -6:], wf[:2], bf[:2], (0, pad[1], pad[2], pad[3]), stride, dil) if stride == (1, 1) and dil == (1, 1) and kh <= 6 else None
    if sub is not None:     # the bottom rows of the last image against the oracle's own loop nest
        rows = sub.shape[1]
        assert np.allclose(imp[-1:, -rows:, :, :2], sub, rtol=2.0 ** -6, atol=2.0 ** -8)


# ---- int8 convolutions with a fused RESCALE (+ CLAMP) and a non-zero input zero point through the GEMM kernel ----
def _fused(ctx, c, out_dtype=np.int8):
    got, st = gpu_ops.conv2d(ctx, c["x"], c["w"], c["bias"], c["pad"], c["stride"], c["dilation"], c["in_zp"], c["w_zp"],
                             rescale=dict(mult=c["mult"], shift=c["shift"], out_zp=c["out_zp"], out_dtype=out_dtype),
                             clamp=c["clamp"])
    acc = cases.conv2d_exact_blas(c["x"], c["w"], c["bias"], c["pad"], c["stride"], c["dilation"], c["in_zp"], c["w_zp"])
    want, wst = oracle.rescale(acc, c["mult"], c["shift"], out_zp=c["out_zp"], out_dtype=out_dtype)
    if c["clamp"] is not None:
        want = oracle.clamp(want, *c["clamp"])
    return got, st, want, wst


FUSED_SHAPES = [  # n, ih, iw, ic, oc, kh, kw, pad, stride
    (8, 56, 56, 64, 64, 3, 3, (1, 1, 1, 1), (1, 1)),        # the headline layer's geometry
    (16, 28, 28, 256, 256, 3, 3, (1, 1, 1, 1), (1, 1)),
    (16, 28, 28, 256, 520, 1, 1, (0, 0, 0, 0), (1, 1)),     # pointwise, ragged channel tiles
    (40, 31, 29, 64, 136, 3, 3, (1, 1, 1, 1), (2, 2)),
]


@pytest.mark.parametrize("shape", FUSED_SHAPES)
@pytest.mark.parametrize("zps", [(4, 0, -3), (-128, 7, 100), (0, 0, 0)])
@pytest.mark.parametrize("out_dtype", [np.int8, np.int16])
def test_conv2d_fused_rescale_gemm_bit_exact(ctx, shape, zps, out_dtype):
    n, ih, iw, ic, oc, kh, kw, pad, stride = shape
    rng = np.random.default_rng(ih + oc + kh)
    c = dict(x=rng.integers(-128, 128, (n, ih, iw, ic)).astype(np.int8),
             w=np.clip(np.rint(rng.normal(0, 40, (oc, kh, kw, ic))), -127, 127).astype(np.int8),
             bias=rng.integers(-(1 << 16), 1 << 16, oc).astype(np.int32), in_zp=zps[0], w_zp=zps[1],
             pad=pad, stride=stride, dilation=(1, 1), mult=rng.integers(1 << 30, 1 << 31, oc).astype(np.int32),
             shift=rng.integers(36, 44, oc).astype(np.int8), out_zp=zps[2] if out_dtype == np.int8 else 0,
             clamp=(-100, 110) if out_dtype == np.int8 else None)
    got, st, want, wst = _fused(ctx, c, out_dtype)
    assert ctx.last_kernel == "gemm_mfma_i8_rescale" + patch_form(got.shape[1], got.shape[2], ic, oc, kh, kw, stride, (1, 1))
    assert st == wst == capi.VALID and np.array_equal(got, want), int(np.count_nonzero(got != want))
    assert len(np.unique(got)) > 50     # the scale keeps the results inside the output range


def test_conv2d_fused_rescale_gemm_reports_require_conditions(ctx):
    """a shift below 32 makes apply_scale_32 check the value range (quant_util.h:59-67): UNPREDICTABLE, as the
    oracle says for the same operands"""
    n, ih, iw, ic, oc = 16, 28, 28, 256, 256
    rng = np.random.default_rng(3)
    c = dict(x=rng.integers(-128, 128, (n, ih, iw, ic)).astype(np.int8),
             w=rng.integers(-127, 128, (oc, 3, 3, ic)).astype(np.int8), bias=np.zeros(oc, np.int32), in_zp=3, w_zp=0,
             pad=(1, 1, 1, 1), stride=(1, 1), dilation=(1, 1), mult=np.full(oc, 1 << 30, np.int32),
             shift=np.full(oc, 12, np.int8), out_zp=0, clamp=None)
    got, st, want, wst = _fused(ctx, c)
    assert ctx.last_kernel == "gemm_mfma_i8_rescale_patch"
    assert st == wst == capi.UNPREDICTABLE and ctx.flags & capi.FLAG_SCALE_VALUE


# ---- which MFMA kernel a convolution gets when the choice is left open ----
@pytest.mark.parametrize("dtype, shape, kernel", [
    # n, ih, iw, ic, oc, k, pad[, stride]
    (capi.INT8, (8, 56, 56, 192, 64, 3, 1), "conv2d_mfma_i8"),         # 3x3 int8: the patch kernel
    (capi.INT8, (16, 28, 28, 256, 256, 3, 1), "gemm_mfma_i8_patch"),   # 3x3 int8 whose patch the GEMM kernel can keep in LDS
    (capi.INT8, (16, 28, 28, 1024, 256, 3, 1), "conv2d_mfma_i8"),      # 3x3 int8 whose patch (6 x 30 x 1 KB) does not fit
    (capi.INT8, (16, 14, 14, 1024, 1024, 1, 0), "gemm_mfma_i8"),       # pointwise: the GEMM kernel
    (capi.INT8, (64, 28, 28, 256, 256, 3, 1, 2), "gemm_mfma_i8"),      # 3x3 int8 with stride 2 and 200 tiles: the GEMM kernel
    (capi.INT8, (32, 28, 28, 256, 256, 3, 1, 2), "conv2d_mfma_i8"),    # the same with 100 tiles: the patch kernel
    (capi.INT8, (20, 28, 28, 1024, 256, 3, 1), "gemm_mfma_i8"),        # 3x3 int8 outside the patch form, 246 tiles: the GEMM kernel
    (capi.INT8, (64, 7, 7, 512, 512, 3, 1), "gemm_mfma_i8"),           # images smaller than a tile, 100 tiles: the GEMM kernel
    (capi.FP16, (16, 28, 28, 256, 256, 3, 1), "gemm_mfma_f16_patch"),  # 3x3 fp16, deep K, the patch fits the LDS
    (capi.FP16, (8, 28, 28, 512, 512, 3, 1), "gemm_mfma_f16"),         # the same with a patch that does not fit
    (capi.FP16, (4, 28, 28, 256, 256, 3, 1), "gemm_mfma_f16_patch"),   # 56 tiles of four output rows: enough for the patch form
    (capi.INT8, (16, 14, 14, 256, 256, 3, 1), "conv2d_ksplit_i8"),     # 50 tiles, 1.8 G multiply-adds: K split over the waves of small workgroups
    (capi.INT8, (32, 14, 14, 256, 256, 3, 1), "conv2d_mfma_i8"),       # 98 tiles, 3.7 G: too much for that, too few tiles for the GEMM kernel
    (capi.INT8, (8, 14, 14, 1024, 512, 1, 0), "conv2d_slab_i8"),       # pointwise on 1024 channels, one round of workgroups: the slab kernel
    (capi.INT8, (8, 7, 7, 2048, 512, 1, 0), "conv2d_pointwise_ksplit_i8"),    # 2048 channels, 411 M multiply-adds on 16 tiles: K split over waves
    (capi.INT8, (8, 28, 28, 512, 256, 1, 0), "conv2d_slab_i8"),        # pointwise on 512 channels, one round of workgroups: the slab kernel
    (capi.INT8, (16, 28, 28, 512, 256, 1, 0), "gemm_mfma_i8"),         # two rounds: the GEMM kernel
    (capi.FP16, (2, 28, 28, 256, 256, 3, 1), "conv2d_mfma_f16"),       # 28 tiles: too few
    (capi.FP16, (1, 14, 14, 1024, 1024, 1, 0), "gemm_mfma_f16"),       # pointwise with 16 tiles: still the GEMM kernel
    (capi.FP16, (64, 7, 7, 512, 512, 3, 1), "gemm_mfma_f16"),          # 3x3, no patch form (49 pixels a tile), 100 tiles
    (capi.FP16, (32, 7, 7, 512, 512, 3, 1), "conv2d_mfma_f16"),        # the same with 52 tiles: the patch kernel
    (capi.FP16, (8, 56, 56, 64, 64, 3, 1), "conv2d_slab_f16"),         # 3x3 fp16 on 128-byte channel vectors: the slab kernel
    (capi.FP16, (8, 56, 56, 64, 128, 3, 1), "conv2d_slab_f16"),        # the same with 128 output channels
    (capi.FP16, (32, 56, 56, 64, 128, 3, 1, 2), "gemm_mfma_f16"),      # and with stride 2, 196 tiles: the GEMM kernel's taps form
    (capi.FP16, (16, 56, 56, 128, 64, 3, 1), "conv2d_mfma_f16"),       # 128 channels in, 64 out: half of the GEMM kernel's tile empty
    (capi.FP16, (16, 56, 56, 128, 96, 3, 1), "gemm_mfma_f16"),         # 96 out
    (capi.FP16, (16, 56, 56, 64, 128, 3, 1, 2), "conv2d_slab_f16"),    # 98 tiles: the slab kernel
    (capi.FP16, (8, 56, 56, 64, 256, 1, 0), "gemm_mfma_f16"),          # pointwise with two blocks of K
    (capi.INT8, (8, 56, 56, 64, 256, 1, 0), "gemm_mfma_i8"),           # int8 pointwise, int32 results, 6.4 M of them: before the slab kernel
    (capi.INT8, (8, 56, 56, 64, 64, 1, 0), "conv2d_pointwise_i8"),     # the same with 1.6 M results: the pointwise kernel
    (capi.INT8, (8, 28, 28, 128, 128, 1, 0), "conv2d_slab_i8"),        # 128 input channels: the slab kernel
    (capi.INT8, (8, 28, 28, 128, 24, 1, 0), "conv2d_pointwise_i8"),    # too few output channels for it: the pointwise kernel
    (capi.INT8, (8, 56, 56, 16, 96, 1, 0), "conv2d_pointwise_i8"),     # int8 pointwise with a short channel vector
    (capi.INT8, (8, 28, 28, 144, 32, 1, 0), "conv2d_pointwise_i8"),    # 144 input channels: no slab kernel
])
def test_automatic_kernel_choice(dtype, shape, kernel):
    n, ih, iw, ic, oc, k, pad = shape[:7]
    stride = shape[7] if len(shape) > 7 else 1
    pads = (pad,) * 4 if stride == 1 else (pad, pad - 1, pad, pad - 1)    # 28 + 1 - 3 is a multiple of 2
    rng = np.random.default_rng(ic + oc + k)
    if dtype == capi.INT8:
        x = rng.integers(-128, 128, (n, ih, iw, ic)).astype(np.int8)
        w = rng.integers(-128, 128, (oc, k, k, ic)).astype(np.int8)
        b = rng.integers(-999, 999, oc).astype(np.int32)
    else:
        x = rng.normal(0, 1, (n, ih, iw, ic)).astype(np.float16)
        w = rng.normal(0, 0.05, (oc, k, k, ic)).astype(np.float16)
        b = rng.normal(0, 1, oc).astype(np.float16)
    c = Context(0)
    try:
        got, st = gpu_ops.conv2d(c, x, w, b, pads, (stride, stride), dtype=dtype)
        assert st == capi.VALID and c.last_kernel == kernel
        # the kernel not chosen, where it takes the shape at all
        c.set_kernel_choice(capi.KERNEL_GEMM if kernel.startswith("conv2d") and "pointwise" not in kernel else capi.KERNEL_MFMA)
        try:
            other, st = gpu_ops.conv2d(c, x, w, b, pads, (stride, stride), dtype=dtype)
        except TmiError:
            # the GEMM kernel refuses layers with too few tiles; the patch kernel, which takes any shape, is then
            # the only one
            assert kernel.startswith("conv2d") and n * ih * iw < 128 * 48
            return
        assert st == capi.VALID and c.last_kernel != kernel
    finally:
        c.close()
    if dtype == capi.INT8:      # both kernels give the one exact result
        assert np.array_equal(got, other)
    else:                       # the same products in fp32, summed in a different order
        assert np.allclose(got.astype(np.float32), other.astype(np.float32), rtol=2.0 ** -8, atol=2.0 ** -6)
