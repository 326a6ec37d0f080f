"""The DOT_PRODUCT data sets S0..S5 against the goldens of the reference's generator tests
(reference_model/test/generate_tests.cpp), bit for bit (CPU only)."""
import numpy as np
import pytest

import oracle

# generate_tests.cpp:315-372: MATMUL fp32, in1 [4,8,2] (param 0) and in2 [4,2,5] (param 1), ks 2: first three values
MATMUL_FIRST3 = {
    (0, 0): [0xbf665aa4, 0xbf736bd3, 0x0], (0, 1): [0x0, 0x0, 0x3f34f2dd],
    (1, 0): [0xdf0a6310, 0xdf114c5a, 0x5f07324b], (1, 1): [0x5ef54579, 0xdec1c31e, 0xdf06758a],
    (2, 0): [0x3f800000, 0x3f14567c, 0x3f800000], (2, 1): [0x3f800000, 0x3f800000, 0x3f800000],
    (3, 0): [0x41800000, 0x3fee6533, 0x41800000], (3, 1): [0xc1800000, 0x41800000, 0xc1800000],
    (4, 0): [0x0, 0xbf000000, 0x0], (4, 1): [0x5dee53e9, 0xdf0cfb23, 0x5f06cb46],
    (5, 0): [0x5df6c4b3, 0x5e6b4088, 0x5ed0fe71], (5, 1): [0xde086d85, 0x5e630878, 0x5eba5c7b],
}

# generate_tests.cpp:444-535: CONV2D fp32, input [1,8,2,4] kernel [2,2], weight [2,2,2,4], bias [2], ks 16: last three
CONV2D_LAST3 = {
    (0, 0): [0x0, 0xbf28bfda, 0xbe99cd47], (0, 1): [0x0, 0x3f648dfd, 0xbd4cb21c], (0, 2): [0x0, 0x0],
    (1, 0): [0x5e4abec5, 0x5e344527, 0x5e684251], (1, 1): [0x5e1b7bf7, 0x5e77c9f4, 0x5e0ebaf2], (1, 2): [0xfd341535, 0x7d582f77],
    (2, 0): [0xbc23026a, 0xbe674c38, 0x3d3d9f96], (2, 1): [0x3d1beb31, 0xbdc7501e, 0x3cc9f5fe], (2, 2): [0x0, 0x0],
    (3, 0): [0xbe00da48, 0x3fb5b808, 0x3e22a8bd], (3, 1): [0xbd725091, 0xbfeaaf15, 0xbfb8b23f], (3, 2): [0x0, 0x0],
    (4, 0): [0xddcab121, 0x5d1b5485, 0xdda4bb36], (4, 1): [0xdde07221, 0xde696320, 0x0], (4, 2): [0x0, 0x0],
    (5, 0): [0x5e719fb9, 0x5e6b329c, 0xdd7617d4], (5, 1): [0xde42f57a, 0x5dd68799, 0xde2ddfcb], (5, 2): [0x0, 0x0],
}

# generate_tests.cpp:1194-1222: DEPTHWISE_CONV2D fp16 (fp16 accumulator), input [1,6,3,4] kernel [1,3], weight
# [1,3,4,2], bias [2], ks 3: first three values
DEPTHWISE_FIRST3_FP16 = {
    (0, 0): [0xbb33, 0xbb9b, 0x0], (0, 1): [0x0, 0x0, 0x39a8], (0, 2): [0x0, 0x0],
    (1, 0): [0xd77d, 0xd7dc, 0x5750], (1, 1): [0x56a2, 0xd53e, 0xd746], (1, 2): [0xf1f9, 0x732c],
}


@pytest.mark.parametrize("key", sorted(MATMUL_FIRST3))
def test_matmul_sets(key):
    s, p = key
    got = oracle.dot_product_data("matmul", s, p, 2, (4, 8, 2) if p == 0 else (4, 2, 5))
    want = MATMUL_FIRST3[key]
    assert got.ravel()[:len(want)].view(np.uint32).tolist() == want


@pytest.mark.parametrize("key", sorted(CONV2D_LAST3))
def test_conv2d_sets(key):
    s, p = key
    shape = [(1, 8, 2, 4), (2, 2, 2, 4), (2,)][p]
    got = oracle.dot_product_data("conv2d", s, p, 16, shape, kernel=(2, 2) if p == 0 else None)
    want = CONV2D_LAST3[key]
    assert got.ravel()[-len(want):].view(np.uint32).tolist() == want


@pytest.mark.parametrize("key", sorted(DEPTHWISE_FIRST3_FP16))
def test_depthwise_sets_fp16(key):
    s, p = key
    shape = [(1, 6, 3, 4), (1, 3, 4, 2), (2,)][p]
    got = oracle.dot_product_data("depthwise", s, p, 3, shape, kind="fp16", kernel=(1, 3) if p == 0 else None, acc16=True)
    want = DEPTHWISE_FIRST3_FP16[key]
    assert got.astype(np.float16).ravel()[:len(want)].view(np.uint16).tolist() == want


def test_set_properties():
    """what the sets are for: S0 pairs every non-zero with a zero; S2 / S3 put the large value first in each
    dot product; values stay inside the operand type's range"""
    a = oracle.dot_product_data("matmul", 0, 0, 64, (2, 16, 64))
    b = oracle.dot_product_data("matmul", 0, 1, 64, (2, 64, 8))
    assert np.all(np.matmul(np.abs(a.astype(np.float64)), np.abs(b.astype(np.float64))) >= 0)
    a2 = oracle.dot_product_data("matmul", 2, 0, 64, (2, 16, 64))
    assert np.all(a2[..., 0] == 1.0) and np.all(np.abs(a2[..., 1:]) <= 1 / 8)
    a3 = oracle.dot_product_data("matmul", 3, 0, 64, (2, 16, 64))
    assert np.all(np.abs(a3[..., 0]) == 16.0)
    for s in range(6):
        h = oracle.dot_product_data("matmul", s, 0, 64, (2, 16, 64), kind="fp16")
        assert np.all(np.isfinite(h.astype(np.float16)))
