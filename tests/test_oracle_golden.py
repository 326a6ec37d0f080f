"""Pins the CPU oracle against the goldens the reference ships for the path:
examples/test_conv2d_1x1_1x32x32x8_qi8_st11_padSAME_dilat11 (int8 CONV2D -> per-channel DOUBLE_ROUND RESCALE), the
graph run by examples/run_ref_model_examples.sh, and examples/test_conv2d_1x1_1x32x32x8_f32_st11_padSAME_dilat11
(FP32 CONV2D), the graph of the reference's own conv2d_f32_test (test/model_runner_tests.cpp:85-125)."""
import os

import numpy as np

import oracle
import tosa_flatbuffer as fb


def _load(golden_dir):
    d = os.path.join(golden_dir, "qi8_conv2d_1x1")
    tensors, ops, inputs, outputs = fb.load_main_block(os.path.join(d, "graph.tosa"))
    x = np.load(os.path.join(d, "placeholder_0.npy"))
    want = np.load(os.path.join(d, "tflite_result.npy"))
    return tensors, ops, x, want


def _run(tensors, ops, x, rounding_mode=None):
    conv = [o for o in ops if o["op"] == fb.OP_CONV2D][0]
    resc = [o for o in ops if o["op"] == fb.OP_RESCALE][0]
    ca, ra = fb.conv_attr(conv["attr"]), fb.rescale_attr(resc["attr"])
    _, wn, bn, izn, wzn = conv["inputs"]
    acc = oracle.conv2d("i8", x, tensors[wn]["data"], tensors[bn]["data"], ca["pad"], ca["stride"], ca["dilation"],
                        in_zp=int(tensors[izn]["data"][0]), w_zp=int(tensors[wzn]["data"][0]))
    _, mn, sn, rizn, rozn = resc["inputs"]
    out, st = oracle.rescale(acc, tensors[mn]["data"], tensors[sn]["data"], in_zp=int(tensors[rizn]["data"][0]),
                             out_zp=int(tensors[rozn]["data"][0]), out_dtype=np.int8, scale32=ra["scale32"],
                             rounding_mode=rounding_mode or ra["rounding_mode"], per_channel=ra["per_channel"],
                             input_unsigned=ra["input_unsigned"], output_unsigned=ra["output_unsigned"])
    return acc, out, st


def test_graph_decodes_as_documented(golden_dir):
    tensors, ops, x, want = _load(golden_dir)
    assert [o["op"] for o in ops] == [fb.OP_CONST] * 7 + [fb.OP_CONV2D, fb.OP_RESCALE]
    assert x.dtype == np.int8 and x.shape == (1, 32, 32, 8)
    assert want.dtype == np.int8 and want.shape == (1, 32, 32, 16)
    assert tensors["layer_4"]["data"][0].ravel().tolist() == [70, -49, -44, 0, 127, 63, -84, 38]
    assert fb.rescale_attr(ops[-1]["attr"])["rounding_mode"] == oracle.ROUND_DOUBLE


def test_qi8_conv_rescale_matches_stored_golden_bit_exact(golden_dir):
    tensors, ops, x, want = _load(golden_dir)
    acc, out, st = _run(tensors, ops, x)
    assert st == oracle.VALID
    assert acc.min() == -57704 and acc.max() == 65348
    assert np.array_equal(out, want)


def test_golden_distinguishes_double_round_from_single_round(golden_dir):
    """The fixture really pins the double-round term: single rounding misses 11 elements by one."""
    tensors, ops, x, want = _load(golden_dir)
    _, out, st = _run(tensors, ops, x, rounding_mode=oracle.ROUND_SINGLE)
    assert st == oracle.VALID
    diff = out.astype(np.int32) - want.astype(np.int32)
    assert np.count_nonzero(diff) == 11 and np.abs(diff).max() == 1


# ---- the FP32 example ---------------------------------------------------------------------------------------
def _load_f32(golden_dir):
    d = os.path.join(golden_dir, "f32_conv2d_1x1")
    tensors, ops, inputs, outputs = fb.load_main_block(os.path.join(d, "graph.tosa"))
    return tensors, ops, np.load(os.path.join(d, "placeholder_0.npy")), np.load(os.path.join(d, "tflite_result.npy"))


def approx_equal(a, b):
    """doctest::Approx as the reference's compareOutput uses it (test/include/test_utils.h:186-193): the default
    epsilon is 100 float epsilons, relative to 1 + max(|a|, |b|)"""
    eps = float(np.finfo(np.float32).eps) * 100
    a64, b64 = a.astype(np.float64), b.astype(np.float64)
    return np.abs(a64 - b64) < eps * (1.0 + np.maximum(np.abs(a64), np.abs(b64)))


def test_f32_graph_decodes(golden_dir):
    tensors, ops, x, want = _load_f32(golden_dir)
    assert [o["op"] for o in ops] == [fb.OP_CONST] * 3 + [fb.OP_CONV2D]
    assert x.dtype == np.float32 and x.shape == (1, 32, 32, 8) and want.shape == (1, 32, 32, 16)
    conv = ops[-1]
    assert tensors[conv["inputs"][1]]["shape"] == [16, 1, 1, 8] and tensors[conv["inputs"][1]]["type"] == 7
    ca = fb.conv_attr(conv["attr"])
    assert ca["pad"] == [0, 0, 0, 0] and ca["stride"] == [1, 1] and ca["dilation"] == [1, 1]


def test_f32_conv_matches_stored_golden_to_the_reference_tests_tolerance(golden_dir):
    tensors, ops, x, want = _load_f32(golden_dir)
    conv = ops[-1]
    _, wn, bn, izn, wzn = conv["inputs"]
    ca = fb.conv_attr(conv["attr"])
    assert float(tensors[izn]["data"][0]) == 0.0 and float(tensors[wzn]["data"][0]) == 0.0
    got = oracle.conv2d("f32", x, tensors[wn]["data"], tensors[bn]["data"], ca["pad"], ca["stride"], ca["dilation"])
    assert got.dtype == np.float32
    assert approx_equal(got, want).all()
    assert np.array_equal(got, want)    # in fact bit for bit: eight products summed in the reference's ic order
    # the fixture is not vacuous (its bias is all zeros, so the products are what it pins): one product less breaks it
    assert not tensors[bn]["data"].any()
    short = oracle.conv2d("f32", x[..., :7], tensors[wn]["data"][..., :7], tensors[bn]["data"], ca["pad"],
                          ca["stride"], ca["dilation"])
    assert not approx_equal(short, want).all()
