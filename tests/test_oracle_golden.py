"""Pins the CPU oracle against the one integer golden the reference ships for the path:
examples/test_conv2d_1x1_1x32x32x8_qi8_st11_padSAME_dilat11 (int8 CONV2D -> per-channel
DOUBLE_ROUND RESCALE), the graph run by examples/run_ref_model_examples.sh."""
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
