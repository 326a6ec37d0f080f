"""The C++ host side (GraphNode-shaped adapters + graph runtime + file readers) through its two executables.

CPU part: the test-only FlatBuffers writer round-trips through the test-only reader, and the runner refuses to
run without a GPU (no CPU fall-back).  GPU part: the reference-style known-answer binary, the reference's
int8 example directory end to end (with and without operator fusion), and synthetic graphs against the oracle,
including the UNPREDICTABLE and ERROR exit codes."""
import json
import os
import subprocess

import numpy as np
import pytest

import cases
import oracle
import tosa_fb_writer as W
import tosa_flatbuffer as R

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
RUN = os.path.join(ROOT, "reference_model_amd", "tosa_mi355_run")
KATS = os.path.join(ROOT, "reference_model_amd", "tosa_mi355_host_kats")


def _write_case(tmp_path, raw_graph, inputs, ofm_names):
    (tmp_path / "graph.tosa").write_bytes(raw_graph)
    desc = {"tosa_file": "graph.tosa", "ifm_name": [], "ifm_file": [], "ofm_name": [], "ofm_file": []}
    for name, arr in inputs.items():
        np.save(tmp_path / f"{name}.npy", arr)
        desc["ifm_name"].append(name)
        desc["ifm_file"].append(f"{name}.npy")
    for name in ofm_names:
        desc["ofm_name"].append(name)
        desc["ofm_file"].append(f"{name}_out.npy")
    (tmp_path / "desc.json").write_text(json.dumps(desc))
    return str(tmp_path / "desc.json")


def _run(desc, *extra):
    return subprocess.run([RUN, f"--test_desc={desc}", *extra], capture_output=True, text=True, timeout=120)


def _conv_graph(c, depthwise=False, with_clamp=True, shift_override=None):
    x, w = c["x"], c["w"]
    oc = w.shape[2] * w.shape[3] if depthwise else w.shape[0]
    kh, kw = (w.shape[0], w.shape[1]) if depthwise else (w.shape[1], w.shape[2])
    oh, ow = oracle.conv_out_hw(x.shape[1], x.shape[2], kh, kw, c["pad"], c["stride"], c["dilation"])
    shift = c["shift"] if shift_override is None else shift_override
    ts = [W.tensor("x", x.shape, np.int8), W.tensor("w", w.shape, np.int8, w), W.tensor("bias", c["bias"].shape, np.int32, c["bias"]),
          W.tensor("izp", [1], np.int8, [c["in_zp"]]), W.tensor("wzp", [1], np.int8, [c["w_zp"]]),
          W.tensor("acc", [x.shape[0], oh, ow, oc], np.int32), W.tensor("mult", [oc], np.int32, c["mult"]),
          W.tensor("shift", [oc], np.int8, shift), W.tensor("rizp", [1], np.int32, [0]),
          W.tensor("rozp", [1], np.int8, [c["out_zp"]]), W.tensor("q", [x.shape[0], oh, ow, oc], np.int8),
          W.tensor("y", [x.shape[0], oh, ow, oc], np.int8)]
    ops = [W.operator(R.OP_CONST, [], [n]) for n in ("w", "bias", "izp", "wzp", "mult", "shift", "rizp", "rozp")]
    ops.append(W.operator(R.OP_DEPTHWISE_CONV2D if depthwise else R.OP_CONV2D, ["x", "w", "bias", "izp", "wzp"], ["acc"],
                          W.conv_attr(c["pad"], c["stride"], c["dilation"])))
    ops.append(W.operator(R.OP_RESCALE, ["acc", "mult", "shift", "rizp", "rozp"], ["q"], W.rescale_attr()))
    out = "q"
    if with_clamp and c["clamp"] is not None:
        ops.append(W.operator(R.OP_CLAMP, ["q"], ["y"], W.clamp_attr(*c["clamp"])))
        out = "y"
    return W.graph(ts, ops, ["x"], [out]), out


def _expect(c, depthwise=False):
    f = oracle.depthwise_conv2d if depthwise else oracle.conv2d
    acc = f("i8", c["x"], c["w"], c["bias"], c["pad"], c["stride"], c["dilation"], c["in_zp"], c["w_zp"])
    want, _ = oracle.rescale(acc, c["mult"], c["shift"], out_zp=c["out_zp"])
    return want if c["clamp"] is None else oracle.clamp(want, *c["clamp"])


# ---- CPU ----------------------------------------------------------------------------------------------------
def test_writer_round_trips_through_reader(tmp_path):
    c = cases.c3(n=1, hw=6)
    raw, out = _conv_graph(c)
    p = tmp_path / "g.tosa"
    p.write_bytes(raw)
    tensors, ops, ins, outs = R.load_main_block(str(p))
    assert ins == ["x"] and outs == [out]
    assert [o["op"] for o in ops][-3:] == [R.OP_CONV2D, R.OP_RESCALE, R.OP_CLAMP]
    assert np.array_equal(tensors["w"]["data"], c["w"]) and np.array_equal(tensors["mult"]["data"], c["mult"])
    assert R.conv_attr(ops[-3]["attr"])["pad"] == [1, 1, 1, 1]
    assert R.rescale_attr(ops[-2]["attr"]) == dict(scale32=True, rounding_mode=3, per_channel=True,
                                                   input_unsigned=False, output_unsigned=False)


def test_runner_refuses_to_run_without_a_gpu(golden_dir):
    import torch
    if torch.cuda.is_available():
        pytest.skip("a GPU is present")
    assert os.path.exists(RUN), "build the host side first: python -m reference_model_amd.build"
    r = _run(os.path.join(golden_dir, "qi8_conv2d_1x1", "desc.json"), "--ofm_file=/tmp/should_not_exist.npy")
    assert r.returncode == 2 and "no CPU fall-back" in r.stderr
    assert not os.path.exists("/tmp/should_not_exist.npy")


# ---- GPU ----------------------------------------------------------------------------------------------------
@pytest.mark.gpu
def test_reference_style_known_answer_binary():
    r = subprocess.run([KATS], capture_output=True, text=True, timeout=120)
    assert r.returncode == 0, r.stdout + r.stderr
    assert r.stdout.count("PASS") == 23 and "FAIL" not in r.stdout


@pytest.mark.gpu
@pytest.mark.parametrize("fusion", [True, False])
def test_reference_qi8_example_directory(golden_dir, tmp_path, fusion):
    out = str(tmp_path / "out.npy")
    args = [f"--ofm_file={out}"] + ([] if fusion else ["--no_fusion"])
    r = _run(os.path.join(golden_dir, "qi8_conv2d_1x1", "desc.json"), *args)
    assert r.returncode == 0, r.stderr
    want = np.load(os.path.join(golden_dir, "qi8_conv2d_1x1", "tflite_result.npy"))
    got = np.load(out)
    assert got.dtype == np.int8 and np.array_equal(got, want)
    assert ("kernels launched: 1, nodes folded into a producer: 1" if fusion else
            "kernels launched: 2, nodes folded into a producer: 0") in r.stderr


@pytest.mark.gpu
def test_reference_f32_example_directory(golden_dir, tmp_path):
    """the graph of the reference's conv2d_f32_test (test/model_runner_tests.cpp:85-125), compared the way that test
    compares: doctest::Approx with its default epsilon (100 float epsilons relative to 1 + |value|)"""
    out = str(tmp_path / "out.npy")
    r = _run(os.path.join(golden_dir, "f32_conv2d_1x1", "desc.json"), f"--ofm_file={out}")
    assert r.returncode == 0, r.stderr
    want = np.load(os.path.join(golden_dir, "f32_conv2d_1x1", "tflite_result.npy")).astype(np.float64)
    got = np.load(out)
    assert got.dtype == np.float32 and got.shape == want.shape
    eps = float(np.finfo(np.float32).eps) * 100
    assert (np.abs(got - want) < eps * (1.0 + np.maximum(np.abs(got), np.abs(want)))).all()
    assert np.array_equal(got, want.astype(np.float32))    # the same eight products in the same order: bit for bit


@pytest.mark.gpu
@pytest.mark.parametrize("which", ["conv_rescale_clamp", "depthwise_rescale"])
def test_synthetic_graphs_match_oracle(tmp_path, which):
    depthwise = which == "depthwise_rescale"
    c = cases.c4(n=2, hw=20, c=32) if depthwise else cases.c3(n=2, hw=14)
    raw, out = _conv_graph(c, depthwise=depthwise)
    desc = _write_case(tmp_path, raw, {"x": c["x"]}, [out])
    for extra in ([], ["--no_fusion"]):
        r = _run(desc, *extra)
        assert r.returncode == 0, r.stderr
        assert np.array_equal(np.load(tmp_path / f"{out}_out.npy"), _expect(c, depthwise)), extra
    assert "nodes folded into a producer: 0" in r.stderr


@pytest.mark.gpu
def test_matmul_graph(tmp_path):
    rng = np.random.default_rng(4)
    a = rng.integers(-128, 128, (2, 40, 96)).astype(np.int8)
    b = rng.integers(-128, 128, (2, 96, 24)).astype(np.int8)
    ts = [W.tensor("a", a.shape, np.int8), W.tensor("b", b.shape, np.int8), W.tensor("azp", [1], np.int8, [-5]),
          W.tensor("bzp", [1], np.int8, [3]), W.tensor("o", [2, 40, 24], np.int32)]
    ops = [W.operator(R.OP_CONST, [], ["azp"]), W.operator(R.OP_CONST, [], ["bzp"]),
           W.operator(R.OP_MATMUL, ["a", "b", "azp", "bzp"], ["o"])]
    desc = _write_case(tmp_path, W.graph(ts, ops, ["a", "b"], ["o"]), {"a": a, "b": b}, ["o"])
    r = _run(desc)
    assert r.returncode == 0, r.stderr
    assert np.array_equal(np.load(tmp_path / "o_out.npy"), oracle.matmul("i8", a, b, -5, 3))


@pytest.mark.gpu
def test_transpose_conv2d_and_conv3d_graphs(tmp_path):
    """TRANSPOSE_CONV2D feeding a RESCALE, and a CONV3D, loaded from flatbuffers and run on the device."""
    rng = np.random.default_rng(9)
    x = rng.integers(-128, 128, (1, 6, 7, 16)).astype(np.int8)
    w = rng.integers(-128, 128, (8, 3, 3, 16)).astype(np.int8)
    bias = rng.integers(-999, 999, 8).astype(np.int32)
    out_pad, stride = (0, 1, -1, 0), (2, 2)
    acc = oracle.transpose_conv2d("i8", x, w, bias, out_pad, stride, in_zp=-4, w_zp=0)
    mult = rng.integers(1 << 30, 1 << 31, 8).astype(np.int32)
    shift = np.full(8, 40, np.int8)
    ts = [W.tensor("x", x.shape, np.int8), W.tensor("w", w.shape, np.int8, w), W.tensor("bias", [8], np.int32, bias),
          W.tensor("izp", [1], np.int8, [-4]), W.tensor("wzp", [1], np.int8, [0]), W.tensor("acc", acc.shape, np.int32),
          W.tensor("mult", [8], np.int32, mult), W.tensor("shift", [8], np.int8, shift),
          W.tensor("rizp", [1], np.int32, [0]), W.tensor("rozp", [1], np.int8, [3]), W.tensor("q", acc.shape, np.int8)]
    ops = [W.operator(R.OP_CONST, [], [n]) for n in ("w", "bias", "izp", "wzp", "mult", "shift", "rizp", "rozp")]
    ops.append(W.operator(10, ["x", "w", "bias", "izp", "wzp"], ["acc"], W.transpose_conv_attr(out_pad, stride)))
    ops.append(W.operator(R.OP_RESCALE, ["acc", "mult", "shift", "rizp", "rozp"], ["q"], W.rescale_attr()))
    d1 = tmp_path / "tconv"
    d1.mkdir()
    r = _run(_write_case(d1, W.graph(ts, ops, ["x"], ["q"]), {"x": x}, ["q"]))
    assert r.returncode == 0, r.stderr
    want, st = oracle.rescale(acc, mult, shift, out_zp=3, out_dtype=np.int8)
    assert st == oracle.VALID and np.array_equal(np.load(d1 / "q_out.npy"), want)

    x3 = rng.integers(-128, 128, (1, 4, 5, 5, 8)).astype(np.int8)
    w3 = rng.integers(-128, 128, (4, 2, 3, 3, 8)).astype(np.int8)
    b3 = np.array([17], np.int32)
    pad, st3, dil = (1, 0, 1, 1, 1, 1), (1, 1, 1), (1, 1, 1)
    want3 = oracle.conv3d("i8", x3, w3, b3, pad, st3, dil, in_zp=2, w_zp=-1)
    ts = [W.tensor("x", x3.shape, np.int8), W.tensor("w", w3.shape, np.int8, w3), W.tensor("bias", [1], np.int32, b3),
          W.tensor("izp", [1], np.int8, [2]), W.tensor("wzp", [1], np.int8, [-1]), W.tensor("o", want3.shape, np.int32)]
    ops = [W.operator(R.OP_CONST, [], [n]) for n in ("w", "bias", "izp", "wzp")]
    ops.append(W.operator(4, ["x", "w", "bias", "izp", "wzp"], ["o"], W.conv_attr(pad, st3, dil)))
    d2 = tmp_path / "conv3d"
    d2.mkdir()
    r = _run(_write_case(d2, W.graph(ts, ops, ["x"], ["o"]), {"x": x3}, ["o"]))
    assert r.returncode == 0, r.stderr
    assert np.array_equal(np.load(d2 / "o_out.npy"), want3)
    # a malformed node is rejected when the graph is validated: exit code 2
    ops[-1] = W.operator(4, ["x", "w", "bias", "izp", "wzp"], ["o"], W.conv_attr((1, 0, 1, 1, 1, 1), (2, 1, 1), dil))
    d3 = tmp_path / "bad"
    d3.mkdir()
    r = _run(_write_case(d3, W.graph(ts, ops, ["x"], ["o"]), {"x": x3}, ["o"]))
    assert r.returncode == 2 and "exact integer output dimensions" in r.stderr


@pytest.mark.gpu
def test_exit_codes_unpredictable_and_error(tmp_path):
    c = cases.c1()
    # shift 12 admits |acc| < 2^11 only: apply_scale_32's value REQUIRE fires -> exit code 1, output still written
    raw, out = _conv_graph(c, shift_override=np.full(16, 12, np.int8))
    d1 = tmp_path / "u"
    d1.mkdir()
    r = _run(_write_case(d1, raw, {"x": c["x"]}, [out]))
    assert r.returncode == 1 and "UNPREDICTABLE" in r.stderr
    # declared output shape that violates the convolution shape rule -> rejected by validateGraph, exit code 2
    bad = dict(c)
    bad["pad"] = (1, 0, 0, 0)
    raw_bad, out = _conv_graph(bad)
    raw_ok, _ = _conv_graph(c)
    d2 = tmp_path / "e"
    d2.mkdir()
    # take the good graph's tensors but the bad attribute by rebuilding with mismatching pad vs declared output
    ts_ops = _conv_graph(c)  # noqa: F841  (documented intent; the mismatch below is what is tested)
    x = c["x"]
    ts = [W.tensor("x", x.shape, np.int8), W.tensor("w", c["w"].shape, np.int8, c["w"]),
          W.tensor("bias", [16], np.int32, c["bias"]), W.tensor("z", [1], np.int8, [0]),
          W.tensor("acc", [1, 32, 32, 16], np.int32)]
    ops = [W.operator(R.OP_CONST, [], [n]) for n in ("w", "bias", "z")]
    ops.append(W.operator(R.OP_CONV2D, ["x", "w", "bias", "z", "z"], ["acc"], W.conv_attr([1, 0, 0, 0], [1, 1], [1, 1])))
    r = _run(_write_case(d2, W.graph(ts, ops, ["x"], ["acc"]), {"x": x}, ["acc"]))
    assert r.returncode == 2 and "Mismatch between output shape provided and expected output shape" in r.stderr
    assert not (d2 / "acc_out.npy").exists()
    # an operator outside the accelerated path (ADD = 15) is refused loudly rather than evaluated on the host
    ts = [W.tensor("x", [4], np.int32), W.tensor("y", [4], np.int32)]
    d3 = tmp_path / "o"
    d3.mkdir()
    r = _run(_write_case(d3, W.graph(ts, [W.operator(15, ["x", "x"], ["y"])], ["x"], ["y"]),
                         {"x": np.arange(4, dtype=np.int32)}, ["y"]))
    assert r.returncode == 2 and "outside the accelerated path" in r.stderr
    # a tensor that an operator names with a dimension of zero: the reference never allocates it and calls the graph
    # UNPREDICTABLE (subgraph_traverser.cpp:579-590) -> exit code 1, nothing written
    x0 = np.zeros((0, 32, 32, 8), np.int8)
    ts = [W.tensor("x", x0.shape, np.int8), W.tensor("w", c["w"].shape, np.int8, c["w"]),
          W.tensor("bias", [16], np.int32, c["bias"]), W.tensor("z", [1], np.int8, [0]),
          W.tensor("acc", [0, 32, 32, 16], np.int32)]
    ops = [W.operator(R.OP_CONST, [], [n]) for n in ("w", "bias", "z")]
    ops.append(W.operator(R.OP_CONV2D, ["x", "w", "bias", "z", "z"], ["acc"], W.conv_attr([0, 0, 0, 0], [1, 1], [1, 1])))
    d4 = tmp_path / "z"
    d4.mkdir()
    r = _run(_write_case(d4, W.graph(ts, ops, ["x"], ["acc"]), {"x": x0}, ["acc"]))
    assert r.returncode == 1 and "UNPREDICTABLE" in r.stderr and "invalid dimension of 0" in r.stderr
    assert not (d4 / "acc_out.npy").exists()


@pytest.mark.gpu
def test_pooling_graph(tmp_path):
    """CONV2D -> RESCALE -> MAX_POOL2D -> AVG_POOL2D: the int8 tail of a classifier block, loaded from a flatbuffer
    and run on the device; every intermediate stays there."""
    rng = np.random.default_rng(21)
    x = rng.integers(-128, 128, (2, 12, 12, 16)).astype(np.int8)
    w = rng.integers(-128, 128, (32, 3, 3, 16)).astype(np.int8)
    bias = rng.integers(-999, 999, 32).astype(np.int32)
    acc = oracle.conv2d("i8", x, w, bias, (1, 1, 1, 1), (1, 1), (1, 1), in_zp=3, w_zp=0)
    mult = rng.integers(1 << 30, 1 << 31, 32).astype(np.int32)
    shift = np.full(32, 41, np.int8)
    q, st = oracle.rescale(acc, mult, shift, out_zp=-2, out_dtype=np.int8)
    mp = oracle.max_pool2d(q, (2, 2), (2, 2))
    ap = oracle.avg_pool2d(mp, (3, 3), (3, 3), in_zp=-2, out_zp=5)
    assert st == oracle.VALID
    ts = [W.tensor("x", x.shape, np.int8), W.tensor("w", w.shape, np.int8, w), W.tensor("bias", [32], np.int32, bias),
          W.tensor("izp", [1], np.int8, [3]), W.tensor("wzp", [1], np.int8, [0]), W.tensor("acc", acc.shape, np.int32),
          W.tensor("mult", [32], np.int32, mult), W.tensor("shift", [32], np.int8, shift),
          W.tensor("rizp", [1], np.int32, [0]), W.tensor("rozp", [1], np.int8, [-2]), W.tensor("q", q.shape, np.int8),
          W.tensor("mp", mp.shape, np.int8), W.tensor("aizp", [1], np.int8, [-2]), W.tensor("aozp", [1], np.int8, [5]),
          W.tensor("ap", ap.shape, np.int8)]
    ops = [W.operator(R.OP_CONST, [], [n]) for n in ("w", "bias", "izp", "wzp", "mult", "shift", "rizp", "rozp", "aizp", "aozp")]
    ops.append(W.operator(3, ["x", "w", "bias", "izp", "wzp"], ["acc"], W.conv_attr((1, 1, 1, 1), (1, 1), (1, 1))))
    ops.append(W.operator(R.OP_RESCALE, ["acc", "mult", "shift", "rizp", "rozp"], ["q"], W.rescale_attr()))
    ops.append(W.operator(8, ["q"], ["mp"], W.pool_attr((2, 2), (2, 2), (0, 0, 0, 0), 1)))
    ops.append(W.operator(2, ["mp", "aizp", "aozp"], ["ap"], W.pool_attr((3, 3), (3, 3), (0, 0, 0, 0), 5)))
    d1 = tmp_path / "pool"
    d1.mkdir()
    r = _run(_write_case(d1, W.graph(ts, ops, ["x"], ["ap", "mp"]), {"x": x}, ["ap", "mp"]))
    assert r.returncode == 0, r.stderr
    assert np.array_equal(np.load(d1 / "mp_out.npy"), mp) and np.array_equal(np.load(d1 / "ap_out.npy"), ap)
    # a window that does not tile the input is rejected when the graph is validated
    ops[-1] = W.operator(2, ["mp", "aizp", "aozp"], ["ap"], W.pool_attr((4, 4), (3, 3), (0, 0, 0, 0), 5))
    d2 = tmp_path / "bad"
    d2.mkdir()
    r = _run(_write_case(d2, W.graph(ts, ops, ["x"], ["ap"]), {"x": x}, ["ap"]))
    assert r.returncode == 2 and "exact integer output dimensions" in r.stderr


@pytest.mark.gpu
def test_int48_rescale_graph(tmp_path):
    """RESCALE of an INT48 tensor (the accumulator type of 16-bit convolutions): the graph input arrives as an
    int64 .npy file, a constant INT48 operand as 6 bytes per element (reference: subgraph_traverser.cpp:652-656)"""
    rng = np.random.default_rng(6)
    x = rng.integers(-(1 << 47), 1 << 47, (3, 5, 8)).astype(np.int64)
    k = rng.integers(-(1 << 47), 1 << 47, (3, 5, 8)).astype(np.int64)
    k.ravel()[:3] = [-(1 << 47), (1 << 47) - 1, -1]
    mult = rng.integers(1, 1 << 15, 8).astype(np.int16)
    shift = rng.integers(40, 63, 8).astype(np.int8)
    kw = dict(out_dtype=np.int16, scale32=False, rounding_mode=oracle.ROUND_SINGLE)
    (want_x, st1), (want_k, st2) = oracle.rescale(x, mult, shift, **kw), oracle.rescale(k, mult, shift, **kw)
    assert st1 == st2 == oracle.VALID
    ts = [W.tensor("x", x.shape, np.int64), W.tensor("k", k.shape, np.int64, k), W.tensor("mult", [8], np.int16, mult),
          W.tensor("shift", [8], np.int8, shift), W.tensor("izp", [1], np.int64, [0]), W.tensor("ozp", [1], np.int16, [0]),
          W.tensor("yx", x.shape, np.int16), W.tensor("yk", k.shape, np.int16)]
    ops = [W.operator(R.OP_CONST, [], [n]) for n in ("k", "mult", "shift", "izp", "ozp")]
    attr = dict(scale32=False, rounding_mode=1)
    ops.append(W.operator(R.OP_RESCALE, ["x", "mult", "shift", "izp", "ozp"], ["yx"], W.rescale_attr(**attr)))
    ops.append(W.operator(R.OP_RESCALE, ["k", "mult", "shift", "izp", "ozp"], ["yk"], W.rescale_attr(**attr)))
    r = _run(_write_case(tmp_path, W.graph(ts, ops, ["x"], ["yx", "yk"]), {"x": x}, ["yx", "yk"]))
    assert r.returncode == 0, r.stderr
    assert np.array_equal(np.load(tmp_path / "yx_out.npy"), want_x)
    assert np.array_equal(np.load(tmp_path / "yk_out.npy"), want_k)
    # scale32 with an INT48 input is rejected when the graph is validated (type_conversion.cpp:122)
    ts[2] = W.tensor("mult", [8], np.int32, mult.astype(np.int32))
    ops[-2] = W.operator(R.OP_RESCALE, ["x", "mult", "shift", "izp", "ozp"], ["yx"], W.rescale_attr(scale32=True, rounding_mode=1))
    d2 = tmp_path / "bad"
    d2.mkdir()
    r = _run(_write_case(d2, W.graph(ts, ops[:-1], ["x"], ["yx"]), {"x": x}, ["yx"]))
    assert r.returncode == 2 and "INT48" in r.stderr


@pytest.mark.gpu
def test_int16_convolution_and_matmul_graphs(tmp_path):
    """the 16-bit instantiations (tensor_ops.cpp:2225, 2247, 2257): INT16 x INT8 -> INT48 CONV2D and DEPTHWISE_CONV2D whose
    result a RESCALE takes back to INT16, and INT16 x INT16 -> INT48 MATMUL; INT48 tensors are int64 .npy files, INT48
    constants 6 bytes per element"""
    rng = np.random.default_rng(21)
    x = rng.integers(-32768, 32768, (2, 9, 8, 12)).astype(np.int16)
    w = rng.integers(-128, 128, (6, 3, 3, 12)).astype(np.int8)
    wd = rng.integers(-128, 128, (3, 3, 12, 1)).astype(np.int8)
    bias = rng.integers(-(1 << 30), 1 << 30, 6).astype(np.int64)
    biasd = rng.integers(-(1 << 30), 1 << 30, 12).astype(np.int64)
    mult = rng.integers(1 << 13, 1 << 15, 6).astype(np.int16)
    shift = rng.integers(24, 30, 6).astype(np.int8)
    acc = oracle.conv2d("i16", x, w, bias, (1, 1, 1, 1), w_zp=2)
    accd = oracle.depthwise_conv2d("i16", x, wd, biasd, (1, 1, 1, 1))
    want, st = oracle.rescale(acc, mult, shift, out_dtype=np.int16, scale32=False, rounding_mode=oracle.ROUND_SINGLE)
    assert st == oracle.VALID and len(np.unique(want)) > 100
    ts = [W.tensor("x", x.shape, np.int16), W.tensor("w", w.shape, np.int8, w), W.tensor("wd", wd.shape, np.int8, wd),
          W.tensor("bias", [6], np.int64, bias), W.tensor("biasd", [12], np.int64, biasd),
          W.tensor("izp", [1], np.int16, [0]), W.tensor("wzp", [1], np.int8, [2]), W.tensor("wzp0", [1], np.int8, [0]),
          W.tensor("acc", [2, 9, 8, 6], np.int64), W.tensor("accd", [2, 9, 8, 12], np.int64),
          W.tensor("mult", [6], np.int16, mult), W.tensor("shift", [6], np.int8, shift),
          W.tensor("rizp", [1], np.int64, [0]), W.tensor("rozp", [1], np.int16, [0]), W.tensor("y", [2, 9, 8, 6], np.int16)]
    ops = [W.operator(R.OP_CONST, [], [n]) for n in ("w", "wd", "bias", "biasd", "izp", "wzp", "wzp0", "mult", "shift", "rizp", "rozp")]
    ops.append(W.operator(R.OP_CONV2D, ["x", "w", "bias", "izp", "wzp"], ["acc"], W.conv_attr((1, 1, 1, 1), (1, 1), (1, 1), acc_type=6)))
    ops.append(W.operator(R.OP_DEPTHWISE_CONV2D, ["x", "wd", "biasd", "izp", "wzp0"], ["accd"],
                          W.conv_attr((1, 1, 1, 1), (1, 1), (1, 1), acc_type=6)))
    ops.append(W.operator(R.OP_RESCALE, ["acc", "mult", "shift", "rizp", "rozp"], ["y"], W.rescale_attr(scale32=False, rounding_mode=1)))
    r = _run(_write_case(tmp_path, W.graph(ts, ops, ["x"], ["y", "accd"]), {"x": x}, ["y", "accd"]))
    assert r.returncode == 0, r.stderr
    assert np.array_equal(np.load(tmp_path / "y_out.npy"), want)
    got_d = np.load(tmp_path / "accd_out.npy")
    assert got_d.dtype == np.int64 and np.array_equal(got_d, accd)

    # TRANSPOSE_CONV2D and CONV3D on INT16 (tensor_ops.cpp:2237, 2291)
    wt = rng.integers(-128, 128, (4, 3, 2, 12)).astype(np.int8)
    bt = rng.integers(-(1 << 40), 1 << 40, 4).astype(np.int64)
    acct = oracle.transpose_conv2d("i16", x, wt, bt, (0, 1, -1, 0), (2, 2), w_zp=2)
    x3 = rng.integers(-32768, 32768, (1, 4, 5, 5, 8)).astype(np.int16)
    w3 = rng.integers(-128, 128, (4, 2, 3, 3, 8)).astype(np.int8)
    pad3, one3 = (1, 0, 1, 1, 1, 1), (1, 1, 1)
    acc3 = oracle.conv3d("i16", x3, w3, bt, pad3, one3, one3, w_zp=2)
    ts = [W.tensor("x", x.shape, np.int16), W.tensor("x3", x3.shape, np.int16), W.tensor("wt", wt.shape, np.int8, wt),
          W.tensor("w3", w3.shape, np.int8, w3), W.tensor("bt", [4], np.int64, bt), W.tensor("izp", [1], np.int16, [0]),
          W.tensor("wzp", [1], np.int8, [2]), W.tensor("ot", acct.shape, np.int64), W.tensor("o3", acc3.shape, np.int64)]
    ops = [W.operator(R.OP_CONST, [], [n]) for n in ("wt", "w3", "bt", "izp", "wzp")]
    ops.append(W.operator(10, ["x", "wt", "bt", "izp", "wzp"], ["ot"], W.transpose_conv_attr((0, 1, -1, 0), (2, 2), acc_type=6)))
    ops.append(W.operator(4, ["x3", "w3", "bt", "izp", "wzp"], ["o3"], W.conv_attr(pad3, one3, one3, acc_type=6)))
    d3 = tmp_path / "t3"
    d3.mkdir()
    r = _run(_write_case(d3, W.graph(ts, ops, ["x", "x3"], ["ot", "o3"]), {"x": x, "x3": x3}, ["ot", "o3"]))
    assert r.returncode == 0, r.stderr
    assert np.array_equal(np.load(d3 / "ot_out.npy"), acct) and np.array_equal(np.load(d3 / "o3_out.npy"), acc3)

    a = rng.integers(-32768, 32768, (2, 20, 33)).astype(np.int16)
    b = rng.integers(-32768, 32768, (2, 33, 7)).astype(np.int16)
    ts = [W.tensor("a", a.shape, np.int16), W.tensor("b", b.shape, np.int16), W.tensor("azp", [1], np.int16, [0]),
          W.tensor("bzp", [1], np.int16, [0]), W.tensor("o", [2, 20, 7], np.int64)]
    ops = [W.operator(R.OP_CONST, [], ["azp"]), W.operator(R.OP_CONST, [], ["bzp"]),
           W.operator(R.OP_MATMUL, ["a", "b", "azp", "bzp"], ["o"])]
    d2 = tmp_path / "mm"
    d2.mkdir()
    r = _run(_write_case(d2, W.graph(ts, ops, ["a", "b"], ["o"]), {"a": a, "b": b}, ["o"]))
    assert r.returncode == 0, r.stderr
    assert np.array_equal(np.load(d2 / "o_out.npy"), oracle.matmul("i16", a, b))


@pytest.mark.gpu
def test_int4_weight_graphs(tmp_path):
    """INT8 x INT4 -> INT32 (tensor_ops.cpp:2224, 2246): the weights are constants of two values to a byte
    (subgraph_traverser.cpp:625-630) and the arithmetic is that of int8 weights; an odd element count leaves half a byte
    unused; a weight zero point other than 0 is an error (tensor_ops.cpp:811)"""
    rng = np.random.default_rng(44)
    x = rng.integers(-128, 128, (2, 7, 9, 5)).astype(np.int8)
    w = rng.integers(-8, 8, (3, 3, 3, 5)).astype(np.int8)         # 135 values: 67 and a half bytes
    wd = rng.integers(-8, 8, (3, 3, 5, 2)).astype(np.int8)
    bias = rng.integers(-1000, 1000, 3).astype(np.int32)
    biasd = rng.integers(-1000, 1000, 10).astype(np.int32)
    assert w.min() == -8 and w.max() == 7
    acc = oracle.conv2d("i8", x, w, bias, (1, 1, 1, 1), in_zp=-5)
    accd = oracle.depthwise_conv2d("i8", x, wd, biasd, (1, 1, 1, 1), in_zp=-5)
    ts = [W.tensor("x", x.shape, np.int8), W.tensor("w", w.shape, np.int8, w, int4=True),
          W.tensor("wd", wd.shape, np.int8, wd, int4=True), W.tensor("bias", [3], np.int32, bias),
          W.tensor("biasd", [10], np.int32, biasd), W.tensor("izp", [1], np.int8, [-5]),
          W.tensor("wzp", [1], np.int8, [0], int4=True), W.tensor("wzp3", [1], np.int8, [3], int4=True),
          W.tensor("acc", [2, 7, 9, 3], np.int32), W.tensor("accd", [2, 7, 9, 10], np.int32)]
    consts = [W.operator(R.OP_CONST, [], [n]) for n in ("w", "wd", "bias", "biasd", "izp", "wzp", "wzp3")]
    ops = consts + [W.operator(R.OP_CONV2D, ["x", "w", "bias", "izp", "wzp"], ["acc"], W.conv_attr((1, 1, 1, 1), (1, 1), (1, 1))),
                    W.operator(R.OP_DEPTHWISE_CONV2D, ["x", "wd", "biasd", "izp", "wzp"], ["accd"],
                               W.conv_attr((1, 1, 1, 1), (1, 1), (1, 1)))]
    r = _run(_write_case(tmp_path, W.graph(ts, ops, ["x"], ["acc", "accd"]), {"x": x}, ["acc", "accd"]))
    assert r.returncode == 0, r.stderr
    assert np.array_equal(np.load(tmp_path / "acc_out.npy"), acc)
    assert np.array_equal(np.load(tmp_path / "accd_out.npy"), accd)
    ops = consts + [W.operator(R.OP_CONV2D, ["x", "w", "bias", "izp", "wzp3"], ["acc"], W.conv_attr((1, 1, 1, 1), (1, 1), (1, 1)))]
    d2 = tmp_path / "zp"
    d2.mkdir()
    r = _run(_write_case(d2, W.graph(ts, ops, ["x"], ["acc"]), {"x": x}, ["acc"]))
    assert r.returncode == 2 and "Weight zero point must be zero for non int8_t data" in r.stderr
    # TRANSPOSE_CONV2D and CONV3D with INT4 weights (tensor_ops.cpp:2235, 2258)
    wt = rng.integers(-8, 8, (4, 3, 3, 5)).astype(np.int8)
    bt = rng.integers(-500, 500, 4).astype(np.int32)
    acct = oracle.transpose_conv2d("i8", x, wt, bt, (0, 1, -1, 0), (2, 2), in_zp=-5, w_zp=0)
    x3 = rng.integers(-128, 128, (1, 4, 5, 5, 8)).astype(np.int8)
    w3 = rng.integers(-8, 8, (4, 2, 3, 3, 8)).astype(np.int8)
    pad3, one3 = (1, 0, 1, 1, 1, 1), (1, 1, 1)
    acc3 = oracle.conv3d("i8", x3, w3, bt, pad3, one3, one3, in_zp=-5, w_zp=0)
    ts3 = [W.tensor("x", x.shape, np.int8), W.tensor("x3", x3.shape, np.int8), W.tensor("wt", wt.shape, np.int8, wt, int4=True),
           W.tensor("w3", w3.shape, np.int8, w3, int4=True), W.tensor("bt", [4], np.int32, bt), W.tensor("izp", [1], np.int8, [-5]),
           W.tensor("wzp", [1], np.int8, [0], int4=True), W.tensor("ot", acct.shape, np.int32), W.tensor("o3", acc3.shape, np.int32)]
    ops = [W.operator(R.OP_CONST, [], [n]) for n in ("wt", "w3", "bt", "izp", "wzp")]
    ops.append(W.operator(10, ["x", "wt", "bt", "izp", "wzp"], ["ot"], W.transpose_conv_attr((0, 1, -1, 0), (2, 2))))
    ops.append(W.operator(4, ["x3", "w3", "bt", "izp", "wzp"], ["o3"], W.conv_attr(pad3, one3, one3)))
    d4 = tmp_path / "t3"
    d4.mkdir()
    r = _run(_write_case(d4, W.graph(ts3, ops, ["x", "x3"], ["ot", "o3"]), {"x": x, "x3": x3}, ["ot", "o3"]))
    assert r.returncode == 0, r.stderr
    assert np.array_equal(np.load(d4 / "ot_out.npy"), acct) and np.array_equal(np.load(d4 / "o3_out.npy"), acc3)
    # INT4 is a weight type only: as a convolution's input it is refused
    ts2 = [W.tensor("x", x.shape, np.int8, int4=True)] + ts[1:]
    ops = consts + [W.operator(R.OP_CONV2D, ["x", "w", "bias", "izp", "wzp"], ["acc"], W.conv_attr((1, 1, 1, 1), (1, 1), (1, 1)))]
    d3 = tmp_path / "in4"
    d3.mkdir()
    r = _run(_write_case(d3, W.graph(ts2, ops, ["x"], ["acc"]), {"x": x}, ["acc"]))
    assert r.returncode == 2


@pytest.mark.gpu
def test_inexact_round_rescale_in_precise_and_compliance_mode(tmp_path):
    """--precise_mode=1 reaches an INEXACT_ROUND RESCALE (type_conversion.cpp:326-346): FP64 maths truncated; on a
    compliance descriptor the normal pass writes the lower edge of the error bound and the bounds pass the upper one"""
    rng = np.random.default_rng(11)
    x = rng.integers(-128, 128, (4, 9, 16)).astype(np.int8)
    mult = rng.integers(1 << 24, 1 << 30, 16).astype(np.int32)
    shift = rng.integers(26, 31, 16).astype(np.int8)
    mult[0], shift[0] = 1 << 30, 31    # halves: on ties the two edges of the compliance bound differ
    kw = dict(in_zp=2, out_zp=-9, out_dtype=np.int8, rounding_mode=oracle.ROUND_INEXACT)
    ts = [W.tensor("x", x.shape, np.int8), W.tensor("mult", [16], np.int32, mult), W.tensor("shift", [16], np.int8, shift),
          W.tensor("izp", [1], np.int8, [2]), W.tensor("ozp", [1], np.int8, [-9]), W.tensor("y", x.shape, np.int8)]
    ops = [W.operator(R.OP_CONST, [], [n]) for n in ("mult", "shift", "izp", "ozp")]
    ops.append(W.operator(R.OP_RESCALE, ["x", "mult", "shift", "izp", "ozp"], ["y"], W.rescale_attr(rounding_mode=2)))
    desc = _write_case(tmp_path, W.graph(ts, ops, ["x"], ["y"]), {"x": x}, ["y"])
    want = {m: oracle.rescale(x, mult, shift, inexact_mode=m, **kw)[0] for m in (0, 1, 2, 3)}
    assert not np.array_equal(want[0], want[1]) and not np.array_equal(want[2], want[3])
    r = _run(desc)
    assert r.returncode == 0 and np.array_equal(np.load(tmp_path / "y_out.npy"), want[0])
    r = _run(desc, "--precise_mode=1")
    assert r.returncode == 0 and np.array_equal(np.load(tmp_path / "y_out.npy"), want[1])
    meta = dict(json.loads(open(desc).read()), test_requirements={"bounds_file_required": True})
    open(desc, "w").write(json.dumps(meta))
    r = _run(desc, "--precise_mode=1")
    assert r.returncode == 0, r.stderr
    assert np.array_equal(np.load(tmp_path / "y_out.npy"), want[2])
    assert np.array_equal(np.load(tmp_path / "bounds_y_out.npy"), want[3])


@pytest.mark.gpu
def test_precise_mode_writes_fp64_results_and_bounds(tmp_path):
    """--precise_mode=1 on a compliance-style descriptor (test_requirements.bounds_file_required): the fp16 CONV2D is
    evaluated in fp64, then once more over absolute values into bounds_<ofm_file> (reference: main.cpp:109-121,
    :246-251, :404-407); both files equal the fp64 oracle bit for bit.  MATMUL likewise."""
    rng = np.random.default_rng(12)
    x = rng.normal(0, 1, (2, 9, 8, 24)).astype(np.float16)
    w = rng.normal(0, 0.2, (10, 3, 3, 24)).astype(np.float16)
    b = rng.normal(0, 1, 10).astype(np.float16)
    pad, stride, dil = (1, 1, 1, 1), (1, 1), (1, 1)
    xf, wf, bf = (v.astype(np.float64) for v in (x, w, b))
    ref = oracle.conv2d("f64", xf, wf, bf, pad, stride, dil)
    # the attribute's local_bound is absent = false here: the bounds pass replaces the input by its largest magnitude
    # (tensor_ops.cpp:797-801)
    bnd = oracle.conv2d("f64", xf, wf, bf, pad, stride, dil, abs_mode=True, local_bound=False)
    ts = [W.tensor("x", x.shape, np.float16), W.tensor("w", w.shape, np.float16, w), W.tensor("b", [10], np.float16, b),
          W.tensor("z", [1], np.float16, [0]), W.tensor("y", ref.shape, np.float16)]
    ops = [W.operator(R.OP_CONST, [], [n]) for n in ("w", "b", "z")]
    ops.append(W.operator(R.OP_CONV2D, ["x", "w", "b", "z", "z"], ["y"], W.conv_attr(pad, stride, dil, acc_type=7)))
    d1 = tmp_path / "conv"
    d1.mkdir()
    desc = _write_case(d1, W.graph(ts, ops, ["x"], ["y"]), {"x": x}, ["y"])
    meta = json.loads(open(desc).read())
    meta["test_requirements"] = {"bounds_file_required": True}
    open(desc, "w").write(json.dumps(meta))
    r = _run(desc, "--precise_mode=1")
    assert r.returncode == 0, r.stderr
    got, got_bnd = np.load(d1 / "y_out.npy"), np.load(d1 / "bounds_y_out.npy")
    assert got.dtype == got_bnd.dtype == np.float64
    assert np.array_equal(got, ref) and np.array_equal(got_bnd, bnd)
    # local_bound = true: the sums over the absolute values themselves
    ops_lb = ops[:-1] + [W.operator(R.OP_CONV2D, ["x", "w", "b", "z", "z"], ["y"],
                                    W.conv_attr(pad, stride, dil, acc_type=7, local_bound=True))]
    d5 = tmp_path / "conv_local"
    d5.mkdir()
    desc5 = _write_case(d5, W.graph(ts, ops_lb, ["x"], ["y"]), {"x": x}, ["y"])
    meta5 = dict(json.loads(open(desc5).read()), test_requirements={"bounds_file_required": True})
    open(desc5, "w").write(json.dumps(meta5))
    r = _run(desc5, "--precise_mode=1")
    assert r.returncode == 0, r.stderr
    local = oracle.conv2d("f64", xf, wf, bf, pad, stride, dil, abs_mode=True)
    assert np.array_equal(np.load(d5 / "bounds_y_out.npy"), local) and np.array_equal(np.load(d5 / "y_out.npy"), ref)
    assert np.all(bnd >= local) and not np.array_equal(bnd, local)
    # without the option the result has the graph's element type and no bounds file appears
    d2 = tmp_path / "plain"
    d2.mkdir()
    r = _run(_write_case(d2, W.graph(ts, ops, ["x"], ["y"]), {"x": x}, ["y"]))
    assert r.returncode == 0 and np.load(d2 / "y_out.npy").dtype == np.float16 and not (d2 / "bounds_y_out.npy").exists()
    # precise mode without the requirement: one run
    d3 = tmp_path / "nobounds"
    d3.mkdir()
    r = _run(_write_case(d3, W.graph(ts, ops, ["x"], ["y"]), {"x": x}, ["y"]), "--precise_mode=1")
    assert r.returncode == 0 and np.array_equal(np.load(d3 / "y_out.npy"), ref) and not (d3 / "bounds_y_out.npy").exists()

    a = rng.normal(0, 1, (2, 5, 40)).astype(np.float16)
    bb = rng.normal(0, 1, (2, 40, 7)).astype(np.float16)
    ts = [W.tensor("a", a.shape, np.float16), W.tensor("b", bb.shape, np.float16), W.tensor("z", [1], np.float16, [0]),
          W.tensor("o", [2, 5, 7], np.float32)]
    ops = [W.operator(R.OP_CONST, [], ["z"]), W.operator(R.OP_MATMUL, ["a", "b", "z", "z"], ["o"])]
    d4 = tmp_path / "matmul"
    d4.mkdir()
    desc = _write_case(d4, W.graph(ts, ops, ["a", "b"], ["o"]), {"a": a, "b": bb}, ["o"])
    meta = json.loads(open(desc).read())
    meta["test_requirements"] = {"bounds_file_required": True}
    open(desc, "w").write(json.dumps(meta))
    r = _run(desc, "--precise_mode=1")
    assert r.returncode == 0, r.stderr
    assert np.array_equal(np.load(d4 / "o_out.npy"), oracle.matmul("f64", a.astype(np.float64), bb.astype(np.float64)))
    assert np.array_equal(np.load(d4 / "bounds_o_out.npy"),
                          oracle.matmul("f64", a.astype(np.float64), bb.astype(np.float64), abs_mode=True))


@pytest.mark.gpu
def test_precise_mode_is_refused_where_no_fp64_pass_exists(tmp_path):
    """floating-point TRANSPOSE_CONV2D / AVG_POOL2D / CLAMP have no fp64 evaluation here: with --precise_mode=1 the
    graph ends with status 2 instead of writing the ordinary result under the precise run's name"""
    rng = np.random.default_rng(13)
    x = rng.normal(0, 1, (1, 6, 6, 8)).astype(np.float16)
    ts = [W.tensor("x", x.shape, np.float16), W.tensor("z", [1], np.float16, [0]), W.tensor("y", [1, 3, 3, 8], np.float16)]
    ops = [W.operator(R.OP_CONST, [], ["z"]),
           W.operator(R.OP_AVG_POOL2D, ["x", "z", "z"], ["y"], W.pool_attr((2, 2), (2, 2), (0, 0, 0, 0), 7))]
    desc = _write_case(tmp_path, W.graph(ts, ops, ["x"], ["y"]), {"x": x}, ["y"])
    assert _run(desc).returncode == 0
    r = _run(desc, "--precise_mode=1")
    assert r.returncode == 2 and "precise-mode" in r.stderr


@pytest.mark.gpu
def test_fp16_conv2d_then_clamp_runs_on_the_device(tmp_path):
    """an fp16 CONV2D followed by a floating-point CLAMP (activation_funcs.cpp:97-106) ends with status 0"""
    rng = np.random.default_rng(14)
    x = rng.normal(0, 1, (1, 7, 7, 16)).astype(np.float16)
    w = rng.normal(0, 0.3, (8, 3, 3, 16)).astype(np.float16)
    b = rng.normal(0, 1, 8).astype(np.float16)
    ts = [W.tensor("x", x.shape, np.float16), W.tensor("w", w.shape, np.float16, w), W.tensor("b", [8], np.float16, b),
          W.tensor("z", [1], np.float16, [0]), W.tensor("c", [1, 7, 7, 8], np.float16), W.tensor("y", [1, 7, 7, 8], np.float16)]
    ops = [W.operator(R.OP_CONST, [], [n]) for n in ("w", "b", "z")]
    ops.append(W.operator(R.OP_CONV2D, ["x", "w", "b", "z", "z"], ["c"], W.conv_attr((1, 1, 1, 1), (1, 1), (1, 1), acc_type=7)))
    ops.append(W.operator(R.OP_CLAMP, ["c"], ["y"], W.clamp_attr(-0.5, 1.25, np.float16)))
    r = _run(_write_case(tmp_path, W.graph(ts, ops, ["x"], ["y"]), {"x": x}, ["y"]))
    assert r.returncode == 0, r.stderr
    got = np.load(tmp_path / "y_out.npy")
    assert got.dtype == np.float16 and got.min() == np.float16(-0.5) and got.max() == np.float16(1.25)
    conv = oracle.conv2d("f32", x, w, b, (1, 1, 1, 1)).astype(np.float64)
    inside = (conv > -0.45) & (conv < 1.2)
    assert np.allclose(got[inside].astype(np.float64), conv[inside], atol=4e-3)


@pytest.mark.gpu
def test_tosa_level_makes_a_violating_graph_unpredictable(tmp_path):
    """--tosa_level=EIGHTK: a pad beyond MAX_KERNEL = 8192 fails a LEVEL_CHECK (tensor_ops.cpp:766-769): the graph
    is evaluated and ends UNPREDICTABLE (func_debug.h:132-141); without a level the same graph is VALID"""
    x = np.ones((1, 2, 2, 8), np.int8)
    w = np.ones((8, 1, 1, 8), np.int8)
    pad = (8193, 0, 0, 0)
    oh = 2 + 8193
    ts = [W.tensor("x", x.shape, np.int8), W.tensor("w", w.shape, np.int8, w), W.tensor("b", [8], np.int32, np.zeros(8, np.int32)),
          W.tensor("z", [1], np.int8, [0]), W.tensor("y", [1, oh, 2, 8], np.int32)]
    ops = [W.operator(R.OP_CONST, [], [n]) for n in ("w", "b", "z")]
    ops.append(W.operator(R.OP_CONV2D, ["x", "w", "b", "z", "z"], ["y"], W.conv_attr(pad, (1, 1), (1, 1))))
    desc = _write_case(tmp_path, W.graph(ts, ops, ["x"], ["y"]), {"x": x}, ["y"])
    assert _run(desc).returncode == 0
    want = np.load(tmp_path / "y_out.npy").copy()
    assert want[0, :8193].max() == 0 and want[0, 8193:].min() == 8
    r = _run(desc, "--tosa_level=EIGHTK")
    assert r.returncode == 1 and "MAX_KERNEL" in r.stderr
    assert np.array_equal(np.load(tmp_path / "y_out.npy"), want)       # evaluated all the same
    assert _run(desc, "--tosa_level=NONE").returncode == 0


# ---- system-under-test module for the reference's conformance runner ----------------------------------------
class _RunnerArgs:
    verbose = False
    precise_mode = False


def _copy_example(golden_dir, tmp_path, name):
    import shutil
    dst = tmp_path / name
    shutil.copytree(os.path.join(golden_dir, name), dst)
    return dst


def test_sut_module_command_line_and_status_without_a_gpu(golden_dir, tmp_path):
    from reference_model_amd import sut_run
    d = _copy_example(golden_dir, tmp_path, "qi8_conv2d_1x1")
    assert sut_run.parse_runner_args(["precise_mode", "runner=/x/y", "timeout=5"]) == {
        "precise_mode": True, "runner": "/x/y", "timeout": "5"}
    sut = sut_run.TosaSUTRunner(_RunnerArgs(), ["no_fusion"], d)
    assert sut.command() == [RUN, f"--test_desc={d / 'desc.json'}", "--no_fusion"]
    sut = sut_run.TosaSUTRunner(_RunnerArgs(), ["precise_mode"], d)
    assert sut.command()[-1] == "--precise_mode=1"
    missing = sut_run.TosaSUTRunner(_RunnerArgs(), ["runner=/nonexistent/tosa_mi355_run"], d)
    result, message = missing.runTestGraph()
    assert result == sut_run.TosaTestRunner.TosaGraphResult.OTHER_ERROR and "nonexistent" in message
    import torch
    if not torch.cuda.is_available():
        result, message = sut_run.TosaSUTRunner(_RunnerArgs(), [], d).runTestGraph()
        assert result == sut_run.TosaTestRunner.TosaGraphResult.TOSA_ERROR and "no CPU fall-back" in message
        assert not (d / "ref_model_output_0.npy").exists()


@pytest.mark.gpu
def test_sut_module_runs_the_reference_example_directory(golden_dir, tmp_path):
    from reference_model_amd import sut_run
    d = _copy_example(golden_dir, tmp_path, "qi8_conv2d_1x1")
    result, message = sut_run.TosaSUTRunner(_RunnerArgs(), [], d).runTestGraph()
    assert result == sut_run.TosaTestRunner.TosaGraphResult.TOSA_VALID and message is None
    assert np.array_equal(np.load(d / "ref_model_output_0.npy"), np.load(d / "tflite_result.npy"))
