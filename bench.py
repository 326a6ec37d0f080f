#!/usr/bin/env python3
"""Benchmark of the hot path on one MI355X.

A step is one pass of the fused INT8 CONV2D -> RESCALE -> CLAMP operator (one C-ABI call) over one batch of
the ResNet-style 3x3 configuration: input NHWC [8,56,56,64] int8 (input_zp -7), weight OHWI [64,3,3,64],
bias int32, stride 1, pad 1, per-channel double-round RESCALE (shift 38) to int8, CLAMP [0,127].
Operands are seeded synthetic tensors, resident in HBM before the timed region starts.

Prints one JSON line: metric / value in int8 TOPS (2 x dense MACs, padded taps counted), the roofline
object for the convolution kernel (MFMA bound, dense int8 peak 5.0 POP/s) and the CPU baseline (the scalar
C oracle, 1 core).
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
for p in (ROOT, os.path.join(ROOT, "tests")):
    if p not in sys.path:
        sys.path.insert(0, p)

INT8_MFMA_PEAK_TOPS = 5000.0  # MI355X dense int8, published
# HBM bytes per launch of the convolution kernel from rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE runs
# (profiles/conv2d_mfma_i8_rescale_c3_pmc.txt); None until measured.
MEASURED_TRAFFIC_BYTES = None


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=2000)
    ap.add_argument("--warmup", type=int, default=200)
    ap.add_argument("--no-cpu-baseline", action="store_true", help="skip the CPU oracle timing")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build runs on exactly one GPU (no collectives, no sharding); use --gpus 1",
              file=sys.stderr)
        return 2

    import numpy as np
    import torch

    import cases
    from reference_model_amd import Context, capi

    if not torch.cuda.is_available():
        print("bench.py: no GPU visible", file=sys.stderr)
        return 2
    dev = torch.device("cuda:0")
    c = cases.c3()
    n, ih, iw, ic = c["x"].shape
    oc, kh, kw, _ = c["w"].shape
    oh, ow = ih, iw
    macs = n * oh * ow * oc * kh * kw * ic
    ops = 2 * macs
    algo_bytes = c["x"].nbytes + c["w"].nbytes + c["bias"].nbytes + c["mult"].nbytes + c["shift"].nbytes + n * oh * ow * oc

    t = {k: torch.from_numpy(np.ascontiguousarray(c[k])).to(dev) for k in ("x", "w", "bias", "mult", "shift")}
    out = torch.empty((n, oh, ow, oc), dtype=torch.int8, device=dev)

    ctx = Context(0)
    stream = torch.cuda.current_stream()
    ctx.set_stream(stream.cuda_stream)
    d = ctx.conv_desc(capi.INT8, capi.INT32, (n, ih, iw, ic), oc, kh, kw, (oh, ow), c["pad"], c["stride"],
                      c["dilation"], c["bias"].shape[0])
    r = ctx.rescale_desc(capi.INT32, capi.INT8, oc, oc, 0, c["out_zp"], True, capi.ROUND_DOUBLE, True)

    def step():
        ctx.conv2d_rescale_clamp(d, t["x"], t["w"], t["bias"], c["in_zp"], c["w_zp"], r, t["mult"], t["shift"], out,
                                 c["clamp"])

    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    ev0, ev1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    t0 = time.perf_counter()
    ev0.record(stream)
    for _ in range(args.steps):
        step()
    ev1.record(stream)
    torch.cuda.synchronize()
    t1 = time.perf_counter()
    status = ctx.sync()
    kernel = ctx.last_kernel
    ms_per_step = (t1 - t0) * 1e3 / args.steps
    ev_ms_per_launch = ev0.elapsed_time(ev1) / args.steps
    tops = ops / (ms_per_step * 1e-3) / 1e12
    achieved = ops / (ev_ms_per_launch * 1e-3) / 1e12

    # parity of what was just timed, against the CPU oracle (bit exact)
    result = {"metric": "int8 CONV2D+RESCALE TOPS at 3x3 ResNet shape; % int8 MFMA peak; bit-exact",
              "value": round(tops, 3), "unit": "TOPS", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
              "ms_per_step": round(ms_per_step, 6), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
              "dtype": "int8", "data": "synthetic",
              "config": {"workload": "configs[2]: INT8 CONV2D ResNet-style 3x3 [8,56,56,64]x[64,3,3,64] s1 p1 "
                                     "+ per-channel RESCALE (shift 38, double_round) + CLAMP [0,127], fused",
                         "kernel": kernel, "ops_per_step": ops, "algorithmic_bytes_per_step": algo_bytes,
                         "graph_status": status},
              "roofline": {"bound": "mfma", "achieved": round(achieved, 3), "peak": INT8_MFMA_PEAK_TOPS,
                           "unit": "TOP/s", "frac": round(achieved / INT8_MFMA_PEAK_TOPS, 5),
                           "traffic": MEASURED_TRAFFIC_BYTES, "us_per_launch": round(ev_ms_per_launch * 1e3, 3)}}

    if not args.no_cpu_baseline:
        import oracle
        best = None
        for _ in range(3):
            c0 = time.perf_counter()
            acc = oracle.conv2d("i8", c["x"], c["w"], c["bias"], c["pad"], c["stride"], c["dilation"], c["in_zp"],
                                c["w_zp"])
            ref, _ = oracle.rescale(acc, c["mult"], c["shift"], out_zp=c["out_zp"])
            ref = oracle.clamp(ref, *c["clamp"])
            dt = time.perf_counter() - c0
            best = dt if best is None else min(best, dt)
        bit_exact = bool(np.array_equal(out.cpu().numpy(), ref))
        result["config"]["bit_exact_vs_oracle"] = bit_exact
        result["cpu_baseline"] = {"value": round(ops / best / 1e12, 6), "unit": "TOPS", "cores": 1, "kind": "port",
                                  "sample": "the full config (1 batch of [8,56,56,64]), min of 3 runs of the scalar "
                                            "C oracle (conv2d + rescale + clamp), %.2f s per run" % best}
        if not bit_exact:
            print("bench.py: GPU result differs from the oracle", file=sys.stderr)
            print(json.dumps(result))
            return 1
    print(json.dumps(result))
    ctx.close()
    return 0


if __name__ == "__main__":
    sys.exit(main())
