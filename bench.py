#!/usr/bin/env python3
"""Benchmark of the hot path on one MI355X.

A step is one pass of one operator (one C-ABI call) over one batch of seeded synthetic operands that are
resident in HBM before the timed region starts.  The default workload is the headline configuration:

  c3   INT8 CONV2D 3x3 [8,56,56,64]x[64,3,3,64] s1 p1 + per-channel RESCALE (shift 38, double_round) +
       CLAMP [0,127], fused (default; unit TOPS, MFMA roofline)

and --config selects the other benchmark configurations, each reported against the roofline that bounds it:

  c2   INT8 MATMUL [8,1024,1024]x[8,1024,1024] -> int32            (TOPS; HBM roofline, int32 result)
  c4   INT8 DEPTHWISE_CONV2D [8,112,112,96] s2 + RESCALE, fused     (GB/s; HBM roofline)
  c5a  FP16 CONV2D 3x3 [16,28,28,256]x[256,3,3,256], fp32 accumulate (TFLOPS; MFMA roofline)
  c5b  BF16 MATMUL [4,2048,4096]x[4,4096,2048] -> fp32              (TFLOPS; MFMA roofline)

and three configurations that measure the box rather than an operator: launch_floor (a kernel that does nothing,
with the grid, block and LDS size of the headline kernel) and copy (copy / read-only / write-only streams).

The timed steps are replayed from HIP graphs of up to 100 steps each (--eager: one host launch per step).  The
region of --steps steps is enqueued --repeats times back to back, each repeat between two HIP events on the launch
stream; ms_per_step, value and roofline.achieved come from the median repeat, and the host clock around the whole
region (synchronised on both sides) is reported beside it.  One JSON line is printed.  cpu_baseline = the C oracle
on a bounded sample of the same workload: on one core (value) and, where its loops are parallel, on all host cores.
"""
from __future__ import annotations

import argparse
import json
import math
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
for p in (ROOT, os.path.join(ROOT, "tests")):
    if p not in sys.path:
        sys.path.insert(0, p)

PEAK = {"int8_mfma": 5000.0, "f16_mfma": 2500.0, "hbm": 8000.0}  # TOP/s, TFLOP/s, GB/s (MI355X, published)
# rocprofv3 summary under profiles/ that holds the HBM traffic of each configuration's dominant kernel
PROFILE_OF = {"c3": "conv2d_slab_wreg_i8_rescale_c3_resnet3x3", "c2": "matmul_gemm_i8_c2_8x1024",
              "c4": "depthwise_mfma_i8_rescale_c4_mobilenet", "c5a": "gemm_mfma_f16_c5a_3x3_256",
              "c5b": "matmul_gemm_bf16_c5b_4x2048x4096", "maxpool": "max_pool2d_i8_32x112x112x64",
              "avgpool": "avg_pool2d_i8_32x112x112x64", "tconv": "transpose_conv2d_slab_i8_8x28x28x128",
              "conv3d": "conv3d_slab_i8_2x16x28x28x32", "rescale": "rescale_fast_i32_to_i8_64x56x56x64",
              "c4x8": "depthwise_mfma_i8_rescale_64x112x112x96", "dw32": "depthwise_stream_i8_rescale_64x112x112x32", "c3x4": "conv2d_slab_wreg_i8_rescale_32x56x56x64"}


def measured_traffic(cfg, kernel):
    """HBM bytes per launch from the committed rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE summary of this configuration
    (each counter scaled by what it reads for a plain copy of known size; the summary holds the raw figures and the
    commands).  The summary names the library kernel it was taken on: when the kernel that has just run is another
    one, the figure is not this kernel's and None is returned with the reason."""
    name = PROFILE_OF.get(cfg)
    path = os.path.join(ROOT, "profiles", (name or "") + ".txt")
    if not name or not os.path.exists(path):
        return None, {"traffic_source": None}
    total, profiled = None, None
    with open(path) as f:
        for line in f:
            if line.startswith("library kernel:"):
                profiled = line.split(":", 1)[1].strip()
            elif line.startswith("total HBM bytes per step:"):
                first = line.split(":", 1)[1].split()[0]
                total = int(first) if first.isdigit() else None
    src = {"traffic_source": "profiles/%s.txt" % name, "traffic_kernel": profiled}
    if total is None or profiled != kernel:
        src["traffic_note"] = "the summary was taken on another kernel than the one that ran (%s)" % kernel
        return None, src
    return total, src


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=None)
    ap.add_argument("--warmup", type=int, default=None)
    ap.add_argument("--repeats", type=int, default=None,
                    help="times the region of --steps steps is run; the median repeat is reported "
                         "(default: enough repeats for 10000 steps, between 5 and 500)")
    ap.add_argument("--copy-mib", type=int, default=1024, help="buffer size of --config copy")
    ap.add_argument("--config", default="c3", choices=["c1", "c2", "c3", "c3x4", "c4", "c5a", "c5b", "rescale", "c4x8", "dw32", "tconv", "conv3d", "maxpool", "avgpool", "precise", "copy", "launch_floor", "networks"])
    ap.add_argument("--batch", type=int, default=8, help="images per layer of --config networks")
    ap.add_argument("--no-cpu-baseline", action="store_true", help="skip the CPU oracle timing and the parity check")
    ap.add_argument("--no-named-configs", action="store_true",
                    help="default configuration only: skip the short GPU legs of the other named configurations")
    ap.add_argument("--kernel-choice", type=int, default=0,
                    help="tmi_ctx_set_kernel_choice for the measured operator (0: the library's own choice; the profiles of "
                         "one layer under two kernels use it)")
    ap.add_argument("--eager", action="store_true",
                    help="issue every step from the host instead of replaying HIP graphs of the steps")
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
    ctx = Context(0)
    stream = torch.cuda.current_stream()
    ctx.set_stream(stream.cuda_stream)
    if args.kernel_choice:
        ctx.set_kernel_choice(args.kernel_choice)

    def the_oracle():
        # the CPU oracle is the checker and the CPU baseline: nothing before the timed region touches it
        import oracle
        return oracle

    def conv_out_hw(ih, iw, kh, kw, pad, stride, dilation):
        return ((ih - 1 + pad[0] + pad[1] - (kh - 1) * dilation[0]) // stride[0] + 1,
                (iw - 1 + pad[2] + pad[3] - (kw - 1) * dilation[1]) // stride[1] + 1)

    def accuracy_figures(imp, ref, bnd, out_type, out_dtype, ks, has_bias, device_only=False):
        """the result against the library's own fp64 pass over the same operands: the DOT_PRODUCT check (device
        reduction), and the largest ULP and relative errors (numpy over the downloaded tensors)"""
        import dot_product_check as dp
        ksb = dp.kernel_size_bound(ks, out_type, has_bias=has_bias)
        r = ctx.dot_product_check(out_dtype, imp.numel(), imp, ref, bnd, ksb, -1)
        ctx.sync()
        if device_only:
            return {"dot_product_compliant": bool(r.compliant), "max_err_in_bound_units": round(float(r.max_abs_err), 4),
                    "allowed_err_in_bound_units": int(r.abs_bound)}
        st = dp.check(imp.cpu().numpy(), ref.cpu().numpy(), bnd.cpu().numpy(), out_type, ksb)
        return {"dot_product_compliant": bool(r.compliant), "max_err_in_bound_units": round(float(r.max_abs_err), 4),
                "allowed_err_in_bound_units": int(r.abs_bound), "max_ulp": round(st["max_ulp"], 3),
                "max_rel_err": float("%.4g" % st["max_rel"]),
                "max_ulp_where_ref_is_at_least_an_eighth_of_the_bound": round(st["max_ulp_conditioned"], 3),
                "max_err_relative_to_sum_of_abs_products": float("%.4g" % st["max_rel_to_bound"])}

    def to_dev(a):
        a = np.ascontiguousarray(a)
        if a.dtype == np.uint16:  # bf16 bit patterns
            return torch.from_numpy(a.view(np.int16)).to(dev)
        return torch.from_numpy(a).to(dev)

    cfg = "c3" if args.config == "launch_floor" else args.config
    if cfg == "copy":
        # what the memory system sustains: copy, read-only and write-only passes over one buffer (1 GiB by default,
        # four times the 256 MiB last-level cache; --copy-mib 64 is the known-size dispatch that calibrates the
        # FETCH_SIZE / WRITE_SIZE counters)
        nbytes = args.copy_mib << 20
        src = torch.zeros(nbytes, dtype=torch.int8, device=dev)
        dst = torch.empty_like(src)
        out = {"metric": "streaming rates of the box", "unit": "GB/s", "bytes": nbytes}
        for mode, name, moved in ((0, "copy", 2 * nbytes), (1, "read", nbytes), (2, "write", nbytes),
                                  (3, "read_into_lds", nbytes)):
            n_steps = args.steps or 20
            for _ in range(3):
                ctx.stream_probe(mode, src, dst, nbytes)
            evs = [torch.cuda.Event(enable_timing=True) for _ in range(n_steps + 1)]
            for i in range(n_steps):
                evs[i].record(stream)
                ctx.stream_probe(mode, src, dst, nbytes)
            evs[n_steps].record(stream)
            torch.cuda.synchronize()
            t = sorted(evs[i].elapsed_time(evs[i + 1]) * 1e-3 for i in range(n_steps))[n_steps // 2]
            out[name] = {"GB_per_s": round(moved / t / 1e9, 1), "us": round(t * 1e6, 2), "bytes_moved": moved,
                         "frac_of_8TBps": round(moved / t / 8e12, 4)}
        print(json.dumps(out))
        ctx.close()
        return 0
    if cfg == "networks":
        # Beyond the named configurations: the int8 layers of ResNet-50 (the first and a following block of every stage)
        # and MobileNetV2 (every block), CONV2D or DEPTHWISE_CONV2D with the fused per-channel RESCALE under the library's
        # own kernel choice, each timed alone by graph replay.  "floor" is the launch floor plus the larger of ops / 5 POP/s and bytes / 8 TB/s.
        N, rng, layers = args.batch, np.random.default_rng(cases.SEED), []
        layers.append(("r50 conv1 7x7 s2", False, 224, 3, 64, 7, 2))
        for hw, cin, mid, cout, s in ((56, 64, 64, 256, 1), (56, 256, 64, 256, 1), (56, 256, 128, 512, 2), (28, 512, 128, 512, 1),
                                      (28, 512, 256, 1024, 2), (14, 1024, 256, 1024, 1), (14, 1024, 512, 2048, 2), (7, 2048, 512, 2048, 1)):
            layers.append(("r50 1x1 %d->%d @%d" % (cin, mid, hw), False, hw, cin, mid, 1, 1))
            layers.append(("r50 3x3 %d s%d @%d" % (mid, s, hw), False, hw, mid, mid, 3, s))
            layers.append(("r50 1x1 %d->%d @%d" % (mid, cout, hw // s), False, hw // s, mid, cout, 1, 1))
        layers.append(("mbv2 conv1 3x3 s2", False, 224, 3, 32, 3, 2))
        layers.append(("mbv2 dw 32 s1 @112", True, 112, 32, 32, 3, 1))
        layers.append(("mbv2 1x1 32->16 @112", False, 112, 32, 16, 1, 1))
        for hw, cin, e, cout, s in ((112, 16, 96, 24, 2), (56, 24, 144, 24, 1), (56, 24, 144, 32, 2), (28, 32, 192, 32, 1),
                                    (28, 32, 192, 64, 2), (14, 64, 384, 64, 1), (14, 64, 384, 96, 1), (14, 96, 576, 96, 1),
                                    (14, 96, 576, 160, 2), (7, 160, 960, 160, 1), (7, 160, 960, 320, 1)):
            layers.append(("mbv2 1x1 %d->%d @%d" % (cin, e, hw), False, hw, cin, e, 1, 1))
            layers.append(("mbv2 dw %d s%d @%d" % (e, s, hw), True, hw, e, e, 3, s))
            layers.append(("mbv2 1x1 %d->%d @%d" % (e, cout, hw // s), False, hw // s, e, cout, 1, 1))
        layers.append(("mbv2 1x1 320->1280 @7", False, 7, 320, 1280, 1, 1))
        launch_floor_us, rows = 1.67, []
        for name, depthwise, hw, ic, oc, k, s in layers:
            p = k // 2
            oh = (hw + 2 * p - k) // s + 1
            ih = (oh - 1) * s + k - 2 * p    # exact output size
            x = to_dev(rng.integers(-128, 128, (N, ih, ih, ic), dtype=np.int8))
            w = to_dev(rng.integers(-128, 128, (k, k, ic, 1) if depthwise else (oc, k, k, ic), dtype=np.int8))
            macs = N * oh * oh * oc * k * k * (1 if depthwise else ic)
            b = to_dev(rng.integers(-1000, 1000, oc, dtype=np.int32))
            m = to_dev(rng.integers(1 << 29, 1 << 30, oc, dtype=np.int32))
            sh = to_dev(np.full(oc, 38, np.int8))
            out = torch.empty((N, oh, oh, oc), dtype=torch.int8, device=dev)
            d = ctx.conv_desc(capi.INT8, capi.INT32, (N, ih, ih, ic), oc, k, k, (oh, oh), (p, p, p, p), (s, s), (1, 1), oc)
            r = ctx.rescale_desc(capi.INT32, capi.INT8, oc, oc, 0, 3, True, capi.ROUND_DOUBLE, True)
            fn = ctx.depthwise_conv2d_rescale_clamp if depthwise else ctx.conv2d_rescale_clamp

            def step():
                fn(d, x, w, b, -3, 0, r, m, sh, out, None)
            for _ in range(5):
                step()
            torch.cuda.synchronize()
            kernel = ctx.last_kernel
            g, side = torch.cuda.CUDAGraph(), torch.cuda.Stream()
            side.wait_stream(stream)
            with torch.cuda.graph(g, stream=side):
                ctx.set_stream(side.cuda_stream)
                for _ in range(50):
                    step()
            ctx.set_stream(stream.cuda_stream)
            g.replay()
            torch.cuda.synchronize()
            ts = []
            for _ in range(15):
                e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
                e0.record(stream)
                g.replay()
                e1.record(stream)
                torch.cuda.synchronize()
                ts.append(e0.elapsed_time(e1) * 20.0)
            us = sorted(ts)[len(ts) // 2]
            nbytes = x.numel() + w.numel() + out.numel() + 9 * oc
            floor = launch_floor_us + max(2 * macs / 5e15, nbytes / 8e12) * 1e6
            rows.append({"layer": name, "us": round(us, 2), "floor_us": round(floor, 2), "kernel": kernel})
        print(json.dumps({"metric": "sum over 62 int8 layers of ResNet-50 and MobileNetV2, each timed alone",
                          "unit": "us", "value": round(sum(r["us"] for r in rows), 1), "higher_is_better": False,
                          "floor_us": round(sum(r["floor_us"] for r in rows), 1), "batch": N, "n_gpus": 1, "data": "synthetic",
                          "dtype": "int8", "config": {"workload": "int8 CONV2D / DEPTHWISE_CONV2D + RESCALE, per layer", "layers": rows}}))
        ctx.close()
        return 0
    def make_workload(cfg):
        """operands in HBM, the step function (one C-ABI call) and the description of one configuration"""
        W = {}
        if cfg == "rescale":
            # stand-alone RESCALE at a size where launch latency no longer matters: the int32 accumulators of eight
            # batches of the ResNet-style layer, per-channel, double round, to int8
            c = cases.c3()
            rng = np.random.default_rng(cases.SEED ^ 66)
            acc = rng.integers(-(1 << 23), 1 << 23, (64, 56, 56, 64)).astype(np.int32)
            tacc, tm, ts = to_dev(acc), to_dev(c["mult"]), to_dev(c["shift"])
            out = torch.empty(acc.shape, dtype=torch.int8, device=dev)
            r = ctx.rescale_desc(capi.INT32, capi.INT8, 64, 64, 0, -3, True, capi.ROUND_DOUBLE, True)
            rows = acc.size // 64

            def step():
                ctx.rescale(r, 4, rows, 64, tacc, tm, ts, out)

            def cpu_ref():
                return the_oracle().rescale(acc[:8], c["mult"], c["shift"], out_zp=-3)[0]

            W = dict(ops=acc.size, bytes=acc.nbytes + acc.size + 64 * 5, exact=True, cpu_ref=cpu_ref, cpu_fraction=1 / 8,
                     result=lambda: out[:8].cpu().numpy(), dtype="int64",
                     metric="stand-alone RESCALE int32->int8 GB/s; % HBM peak; bit-exact", unit="GB/s", bound="hbm",
                     peak=PEAK["hbm"], runit="GB/s",
                     workload="RESCALE int32 [64,56,56,64] -> int8, per-channel multiplier/shift 38, double_round, "
                              "output_zp -3 (5 bytes per element)")
        elif cfg == "precise":
            # the fp64 precise-mode pass of the compliance flow at the shape of the named fp16 CONV2D configuration
            c = cases.c5_conv()
            n, ih, iw, ic = c["x"].shape
            oc, kh, kw, _ = c["w"].shape
            tx, tw, tb = to_dev(c["x"]), to_dev(c["w"]), to_dev(c["bias"])
            out = torch.empty((n, ih, iw, oc), dtype=torch.float64, device=dev)
            d = ctx.conv_desc(capi.FP16, capi.FP16, (n, ih, iw, ic), oc, kh, kw, (ih, iw), c["pad"], c["stride"],
                              c["dilation"], oc)
            step = lambda: ctx.conv2d_precise(d, tx, tw, tb, False, out)
            x64, w64, b64 = (c[k].astype(np.float64) for k in ("x", "w", "bias"))
            cpu_ref = lambda: the_oracle().conv2d("f64", x64[:1], w64, b64, c["pad"], c["stride"], c["dilation"])
            W = dict(ops=2 * n * ih * iw * oc * kh * kw * ic, bytes=c["x"].nbytes + c["w"].nbytes + c["bias"].nbytes +
                     out.numel() * 8, exact=True, cpu_ref=cpu_ref, cpu_fraction=1.0 / n, parallel_oracle=True,
                     result=lambda: out[:1].cpu().numpy(), dtype="f64",
                     metric="fp64 precise-mode CONV2D TFLOPS 3x3 [16,28,28,256]x[256,3,3,256]; bit-exact vs the fp64 oracle",
                     unit="TFLOPS", bound="mfma", peak=78.6, runit="TFLOP/s",
                     workload="precise-mode (fp64) pass of configs[4a]: CONV2D 3x3 [16,28,28,256]x[256,3,3,256] s1 p1, "
                              "fp16 operands, fp64 products and sums in the reference's loop order")
        elif cfg in ("maxpool", "avgpool"):
            # the pooling neighbours at sizes where launch latency no longer dominates: the 3x3 stride-2 max pooling
            # behind a ResNet stem for 32 images, and a 2x2 stride-2 average pooling of the same tensor
            rng = np.random.default_rng(cases.SEED ^ (8 if cfg == "maxpool" else 2))
            x = rng.integers(-128, 128, (32, 112, 112, 64)).astype(np.int8)
            pk, ps, pp = ((3, 3), (2, 2), (0, 1, 0, 1)) if cfg == "maxpool" else ((2, 2), (2, 2), (0, 0, 0, 0))
            d = capi.PoolDesc()
            d.dtype, d.acc_dtype = capi.INT8, capi.INT32
            d.N, d.IH, d.IW, d.C, d.OH, d.OW = 32, 112, 112, 64, 56, 56
            d.kernel[:], d.stride[:], d.pad[:], d.nan_mode = list(pk), list(ps), list(pp), 1
            tx = to_dev(x)
            out = torch.empty((32, 56, 56, 64), dtype=torch.int8, device=dev)
            if cfg == "maxpool":
                step = lambda: ctx.max_pool2d(d, tx, out)
                cpu_ref = lambda: the_oracle().max_pool2d(x[:4], pk, ps, pp)
            else:
                step = lambda: ctx.avg_pool2d(d, tx, -3, 4, out)
                cpu_ref = lambda: the_oracle().avg_pool2d(x[:4], pk, ps, pp, -3, 4)
            W = dict(ops=out.numel() * pk[0] * pk[1], bytes=x.nbytes + out.numel(), exact=True, cpu_ref=cpu_ref,
                     cpu_fraction=1 / 8, result=lambda: out[:4].cpu().numpy(), dtype="int8" if cfg == "maxpool" else "int32",
                     metric="int8 %s GB/s; %% HBM peak; bit-exact" % ("MAX_POOL2D" if cfg == "maxpool" else "AVG_POOL2D"),
                     unit="GB/s", bound="hbm", peak=PEAK["hbm"], runit="GB/s",
                     workload="%s int8 [32,112,112,64] -> [32,56,56,64], kernel %s stride %s pad %s%s"
                              % ("MAX_POOL2D" if cfg == "maxpool" else "AVG_POOL2D", list(pk), list(ps), list(pp),
                                 "" if cfg == "maxpool" else ", input_zp -3, output_zp 4"))
        elif cfg in ("tconv", "conv3d"):
            # the two neighbouring operators, at shapes of the same family as the named CONV2D configuration (no
            # configuration of theirs is named): the timed step includes the operand re-layout kernels
            rng = np.random.default_rng(cases.SEED ^ (10 if cfg == "tconv" else 4))
            if cfg == "tconv":
                x = rng.integers(-128, 128, (8, 28, 28, 128)).astype(np.int8)
                w = np.clip(np.rint(rng.normal(0, 30, (64, 3, 3, 128))), -127, 127).astype(np.int8)
                bias = np.rint(rng.normal(0, 2 ** 14, 64)).astype(np.int32)
                out_pad, stride = (0, 1, 0, 1), (2, 2)
                oh = ow = (28 - 1) * 2 + 1 + 3
                d = capi.TconvDesc()
                d.in_dtype, d.out_dtype = capi.INT8, capi.INT32
                d.N, d.IH, d.IW, d.IC, d.OC, d.KH, d.KW, d.OH, d.OW = 8, 28, 28, 128, 64, 3, 3, oh, ow
                d.out_pad[:], d.stride[:], d.bias_len = list(out_pad), list(stride), 64
                out = torch.empty((8, oh, ow, 64), dtype=torch.int32, device=dev)
                macs = 8 * oh * ow * 64 * 9 * 128    # dense count over the zero-inserted input, as for CONV2D
                fn, name = ctx.transpose_conv2d, "TRANSPOSE_CONV2D [8,28,28,128]x[64,3,3,128] s2 out_pad [0,1,0,1] -> [8,56,56,64] int32"

                def cpu_ref():
                    return the_oracle().transpose_conv2d("i8", x[:1], w, bias, out_pad, stride, -7, 0)
                frac = 1 / 8
            else:
                x = rng.integers(-128, 128, (2, 16, 28, 28, 32)).astype(np.int8)
                w = np.clip(np.rint(rng.normal(0, 30, (64, 3, 3, 3, 32))), -127, 127).astype(np.int8)
                bias = np.rint(rng.normal(0, 2 ** 14, 64)).astype(np.int32)
                pad, st3, dil = (1, 1, 1, 1, 1, 1), (1, 1, 1), (1, 1, 1)
                d = capi.Conv3dDesc()
                d.in_dtype, d.out_dtype = capi.INT8, capi.INT32
                d.N, d.ID, d.IH, d.IW, d.IC, d.OC, d.KD, d.KH, d.KW = 2, 16, 28, 28, 32, 64, 3, 3, 3
                d.OD, d.OH, d.OW = 16, 28, 28
                d.pad[:], d.stride[:], d.dilation[:], d.bias_len = list(pad), list(st3), list(dil), 64
                out = torch.empty((2, 16, 28, 28, 64), dtype=torch.int32, device=dev)
                macs = 2 * 16 * 28 * 28 * 64 * 27 * 32
                fn, name = ctx.conv3d, "CONV3D [2,16,28,28,32]x[64,3,3,3,32] s1 p1 -> [2,16,28,28,64] int32"

                def cpu_ref():
                    return the_oracle().conv3d("i8", x[:1], w, bias, pad, st3, dil, -7, 0)
                frac = 1 / 2
            tx, tw, tb = to_dev(x), to_dev(w), to_dev(bias)

            def step():
                fn(d, tx, tw, tb, -7, 0, out)

            W = dict(ops=2 * macs, bytes=x.nbytes + w.nbytes + bias.nbytes + out.numel() * 4, exact=True, cpu_ref=cpu_ref,
                     cpu_fraction=frac, result=lambda: out[:1].cpu().numpy(), dtype="int8",
                     metric="int8 %s TOPS; %% int8 MFMA peak; bit-exact" % cfg.upper(), unit="TOPS", bound="mfma",
                     peak=PEAK["int8_mfma"], runit="TOP/s", workload="INT8 " + name)
        elif cfg in ("c1", "c3", "c3x4", "c4", "c4x8", "dw32"):
            c = {"c1": cases.c1, "c3": cases.c3, "c3x4": lambda: cases.c3(n=32), "c4": cases.c4,
                 "c4x8": lambda: cases.c4(n=64), "dw32": lambda: cases.c4(n=64, c=32, stride=1)}[cfg]()
            depthwise = cfg in ("c4", "c4x8", "dw32")
            n, ih, iw, ic = c["x"].shape
            if depthwise:
                kh, kw, _, m = c["w"].shape
                oc = ic * m
            else:
                oc, kh, kw, _ = c["w"].shape
            oh, ow = conv_out_hw(ih, iw, kh, kw, c["pad"], c["stride"], c["dilation"])
            macs = n * oh * ow * oc * kh * kw * (1 if depthwise else ic)
            t = {k: to_dev(c[k]) for k in ("x", "w", "bias", "mult", "shift")}
            out = torch.empty((n, oh, ow, oc), dtype=torch.int8, device=dev)
            d = ctx.conv_desc(capi.INT8, capi.INT32, (n, ih, iw, ic), oc, kh, kw, (oh, ow), c["pad"], c["stride"],
                              c["dilation"], c["bias"].shape[0])
            r = ctx.rescale_desc(capi.INT32, capi.INT8, oc, oc, 0, c["out_zp"], True, capi.ROUND_DOUBLE, True)
            fn = ctx.depthwise_conv2d_rescale_clamp if depthwise else ctx.conv2d_rescale_clamp

            def step():
                fn(d, t["x"], t["w"], t["bias"], c["in_zp"], c["w_zp"], r, t["mult"], t["shift"], out, c["clamp"])

            def cpu_ref():
                f = the_oracle().depthwise_conv2d if depthwise else the_oracle().conv2d
                acc = f("i8", c["x"], c["w"], c["bias"], c["pad"], c["stride"], c["dilation"], c["in_zp"], c["w_zp"])
                ref, _ = the_oracle().rescale(acc, c["mult"], c["shift"], out_zp=c["out_zp"])
                return ref if c["clamp"] is None else the_oracle().clamp(ref, *c["clamp"])

            W = dict(ops=2 * macs, bytes=sum(c[k].nbytes for k in ("x", "w", "bias", "mult", "shift")) + out.numel(),
                     exact=True, cpu_ref=cpu_ref, cpu_fraction=1.0, result=lambda: out.cpu().numpy(), dtype="int8",
                     parallel_oracle=True)
            if cfg == "c1":
                W.update(metric="int8 CONV2D 1x1 + RESCALE GB/s at the reference's example shape; bit-exact", unit="GB/s",
                         bound="hbm", peak=PEAK["hbm"], runit="GB/s",
                         workload="configs[0]: INT8 CONV2D 1x1 [1,32,32,8]x[16,1,1,8] + per-channel RESCALE (shift 36..40, "
                                  "double_round, output_zp 5), fused (launch-bound: a correctness configuration)")
            elif cfg in ("c3", "c3x4"):
                W.update(metric="int8 CONV2D+RESCALE TOPS at 3x3 ResNet shape; % int8 MFMA peak; bit-exact", unit="TOPS",
                         bound="mfma", peak=PEAK["int8_mfma"], runit="TOP/s",
                         workload="configs[2]: INT8 CONV2D ResNet-style 3x3 [8,56,56,64]x[64,3,3,64] s1 p1 + per-channel "
                                  "RESCALE (shift 38, double_round) + CLAMP [0,127], fused")
                if cfg == "c3x4":    # the same layer at four times the batch: the kernel's rate with the launch amortised
                    W["workload"] = W["workload"].replace("configs[2]: ", "").replace("[8,56,56,64]", "[32,56,56,64]") + \
                        " (4x the named batch; never the headline)"
            else:
                W.update(metric="int8 DEPTHWISE_CONV2D+RESCALE GB/s at MobileNetV2 shape; % HBM peak; bit-exact",
                         unit="GB/s", bound="hbm", peak=PEAK["hbm"], runit="GB/s",
                         workload="configs[3]: INT8 DEPTHWISE_CONV2D [8,112,112,96] 3x3 s2 pad [0,1,0,1] + per-channel "
                                  "RESCALE (shift 34..40, double_round), fused")
                if cfg == "c4x8":    # the same layer at eight times the batch: the kernel's rate without the launch floor
                    W["workload"] = W["workload"].replace("[8,112,112,96]", "[64,112,112,96]") + " (8x the named batch)"
                if cfg == "dw32":    # the network's first depthwise layer, 64 images: no named configuration
                    W["workload"] = "INT8 DEPTHWISE_CONV2D [64,112,112,32] 3x3 s1 pad 1 + per-channel RESCALE (shift 34..40, " \
                                    "double_round), fused (MobileNetV2's first depthwise layer; not a named configuration)"
        elif cfg in ("c2", "c5b"):
            c = cases.c2() if cfg == "c2" else cases.c5_matmul()
            n, h, k = c["a"].shape
            w = c["b"].shape[2]
            in_dtype = capi.INT8 if cfg == "c2" else capi.BF16
            ta, tb = to_dev(c["a"]), to_dev(c["b"])
            out = torch.empty((n, h, w), dtype=torch.int32 if cfg == "c2" else torch.float32, device=dev)
            a_zp, b_zp = (c["a_zp"], c["b_zp"]) if cfg == "c2" else (0, 0)

            def step():
                ctx.matmul(in_dtype, n, h, k, w, ta, tb, a_zp, b_zp, out)

            rows = 64 if cfg == "c2" else 8  # bounded CPU sample: the first `rows` rows of batch 0

            def cpu_ref():
                if cfg == "c2":
                    return the_oracle().matmul("i8", c["a"][:1, :rows], c["b"][:1], a_zp, b_zp)
                return the_oracle().matmul("f32", cases.bf16_bits_to_float(c["a"][:1, :rows]), cases.bf16_bits_to_float(c["b"][:1]))

            W = dict(ops=2 * n * h * k * w, bytes=c["a"].nbytes + c["b"].nbytes + out.numel() * 4, exact=cfg == "c2",
                     cpu_ref=cpu_ref, cpu_fraction=rows / (n * h), result=lambda: out[:1, :rows].cpu().numpy(),
                     dtype="int8" if cfg == "c2" else "bf16", parallel_oracle=True)
            if cfg == "c5b":
                def accuracy(device_only=False):
                    ref = torch.empty((n, h, w), dtype=torch.float64, device=dev)
                    bnd = torch.empty_like(ref)
                    ctx.matmul_precise(in_dtype, n, h, k, w, ta, tb, False, ref)
                    ctx.matmul_precise(in_dtype, n, h, k, w, ta, tb, True, bnd)
                    return accuracy_figures(out, ref, bnd, "fp32", capi.FP32, k, False, device_only)
                W["accuracy"] = accuracy
            if cfg == "c2":
                W.update(metric="int8 MATMUL TOPS [8,1024,1024]x[8,1024,1024]; bit-exact", unit="TOPS", bound="hbm",
                         peak=PEAK["hbm"], runit="GB/s",
                         workload="configs[1]: INT8 MATMUL [8,1024,1024]x[8,1024,1024] -> int32, a_zp -5, b_zp 3")
            else:
                W.update(metric="bf16 MATMUL TFLOPS [4,2048,4096]x[4,4096,2048], fp32 accumulate", unit="TFLOPS",
                         bound="mfma", peak=PEAK["f16_mfma"], runit="TFLOP/s",
                         workload="configs[4b]: BF16 MATMUL [4,2048,4096]x[4,4096,2048] -> fp32")
        else:  # c5a
            c = cases.c5_conv()
            n, ih, iw, ic = c["x"].shape
            oc, kh, kw, _ = c["w"].shape
            tx, tw, tb = to_dev(c["x"]), to_dev(c["w"]), to_dev(c["bias"])
            out = torch.empty((n, ih, iw, oc), dtype=torch.float16, device=dev)
            d = ctx.conv_desc(capi.FP16, capi.FP16, (n, ih, iw, ic), oc, kh, kw, (ih, iw), c["pad"], c["stride"],
                              c["dilation"], oc)

            def step():
                ctx.conv2d(d, tx, tw, tb, 0, 0, out)


            def cpu_ref():  # bounded CPU sample: image 0 only
                return the_oracle().conv2d("f32", c["x"][:1], c["w"], c["bias"], c["pad"], c["stride"], c["dilation"])

            W = dict(ops=2 * n * ih * iw * oc * kh * kw * ic, bytes=c["x"].nbytes + c["w"].nbytes + c["bias"].nbytes +
                     out.numel() * 2, exact=False, cpu_ref=cpu_ref, cpu_fraction=1.0 / n, parallel_oracle=True,
                     result=lambda: out[:1].cpu().numpy(), dtype="fp16",
                     metric="fp16 CONV2D TFLOPS 3x3 [16,28,28,256]x[256,3,3,256], fp32 accumulate", unit="TFLOPS",
                     bound="mfma", peak=PEAK["f16_mfma"], runit="TFLOP/s",
                     workload="configs[4a]: FP16 CONV2D 3x3 [16,28,28,256]x[256,3,3,256] s1 p1, fp32 accumulate")

            def accuracy(device_only=False):
                ref = torch.empty((n, ih, iw, oc), dtype=torch.float64, device=dev)
                bnd = torch.empty_like(ref)
                ctx.conv2d_precise(d, tx, tw, tb, False, ref)
                ctx.conv2d_precise(d, tx, tw, tb, True, bnd)
                return accuracy_figures(out, ref, bnd, "fp16", capi.FP16, kh * kw * ic, True, device_only)

            # a cheaper CPU sample for the short leg of the default run: the first four output rows of image 0
            W["quick_ref"] = lambda: the_oracle().conv2d("f32", c["x"][:1, :5], c["w"], c["bias"], (1, 0, 1, 1), c["stride"],
                                                         c["dilation"])
            W["quick_result"] = lambda: out[:1, :4].cpu().numpy()
            W["accuracy"] = accuracy

        return W, step

    W, step = make_workload(cfg)

    if args.config == "launch_floor":
        # a kernel that does nothing, launched with the grid, block and LDS size the headline kernel has just used
        step()
        ctx.sync()
        grid, block, lds = ctx.last_launch_shape()
        if not grid:
            print("bench.py: the headline configuration did not run on the kernel whose launch is measured", file=sys.stderr)
            return 1
        step = lambda: ctx.launch_empty(grid, block, lds)
        W = dict(ops=0, bytes=0, exact=True, cpu_ref=None, cpu_fraction=0.0, result=None, dtype="none",
                 metric="launch floor: microseconds per launch of a kernel without work", unit="us", bound="hbm",
                 peak=PEAK["hbm"], runit="GB/s", workload="empty kernel, %d workgroups of %d threads, %d bytes of LDS each "
                 "(the launch shape of configs[2]'s kernel)" % (grid, block, lds))
        cfg = "launch_floor"

    big = cfg in ("c5b", "precise")
    steps = args.steps if args.steps is not None else (200 if big else 2000)
    warmup = args.warmup if args.warmup is not None else (20 if big else 200)
    repeats = args.repeats if args.repeats is not None else max(5, min(500, -(-10000 // steps)))
    if big and args.repeats is None:
        repeats = 5

    def measure(step, steps, warmup, repeats, use_graph):
        """`warmup` untimed steps, then the region of `steps` steps `repeats` times back to back.  The host clock
        brackets all of it with a synchronisation on both sides; HIP events on the launch stream cut it into timed
        units: one graph replay (a graph holds up to 100 steps and may span several short regions, since a replay
        costs about 10 us by itself), or one region when every step is launched from the host.  A GPU that has just
        woken up runs its first units at ramping clocks: the median unit is the figure reported.  Returns the
        sorted seconds per step of the units, the host clock's seconds per step, and the unit layout."""
        for _ in range(warmup):
            step()
        torch.cuda.synchronize()
        total = steps * repeats
        chunk = math.gcd(total, 100) if use_graph else steps
        units = total // chunk
        graph = None
        if use_graph:
            # The steps are recorded into a HIP graph (nothing but their kernel launches) and the graph is replayed:
            # a launch from the host costs about as much as the small configurations' kernels run, and a serving
            # loop would not pay it per layer either.
            graph = torch.cuda.CUDAGraph()
            side = torch.cuda.Stream()
            side.wait_stream(stream)
            with torch.cuda.graph(graph, stream=side):
                ctx.set_stream(side.cuda_stream)
                for _ in range(chunk):
                    step()
            ctx.set_stream(stream.cuda_stream)
            graph.replay()    # untimed: the first replay uploads the graph
            torch.cuda.synchronize()
        events = [torch.cuda.Event(enable_timing=True) for _ in range(units + 1)]
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for u in range(units):
            events[u].record(stream)
            if use_graph:
                graph.replay()
            else:
                for _ in range(chunk):
                    step()
        events[units].record(stream)
        torch.cuda.synchronize()
        t1 = time.perf_counter()
        per_unit = sorted(events[i].elapsed_time(events[i + 1]) * 1e-3 / chunk for i in range(units))
        return per_unit, (t1 - t0) / total, (total, units, chunk)

    def median(v):
        return v[len(v) // 2] if len(v) % 2 else 0.5 * (v[len(v) // 2 - 1] + v[len(v) // 2])

    use_graph = not args.eager and cfg != "precise"    # --eager times host-issued launches instead of graph replays
    per_unit, host_s_per_step, (total, units, chunk) = measure(step, steps, warmup, repeats, use_graph)
    status = ctx.sync()
    kernel = ctx.last_kernel
    s_per_step = median(per_unit)
    ms_per_step = s_per_step * 1e3
    host_ms_per_step = host_s_per_step * 1e3

    if cfg == "launch_floor":
        print(json.dumps({"metric": W["metric"], "value": round(s_per_step * 1e6, 4), "unit": "us", "n_gpus": 1,
                          "steps": steps, "warmup": warmup, "repeats": repeats, "ms_per_step": round(ms_per_step, 6),
                          "higher_is_better": False, "data": "synthetic",
                          "config": {"workload": W["workload"], "kernel": kernel,
                                     "launch": "%d steps as %d HIP graphs of %d launches; the median graph by HIP "
                                               "events on the launch stream" % (total, units, chunk) if use_graph
                                     else "one host launch per step",
                                     "us_per_launch_fastest_unit": round(per_unit[0] * 1e6, 4),
                                     "us_per_launch_slowest_unit": round(per_unit[-1] * 1e6, 4),
                                     "host_clock_us_per_launch": round(host_ms_per_step * 1e3, 4)}}))
        ctx.close()
        return 0

    work = W["bytes"] / 1e9 if W["unit"] == "GB/s" else W["ops"] / 1e12
    value = work / s_per_step
    rwork = W["bytes"] / 1e9 if W["bound"] == "hbm" else W["ops"] / 1e12
    achieved = rwork / s_per_step

    launch = "%d repeats of the %d-step region back to back (%d steps), " % (repeats, steps, total)
    launch += ("replayed as %d HIP graphs of %d steps" % (units, chunk) if use_graph
               else "one host launch per step, %d units of %d steps" % (units, chunk))
    launch += "; ms_per_step = the median unit by HIP events on the launch stream"
    result = {"metric": W["metric"], "value": round(value, 3), "unit": W["unit"], "n_gpus": 1, "steps": steps,
              "warmup": warmup, "repeats": repeats, "ms_per_step": round(ms_per_step, 6), "higher_is_better": True,
              "scaling": "weak", "vs_baseline": None, "dtype": W["dtype"], "data": "synthetic",
              "config": {"workload": W["workload"], "kernel": kernel, "ops_per_step": W["ops"],
                         "algorithmic_bytes_per_step": W["bytes"], "graph_status": status, "launch": launch,
                         "ms_per_step_fastest_unit": round(per_unit[0] * 1e3, 6),
                         "ms_per_step_slowest_unit": round(per_unit[-1] * 1e3, 6),
                         "host_clock_ms_per_step_whole_region": round(host_ms_per_step, 6)},
              "roofline": {"bound": W["bound"], "achieved": round(achieved, 3), "peak": W["peak"], "unit": W["runit"],
                           "frac": round(achieved / W["peak"], 5), "traffic": None,
                           "us_per_launch": round(s_per_step * 1e6, 3)}}
    traffic, traffic_source = measured_traffic(cfg, kernel)
    result["roofline"]["traffic"] = traffic
    result["roofline"].update(traffic_source)
    if W["bound"] == "hbm" and W["unit"] != "GB/s":
        result["roofline"]["mfma_frac"] = round(W["ops"] / 1e12 / s_per_step / PEAK["int8_mfma"], 5)

    rc = 0
    if args.config == "c3" and not args.no_named_configs and not args.no_cpu_baseline:
        # The other named configurations, GPU leg only: the same graph replays and median unit over about a second of
        # steps each, and the result checked against the CPU oracle on a small sample (all of it where that is cheap).
        named = {}
        for name in ("c1", "c2", "c4", "c5a", "c5b"):
            Wn, stepn = make_workload(name)
            # as many steps as the headline's own measurement where a step is short: a leg of a few milliseconds reads
            # 5-10 % slow (the engine clock has not settled)
            n_steps = 3000 if name == "c5b" else 10000
            pu, _, _ = measure(stepn, n_steps, 200, 1, use_graph)
            st_n, kern_n, t_n = ctx.sync(), ctx.last_kernel, median(pu)
            got_n = (Wn.get("quick_result") or Wn["result"])()
            ref_n = (Wn.get("quick_ref") or Wn["cpu_ref"])()
            if Wn["exact"]:
                ok_n = bool(np.array_equal(got_n, ref_n))
                entry = {"bit_exact_vs_oracle_sample": ok_n}
            else:
                err = float(np.max(np.abs(got_n.astype(np.float64) - np.asarray(ref_n, np.float64)) /
                                   np.maximum(np.abs(np.asarray(ref_n, np.float64)), 1e-3)))
                acc_n = Wn["accuracy"](device_only=True)    # the whole result against the library's fp64 passes
                ok_n = err < 2e-2 and acc_n["dot_product_compliant"]
                entry = {"max_rel_err_vs_fp32_oracle_sample": float("%.3g" % err), "accuracy_vs_fp64": acc_n}
            rate = (Wn["bytes"] / 1e9 if Wn["bound"] == "hbm" else Wn["ops"] / 1e12) / t_n
            entry.update({"workload": Wn["workload"], "kernel": kern_n, "us": round(t_n * 1e6, 3), "steps": n_steps,
                          "bound": Wn["bound"], "achieved": round(rate, 2), "unit": Wn["runit"],
                          "frac": round(rate / Wn["peak"], 5), "graph_status": st_n, "ok": bool(ok_n and st_n == 0)})
            if Wn["bound"] == "hbm" and Wn["unit"] != "GB/s":
                entry["mfma_frac"] = round(Wn["ops"] / 1e12 / t_n / PEAK["int8_mfma"], 5)
            named[name] = entry
            if not entry["ok"]:
                print("bench.py: %s differs from the oracle" % name, file=sys.stderr)
                rc = 1
            del Wn, stepn
            torch.cuda.empty_cache()
        result["config"]["named_configs"] = named
    if not args.no_cpu_baseline:
        got = W["result"]()

        def time_oracle(budget):
            # repeated over the sample until about `budget` seconds of CPU work have been timed
            best, ref, spent, runs = None, None, 0.0, 0
            while runs < 3 or (spent < budget and runs < 400):
                c0 = time.perf_counter()
                ref = W["cpu_ref"]()
                dt = time.perf_counter() - c0
                best = dt if best is None else min(best, dt)
                spent += dt
                runs += 1
                if best > budget:
                    break
            return best, ref, spent, runs

        orc = the_oracle()
        orc.set_parallel(False)
        best, ref, spent, runs = time_oracle(10.0)
        if W["exact"]:
            ok = bool(np.array_equal(got, ref))
            result["config"]["bit_exact_vs_oracle"] = ok
        else:
            g64 = got.astype(np.float64)
            r64 = np.asarray(ref, np.float64)
            err = float(np.max(np.abs(g64 - r64) / np.maximum(np.abs(r64), 1e-3)))
            ok = err < 2e-2  # sanity only: the figures against fp64 follow
            result["config"]["max_rel_err_vs_fp32_oracle"] = err
            if "accuracy" in W:
                acc = W["accuracy"]()
                result["config"]["accuracy_vs_fp64"] = acc
                ok = ok and acc["dot_product_compliant"]
        cpu_work = work * W["cpu_fraction"]
        cpu_model = "unknown"
        try:
            with open("/proc/cpuinfo") as f:
                cpu_model = next(line.split(":", 1)[1].strip() for line in f if line.startswith("model name"))
        except (OSError, StopIteration):
            pass
        sample = "whole batch" if W["cpu_fraction"] == 1.0 else "leading rows / first image"
        result["cpu_baseline"] = {"value": round(cpu_work / best, 6), "unit": W["unit"], "cores": 1, "kind": "port",
                                  "sample": "%.4g of one step's work (%s), fastest of %d runs of the scalar C oracle "
                                            "(%.1f s of CPU work in all), %.3f s per run"
                                            % (W["cpu_fraction"], sample, runs, spent, best),
                                  "cpu_model": cpu_model, "host_logical_cpus": os.cpu_count()}
        if W.get("parallel_oracle"):
            # the same C source built with OpenMP: the operator's outer loops over all the threads the host grants
            orc.set_parallel(True)
            threads = orc.threads()
            pbest, pref, pspent, pruns = time_oracle(5.0)
            orc.set_parallel(False)
            same = bool(np.array_equal(np.asarray(pref), np.asarray(ref)))
            result["cpu_baseline"]["all_cores"] = {
                "value": round(cpu_work / pbest, 6), "unit": W["unit"], "cores": threads, "kind": "port",
                "sample": "the same sample with the OpenMP build of the oracle on %d threads, fastest of %d runs, "
                          "%.3f s per run; results identical to the scalar build: %s" % (threads, pruns, pbest, same)}
        if not ok:
            print("bench.py: GPU result differs from the oracle", file=sys.stderr)
            rc = 1
    print(json.dumps(result))
    ctx.close()
    return rc


if __name__ == "__main__":
    sys.exit(main())
