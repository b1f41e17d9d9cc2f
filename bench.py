#!/usr/bin/env python3
"""Benchmark of the quantized-inference hot path on one MI355X.

A step = one forward pass of the ResNet-50-shaped int8 case (BASELINE.json configs[4]: 64x3x224x224 fp32
input -> quantize -> 53 uint8 convs, 16 residual adds, 2 pools, FC 2048->1000 -> dequantize) over one
synthetic batch that is already resident in HBM.  The pass is recorded once into a HIP graph and replayed.

Prints ONE JSON line with images/s (`value`), the roofline figures of the dominant kernel (the int8 MFMA
convolution: algorithmic ops of all its launches / their measured durations, against the chip's dense int8
MFMA peak) and the reference CPU quant module timed on this box's host cores on a bounded sample.
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

PEAK_INT8_TOPS = 5000.0   # MI355X dense int8 MFMA, TOP/s (published)
PEAK_HBM_GBS = 8000.0     # MI355X HBM3E, GB/s (published)
# HBM bytes per launch of the dominant kernel family, from rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE runs of this very
# command (profiles/conv_mfma_i8_resnet50_n64.md holds the counter readings and the copy-kernel scale factors).
# A counter run cannot be made from inside the benchmark, so the figure is recorded here for the default workload.
MEASURED_TRAFFIC = {("resnet50", 64, True): 35.08e6}


def time_steps(fn, steps, warmup):
    import torch
    for _ in range(warmup):
        fn()
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    t0 = time.perf_counter()
    e0.record()
    for _ in range(steps):
        fn()
    e1.record()
    torch.cuda.synchronize()
    wall = (time.perf_counter() - t0) * 1e3
    return e0.elapsed_time(e1) / steps, wall / steps


def per_kernel_times(ex, reps):
    """Average duration of every launch of the pass, measured with HIP events on the launch stream around
    `reps` back-to-back launches of that one operator (inputs resident, same stream as the kernels)."""
    import torch
    out = []
    for s in ex.steps:
        for _ in range(3):
            s["fn"]()
        torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(reps):
            s["fn"]()
        e1.record()
        torch.cuda.synchronize()
        out.append(e0.elapsed_time(e1) / reps)
    return out


def cpu_baseline(case_builder, gpu_first_image, budget_s=30.0):
    """The reference CPU quant module (compiled from its own sources into oracle/_ref) on ONE image of the
    same network, one host thread (the reference has no threading).  Falls back to the oracle restatement
    ("port") where the compiled reference is absent.  Also cross-checks the GPU's output for that image."""
    import numpy as np
    from oracle import casecpu
    case1 = case_builder(1)
    x = gpu_first_image["x"]
    n_img = 1
    if casecpu.reference_available():
        kind = "reference"
        rc = casecpu.ReferenceCase(case1)
        t0 = time.perf_counter()
        y = rc.run(x)
        dt = time.perf_counter() - t0
        while dt < budget_s / 3 and n_img < 64:  # bounded sample: about 10 s of single-thread work
            rc.run(x)
            n_img += 1
            dt = time.perf_counter() - t0
    else:
        kind = "port"
        t0 = time.perf_counter()
        y = casecpu.run_case(case1, x)[case1.output.name]
        dt = time.perf_counter() - t0
    match = bool(np.array_equal(y.view(np.uint32), gpu_first_image["y"].view(np.uint32)))
    return {"value": round(n_img / dt, 4), "unit": "images/s", "cores": 1, "kind": kind,
            "sample": "%d batch-1 passes through all %d operators of the same network, %.2f s"
                      % (n_img, len(case1.nodes), dt),
            "output_equals_gpu": match}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--batch", type=int, default=None, help="images per step (fc: rows M); default 64, for --workload fc 128 (BASELINE configs[1])")
    ap.add_argument("--workload", default="resnet50", choices=["resnet50", "resnet18", "mobilenetv2", "conv", "fc"])
    ap.add_argument("--kernel-reps", type=int, default=20)
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--no-graph", action="store_true", help="launch eagerly instead of replaying a HIP graph")
    ap.add_argument("--no-fuse", action="store_true", help="run every residual add as its own kernel")
    ap.add_argument("--no-branches", action="store_true",
                    help="skip the extra measurement of the pass as two half-batch branches of one HIP graph")
    ap.add_argument("--layers", action="store_true", help="print a per-layer table to stderr")
    ap.add_argument("--tune", action="store_true",
                    help="before timing, let the executor search tile shape / load stages per convolution inside the network "
                         "(HipqExecutor.tune); off by default: the built-in choice is what a NART runner gets")
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="also launch a plain 256 MiB device copy (copy_bytes_kernel): the known-size reference that a "
                         "rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE run of this command is scaled by")
    args = ap.parse_args()
    if args.batch is None:
        args.batch = 128 if args.workload == "fc" else 64
    if args.gpus != 1:
        sys.exit("bench.py measures one GPU's share of the batch: this build runs on a single GPU only "
                 "(--gpus %d refused; batch-sharded inference needs no collectives)." % args.gpus)

    import numpy as np
    import torch
    from nart_amd import cases
    from nart_amd.runner import HipqExecutor
    if not torch.cuda.is_available():
        sys.exit("bench.py needs a GPU (the HIP path has no host fallback)")

    builders = {"resnet50": lambda n: cases.resnet50(N=n), "resnet18": lambda n: cases.resnet18(N=n),
                "mobilenetv2": lambda n: cases.mobilenet_v2(N=n), "conv": lambda n: cases.single_conv(N=n),
                "fc": lambda n: cases.single_fc(M=n)}
    build = builders[args.workload]
    case = build(args.batch)
    ex = HipqExecutor(case, fuse_add=not args.no_fuse)
    rng = np.random.default_rng(0)
    if case.input.dtype == "f32":
        x = (rng.standard_normal(case.input.shape) * 1.2).astype(np.float32)
    else:
        x = rng.integers(0, 256, case.input.shape, dtype=np.uint8)
    ex.set_input(x)
    ex.run()
    torch.cuda.synchronize()
    y = ex.output()

    if args.calibrate_copy:
        from nart_amd import hipq
        n = 256 << 20
        src = torch.zeros(n, dtype=torch.uint8, device="cuda")
        dst = torch.empty(n, dtype=torch.uint8, device="cuda")
        for _ in range(3):
            hipq.check(hipq.lib().hipq_copy_bytes(src.data_ptr(), dst.data_ptr(), n, torch.cuda.current_stream().cuda_stream))
        torch.cuda.synchronize()
        del src, dst

    if args.tune:
        ex.tune()
    if args.no_graph:
        step = ex.run
    else:
        ex.capture()
        step = ex.replay
    ms, wall_ms = time_steps(step, args.steps, args.warmup)

    # ---- per-kernel durations and the roofline of the dominant kernel ------------------------------------
    kt = per_kernel_times(ex, args.kernel_reps)
    fam = {}
    for s, t in zip(ex.steps, kt):
        key = "conv_mfma_i8" if s["kernel"].startswith("conv_mfma") else s["kernel"]
        f = fam.setdefault(key, {"ms": 0.0, "ops": 0, "bytes": 0, "launches": 0})
        f["ms"] += t
        f["ops"] += s["ops"]
        f["bytes"] += s["bytes"]
        f["launches"] += 1
    dom = max(fam, key=lambda k: fam[k]["ms"])
    d = fam[dom]
    if d["ops"] > 0:
        achieved = d["ops"] / (d["ms"] * 1e-3) / 1e12
        roof = {"kernel": dom, "bound": "mfma", "achieved": round(achieved, 2), "peak": PEAK_INT8_TOPS, "unit": "TOP/s",
                "frac": round(achieved / PEAK_INT8_TOPS, 4), "traffic": None}
    else:
        achieved = d["bytes"] / (d["ms"] * 1e-3) / 1e9
        roof = {"kernel": dom, "bound": "hbm", "achieved": round(achieved, 1), "peak": PEAK_HBM_GBS, "unit": "GB/s",
                "frac": round(achieved / PEAK_HBM_GBS, 4), "traffic": None}
    roof["traffic"] = MEASURED_TRAFFIC.get((args.workload, args.batch, not args.no_fuse))
    roof["algorithmic_bytes_per_launch"] = round(d["bytes"] / d["launches"])
    roof["algorithmic_ops_per_launch"] = round(d["ops"] / d["launches"]) if d["ops"] else None
    roof["launches_per_step"] = d["launches"]
    roof["avg_launch_us"] = round(d["ms"] / d["launches"] * 1e3, 2)
    roof["sum_kernel_ms"] = round(sum(kt), 4)
    families = {k: {"ms": round(v["ms"], 4), "launches": v["launches"],
                    "TOPs": round(v["ops"] / (v["ms"] * 1e-3) / 1e12, 2) if v["ops"] else None,
                    "GBs": round(v["bytes"] / (v["ms"] * 1e-3) / 1e9, 1)} for k, v in fam.items()}
    if args.layers:
        for s, t in zip(ex.steps, kt):
            tp = "%8.1f TOP/s" % (s["ops"] / (t * 1e-3) / 1e12) if s["ops"] else "            "
            shape = case.tensors[s["label"]].shape
            print("%-12s %-28s %-22s %8.1f us %s %8.1f GB/s" % (s["label"], s["kernel"], shape, t * 1e3, tp,
                                                                 s["bytes"] / (t * 1e-3) / 1e9), file=sys.stderr)

    # The two extra measurements below never decide whether the headline line is printed: a failure in them is reported
    # in the line instead.
    branched = in_flight = None
    try:
        # ---- the same pass as two half-batch branches of one graph (reported beside `value` as well) --------------------------------
        if not args.no_branches and not args.no_graph and args.batch >= 2:
            from nart_amd.runner import BranchedExecutor
            out_t = ex.buf[case.output.name]
            whole = out_t.clone()
            br = BranchedExecutor(ex, build, 2)
            out_t.zero_()
            br.capture()
            bms, _ = time_steps(br.replay, args.steps, args.warmup)
            branched = {"branches": 2, "ms_per_step": round(bms, 4), "value": round(args.batch / (bms * 1e-3), 1),
                        "output_equals_single_branch": bool(torch.equal(out_t, whole))}
            del br
        # ---- two batches in flight: a second copy of the network (own tensors, graph and stream) takes every other step and
        # nothing joins the two chains until the end of the timed region; throughput of the same K passes, reported beside
        # `value`, never as `value`: the roofline above is that of kernels launched one at a time ------------------------------------------------------------------------
        if not args.no_branches and not args.no_graph:
            from nart_amd.runner import PipelinedExecutor
            pipe = PipelinedExecutor(lambda: build(args.batch), depth=2, fuse_add=not args.no_fuse, first=ex)
            pipe.execs[1].set_input(x)
            torch.cuda.synchronize()
            for _ in range(2 * max(1, args.warmup)):
                pipe.submit()
            pipe.wait()
            t0 = time.perf_counter()
            for _ in range(args.steps):
                pipe.submit()
            pipe.wait()
            pms = (time.perf_counter() - t0) * 1e3 / args.steps
            same = torch.equal(pipe.execs[1].buf[case.output.name], ex.buf[case.output.name])
            in_flight = {"batches_in_flight": 2, "ms_per_step": round(pms, 4), "value": round(args.batch / (pms * 1e-3), 1),
                         "conv_tops_whole_step": round(case.conv_ops() / (pms * 1e-3) / 1e12, 2),
                         "timer": "host clock around the K submissions and the final synchronisation",
                         "outputs_equal_single_stream": bool(same)}
            del pipe
    except Exception as e:  # noqa: BLE001
        branched = branched or {"error": repr(e)}
        in_flight = in_flight or {"error": repr(e)}

    unit = "images/s"
    value = args.batch / (ms * 1e-3)
    res = {"metric": "ResNet-50-int8 images/sec @bs64; int8 conv TOPS (% of MFMA i8 peak)" if args.workload == "resnet50"
           else "%s images/sec" % args.workload,
           "value": round(value, 1), "unit": unit, "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
           "ms_per_step": round(ms, 4), "wall_ms_per_step": round(wall_ms, 4), "higher_is_better": True,
           "scaling": "weak", "vs_baseline": None, "dtype": "u8", "data": "synthetic",
           "config": {"workload": case.name, "batch": args.batch, "input": list(case.input.shape),
                      "operators": len(case.nodes), "graph_replay": not args.no_graph, "tuned": bool(args.tune), "fused_residual_adds": len(ex.fused),
                      "conv_fc_gop_per_step": round(case.conv_ops() / 1e9, 2)},
           "conv_tops_whole_step": round(case.conv_ops() / (ms * 1e-3) / 1e12, 2),
           "roofline": roof, "kernel_families": families}
    if branched is not None:
        res["two_branch_graph"] = branched
    if in_flight is not None:
        res["two_batches_in_flight"] = in_flight
    if not args.no_cpu:
        i0 = {"x": x[:1], "y": y[:1]}
        res["cpu_baseline"] = cpu_baseline(build, i0)
    print(json.dumps(res))


if __name__ == "__main__":
    main()
