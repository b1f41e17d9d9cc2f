#!/usr/bin/env python3
"""Benchmark of the quantized-inference hot path on one MI355X.

A step = one forward pass of the ResNet-50-shaped int8 case (BASELINE.json configs[4]: 64x3x224x224 fp32
input -> quantize -> 53 uint8 convs, 16 residual adds, 2 pools, FC 2048->1000 -> dequantize) over one
synthetic batch that is already resident in HBM.  The pass is recorded once into a HIP graph and replayed.

Prints ONE JSON line:
  value / ms_per_step   images/s of the single chain of kernels (K graph replays between two events on the launch stream)
  roofline              the dominant kernel family (the int8 MFMA convolutions): algorithmic ops of all its launches over
                        their measured durations, against the chip's dense int8 MFMA peak
  kernel_families       every family's time, TOP/s and GB/s (launch-by-launch timing, see per_kernel_times)
  sustained             the same replay loop kept running for at least two seconds
  library_int8_gemm     a yardstick: the vendor library's plain int8 GEMM (int32 output) on every layer's GEMM shape, summed,
                        beside the sum of this build's convolution-family launches
  module_path           the same network as an engine file run by nart_promark on the `hip` workspace (the drop-in path),
                        a child process
  other_workloads       BASELINE configs[0..3] at their stated sizes: time, rate, fraction of the roof that bounds them,
                        and a slice of the output compared with the CPU oracle
  cpu_baseline          the reference CPU quant module timed on this box's host cores on a bounded sample
"""
import argparse
import json
import os
import re
import subprocess
import sys
import tempfile
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

PEAK_INT8_TOPS = 5000.0   # MI355X dense int8 MFMA, TOP/s (published)
PEAK_HBM_GBS = 8000.0     # MI355X HBM3E, GB/s (published)
# HBM bytes per launch of the dominant kernel family, from rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE runs of this very
# command.  A counter run cannot be made from inside the benchmark, so the figure is carried here together with the
# file that holds the counter readings and a digest of the kernel sources it was taken with: the line reports it only
# for the default workload with default flags and only while the sources under nart_amd/csrc/hipq still have that digest
# (traffic is null, with the reason, once a kernel has changed and the profile has not been taken again).
TRAFFIC_FROM_PROFILE = {"workload": "resnet50", "batch": 64, "bytes_per_launch": 52.40e6,
                        "source": "profiles/conv_mfma_i8_resnet50_n64.md",
                        "sources_sha256": "7b2ea2a739053335"}


def kernel_sources_digest():
    """sha256 over the kernel sources (names and contents, in name order): ties a profile to the code it measured."""
    import hashlib
    d = os.path.join(ROOT, "nart_amd", "csrc", "hipq")
    h = hashlib.sha256()
    for f in sorted(os.listdir(d)):
        if f.endswith((".hip", ".h", ".cpp")):
            h.update(f.encode())
            with open(os.path.join(d, f), "rb") as fh:
                h.update(fh.read())
    return h.hexdigest()[:16]


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


def graph_of(fn, count, stream):
    """`count` calls of fn recorded into one HIP graph on `stream`."""
    import torch
    g = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g, stream=stream):
        for _ in range(count):
            fn()
    return g


def per_kernel_times(ex, reps):
    """Average duration of every launch of the pass: `reps` back-to-back launches of that one operator are recorded into
    a HIP graph of their own, and replays of that graph are bracketed by HIP events on the launch stream (a launch from
    Python costs more than the short kernels last, so eager launches would time the host).  Inputs are resident and warm:
    an upper bound of what the kernel does inside the pass, where its input was just written by another kernel."""
    import torch
    out = []
    st = torch.cuda.Stream()
    for s in ex.steps:
        s["fn"]()
        torch.cuda.synchronize()
        with torch.cuda.stream(st):
            g = graph_of(s["fn"], reps, st)

            def timed(warm, n):
                for _ in range(warm):
                    g.replay()
                torch.cuda.synchronize()
                e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
                e0.record(st)
                for _ in range(n):
                    g.replay()
                e1.record(st)
                torch.cuda.synchronize()
                return e0.elapsed_time(e1) / (n * reps)
            t = timed(3, 5)
            if t < 0.010:  # a kernel under 10 us: clocks and caches settle over more replays, and more are averaged
                t = timed(10, 20)
        out.append(t)
        del g
    return out


def families_of(ex, kt):
    fam = {}
    for s, t in zip(ex.steps, kt):
        key = "conv_mfma_i8" if s["kernel"].startswith("conv_mfma") else s["kernel"]
        f = fam.setdefault(key, {"ms": 0.0, "ops": 0, "bytes": 0, "launches": 0})
        f["ms"] += t
        f["ops"] += s["ops"]
        f["bytes"] += s["bytes"]
        f["launches"] += 1
    return fam


def roofline_of(fam, kt):
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
    roof["algorithmic_bytes_per_launch"] = round(d["bytes"] / d["launches"])
    roof["algorithmic_ops_per_launch"] = round(d["ops"] / d["launches"]) if d["ops"] else None
    roof["launches_per_step"] = d["launches"]
    roof["avg_launch_us"] = round(d["ms"] / d["launches"] * 1e3, 2)
    roof["sum_kernel_ms"] = round(sum(kt), 4)
    roof["timing"] = "HIP events on the launch stream around graph replays of back-to-back launches of each operator, inputs warm"
    roof["family_ms"] = round(d["ms"], 4)
    roof["other_kernels_ms"] = round(sum(kt) - d["ms"], 4)
    return roof


def add_in_pass(roof, ms_per_step):
    """The same fraction with the family's launches timed INSIDE the replayed step: the step minus the other kernels'
    durations, i.e. with every launch gap and every cold input of the pass charged to the family."""
    in_pass = ms_per_step - roof["other_kernels_ms"]
    if roof["bound"] == "mfma" and roof["algorithmic_ops_per_launch"] and in_pass > 0:
        ach = roof["algorithmic_ops_per_launch"] * roof["launches_per_step"] / (in_pass * 1e-3) / 1e12
        roof["achieved_in_pass"] = round(ach, 2)
        roof["frac_in_pass"] = round(ach / roof["peak"], 4)
        roof["avg_launch_us_in_pass"] = round(in_pass / roof["launches_per_step"] * 1e3, 2)


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


def random_input(case, seed=0):
    import numpy as np
    rng = np.random.default_rng(seed)
    if case.input.dtype == "f32":
        return (rng.standard_normal(case.input.shape) * 1.2).astype(np.float32)
    return rng.integers(0, 256, case.input.shape, dtype=np.uint8)


def measure_workload(build, batch, inner, kernel_reps, check_rows):
    """One of the other BASELINE configurations: a HIP graph of `inner` passes replayed a few times (a pass of one kernel
    is shorter than a graph launch), the per-kernel roofline of its dominant family, and the rows / images `check_rows`
    of the output compared with the CPU oracle run on those rows alone."""
    import numpy as np
    import torch
    from nart_amd.runner import HipqExecutor
    from oracle import casecpu
    case = build(batch)
    ex = HipqExecutor(case, fuse_add=True)
    x = random_input(case, seed=1)
    ex.set_input(x)
    ex.run()
    torch.cuda.synchronize()
    y = ex.output()
    st = torch.cuda.Stream()
    with torch.cuda.stream(st):
        g = graph_of(ex.run, inner, st)
        for _ in range(10):  # clocks and caches as in a loop that keeps running
            g.replay()
        torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        reps = 50
        e0.record(st)
        for _ in range(reps):
            g.replay()
        e1.record(st)
        torch.cuda.synchronize()
    ms = e0.elapsed_time(e1) / (reps * inner)
    del g
    kt = per_kernel_times(ex, kernel_reps)
    fam = families_of(ex, kt)
    roof = roofline_of(fam, kt)
    ok = True
    case1 = build(1)
    for i in check_rows:
        want = casecpu.run_case(case1, x[i:i + 1])[case1.output.name]
        got = np.ascontiguousarray(y[i:i + 1])
        ok = ok and bool(np.array_equal(got.view(np.uint8).reshape(-1), np.ascontiguousarray(want).view(np.uint8).reshape(-1)))
    d = fam[roof["kernel"]]
    res = {"workload": case.name, "ms_per_pass": round(ms, 5), "per_second": round(batch / (ms * 1e-3), 1),
           "conv_fc_gop": round(case.conv_ops() / 1e9, 3),
           "tops_whole_pass": round(case.conv_ops() / (ms * 1e-3) / 1e12, 2),
           "dominant_kernel": roof["kernel"], "bound": roof["bound"], "achieved": roof["achieved"], "unit": roof["unit"],
           "frac": roof["frac"], "avg_launch_us": roof["avg_launch_us"],
           "GBs_of_compulsory_bytes": round(d["bytes"] / (d["ms"] * 1e-3) / 1e9, 1),
           "output_equals_oracle": ok, "oracle_checked_rows": list(check_rows)}
    del ex
    return res


def library_gemm(case, ex, kt):
    """The vendor library's plain int8 GEMM (`torch._int_mm`: int8 x int8 -> int32, hipBLASLt) on the GEMM shape of
    every dense convolution and fully-connected layer of the case - M = N*OH*OW pixels, K = C*R*S, N = output channels,
    operands already laid out (no patch gathering, no requantisation, no residual add, an int32 result) - summed over
    the layers, beside the sum of this build's launches that do the whole of that work.  A yardstick for what the
    matrix pipes deliver on these shapes, not a code path of the library."""
    import numpy as np
    import torch
    shapes = []
    for n in case.nodes:
        y, x = case.tensors[n.output], case.tensors[n.inputs[0]]
        if n.kind == "conv" and n.attrs["group"] == 1:
            shapes.append((int(np.prod(y.shape)) // y.shape[1], x.shape[1] * n.attrs["k"] ** 2, y.shape[1]))
        elif n.kind == "ip":
            shapes.append((y.shape[0], int(np.prod(x.shape[1:])), y.shape[1]))
    times, skipped = {}, 0
    for s in set(shapes):
        M, K, N = s
        K8 = (K + 7) // 8 * 8          # the library wants multiples of 8: the stem's 147 is padded with zeros
        if M <= 16 or N % 8:
            continue
        a = torch.randint(-128, 128, (M, K8), dtype=torch.int8, device="cuda")
        b = torch.randint(-128, 128, (N, K8), dtype=torch.int8, device="cuda").t()   # k contiguous, as the packed weights
        try:
            for _ in range(2):
                torch._int_mm(a, b)
            torch.cuda.synchronize()
            g = torch.cuda.CUDAGraph()
            with torch.cuda.graph(g):
                for _ in range(10):
                    torch._int_mm(a, b)
            g.replay()
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record()
            g.replay()
            e1.record()
            torch.cuda.synchronize()
            times[s] = e0.elapsed_time(e1) / 10
        except RuntimeError:
            pass
        del a, b
    done = [s for s in shapes if s in times]
    skipped = len(shapes) - len(done)
    lib_ms = sum(times[s] for s in done)
    ops = sum(2.0 * s[0] * s[1] * s[2] for s in done)
    ours_ms = sum(t for s, t in zip(ex.steps, kt) if s["kernel"].startswith("conv_mfma") and s["ops"])
    ours_ops = sum(s["ops"] for s in ex.steps if s["kernel"].startswith("conv_mfma") and s["ops"])
    return {"layers": len(done), "layers_skipped": skipped, "library_ms": round(lib_ms, 4),
            "library_TOPs": round(ops / (lib_ms * 1e-3) / 1e12, 1) if lib_ms else None,
            "this_build_ms": round(ours_ms, 4),
            "this_build_TOPs": round(ours_ops / (ours_ms * 1e-3) / 1e12, 1) if ours_ms else None,
            "note": "library: torch._int_mm per layer shape, int32 output, no im2col / requantisation / add / pooling; "
                    "this build: its convolution-family launches, which include all of those"}


def module_path(build, batch, steps):
    """The drop-in path: the network as an engine file, run by nart_promark (the counterpart of the reference's
    tools/promark.cpp) on the `hip` workspace through hip_module_tp, every operator launched by the module's run
    functions.  A child process: this process keeps its GPU context and never replaces itself."""
    from nart_amd import engine
    exe = os.path.join(ROOT, "nart_amd", "lib", "nart_promark")
    if not os.path.exists(exe):
        return {"error": "nart_amd/lib/nart_promark has not been built"}
    case = build(1)  # the file carries batch 1; -b reshapes it, as a NART user would
    with tempfile.TemporaryDirectory() as d:
        fp = os.path.join(d, "engine.bin")
        with open(fp, "wb") as f:
            f.write(engine.write_engine(case))
        with open(fp + ".json", "w") as f:
            json.dump({"workspaces": {"hip": {}}, "input_workspace": "hip"}, f)
        cmd = [exe, "-m", fp, "-c", fp + ".json", "-b", str(batch), "-n", str(steps)]
        p = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.PIPE, text=True, timeout=300)
    m = re.search(r"average cost: ([0-9.eE+-]+)ms", p.stdout)
    if p.returncode != 0 or not m:
        return {"error": "nart_promark exit %d: %s" % (p.returncode, (p.stderr or p.stdout)[-300:])}
    ms = float(m.group(1))
    return {"runner": "nart_promark -b %d -n %d (engine.bin on the hip workspace through hip_module_tp, eager launches, no host copies)" % (batch, steps),
            "ms_per_batch": round(ms, 4), "value": round(batch / (ms * 1e-3), 1)}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--batch", type=int, default=None,
                    help="images per step (fc: rows M); default 64, for --workload fc 128 (BASELINE configs[1])")
    ap.add_argument("--workload", default="resnet50", choices=["resnet50", "resnet18", "mobilenetv2", "conv", "fc"])
    ap.add_argument("--kernel-reps", type=int, default=10)
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--no-graph", action="store_true", help="launch eagerly instead of replaying a HIP graph")
    ap.add_argument("--no-fuse", action="store_true", help="run every residual add as its own kernel")
    ap.add_argument("--no-branches", action="store_true",
                    help="skip the extra measurements of the pass as two half-batch branches / two batches in flight")
    ap.add_argument("--no-extras", action="store_true",
                    help="skip sustained, module_path and other_workloads (profiling runs want the headline kernels only)")
    ap.add_argument("--layers", action="store_true", help="print a per-layer table (markdown rows) to stderr")
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
    x = random_input(case)
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
    # a pass of one or two kernels is shorter than a graph launch: such workloads replay `inner` passes per graph
    inner = 1 if (len(ex.steps) > 8 or args.no_graph) else 20
    if args.no_graph:
        step = ex.run
    else:
        ex.capture(passes=inner)
        step = ex.replay
    ms, wall_ms = time_steps(step, args.steps, args.warmup)
    ms, wall_ms = ms / inner, wall_ms / inner

    # ---- per-kernel durations and the roofline of the dominant kernel ------------------------------------
    kt = per_kernel_times(ex, args.kernel_reps)
    fam = families_of(ex, kt)
    roof = roofline_of(fam, kt)
    default_flags = not (args.tune or args.no_graph or args.no_fuse)
    add_in_pass(roof, ms)
    if (default_flags and args.workload == TRAFFIC_FROM_PROFILE["workload"] and args.batch == TRAFFIC_FROM_PROFILE["batch"]
            and roof["kernel"] == "conv_mfma_i8"):
        digest = kernel_sources_digest()
        roof["kernel_sources_sha256"] = digest
        if digest == TRAFFIC_FROM_PROFILE["sources_sha256"]:
            roof["traffic"] = TRAFFIC_FROM_PROFILE["bytes_per_launch"]
            roof["traffic_source"] = (TRAFFIC_FROM_PROFILE["source"]
                                      + " (rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE of this command, copy-kernel calibrated)")
        else:
            roof["traffic_source"] = ("null: the kernel sources changed since %s was taken (digest %s there)"
                                      % (TRAFFIC_FROM_PROFILE["source"], TRAFFIC_FROM_PROFILE["sources_sha256"]))
    families = {k: {"ms": round(v["ms"], 4), "launches": v["launches"],
                    "TOPs": round(v["ops"] / (v["ms"] * 1e-3) / 1e12, 2) if v["ops"] else None,
                    "GBs": round(v["bytes"] / (v["ms"] * 1e-3) / 1e9, 1)} for k, v in fam.items()}
    if args.layers:
        print("| layer | kernel | output | us | GOP | MB (compulsory) | binding roof, us | of that roof |", file=sys.stderr)
        print("|---|---|---|---|---|---|---|---|", file=sys.stderr)
        for s, t in zip(ex.steps, kt):
            shape = case.tensors[s["label"]].shape
            t_mfma = s["ops"] / (PEAK_INT8_TOPS * 1e12) * 1e6
            t_hbm = s["bytes"] / (PEAK_HBM_GBS * 1e9) * 1e6
            roof_us = max(t_mfma, t_hbm)
            print("| %s | %s | %s | %.1f | %.3f | %.2f | %s %.1f | %.0f %% |" % (
                s["label"], s["kernel"], "x".join(map(str, shape)), t * 1e3, s["ops"] / 1e9, s["bytes"] / 1e6,
                "mfma" if t_mfma >= t_hbm else "hbm", roof_us, 100.0 * roof_us / (t * 1e3)), file=sys.stderr)

    value = args.batch / (ms * 1e-3)
    res = {"metric": "ResNet-50-int8 images/sec @bs64; int8 conv TOPS (% of MFMA i8 peak)" if args.workload == "resnet50"
           else "%s %s/sec" % (args.workload, "rows" if args.workload == "fc" else "images"),
           "value": round(value, 1), "unit": "rows/s" if args.workload == "fc" else "images/s", "n_gpus": 1,
           "steps": args.steps, "warmup": args.warmup,
           "ms_per_step": round(ms, 5), "wall_ms_per_step": round(wall_ms, 5), "higher_is_better": True,
           "scaling": "weak", "vs_baseline": None, "dtype": "u8", "data": "synthetic",
           "config": {"workload": case.name, "batch": args.batch, "input": list(case.input.shape),
                      "operators": len(case.nodes), "graph_replay": not args.no_graph, "passes_per_graph": inner,
                      "tuned": bool(args.tune), "fused_residual_adds": len(ex.fused), "whole_blocks": len(ex.blocks),
                      "block_tails": len(ex.tails), "dual_shortcut_adds": len(ex.duals), "launches_per_step": len(ex.steps),
                      "conv_fc_gop_per_step": round(case.conv_ops() / 1e9, 2)},
           "conv_tops_whole_step": round(case.conv_ops() / (ms * 1e-3) / 1e12, 2),
           "roofline": roof, "kernel_families": families}

    # Everything below is reported beside the headline and never decides whether the line is printed: a failure is
    # recorded in the line instead.
    def extra(key, fn):
        try:
            res[key] = fn()
        except Exception as e:  # noqa: BLE001
            res[key] = {"error": repr(e)}

    if not args.no_extras and not args.no_graph:
        def sustained():
            n, t0 = 0, time.perf_counter()
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record()
            while time.perf_counter() - t0 < 2.0:
                for _ in range(100):
                    step()
                n += 100
                torch.cuda.current_stream().synchronize()
            e1.record()
            torch.cuda.synchronize()
            sms = e0.elapsed_time(e1) / (n * inner)
            return {"seconds": round(time.perf_counter() - t0, 2), "steps": n * inner, "ms_per_step": round(sms, 5),
                    "value": round(args.batch / (sms * 1e-3), 1)}
        extra("sustained", sustained)

    if not args.no_branches and not args.no_graph and len(ex.steps) > 8:
        def two_branch():
            from nart_amd.runner import BranchedExecutor
            out_t = ex.buf[case.output.name]
            whole = out_t.clone()
            br = BranchedExecutor(ex, build, 2)
            out_t.zero_()
            br.capture()
            bms, _ = time_steps(br.replay, min(args.steps, 50), 5)
            return {"branches": 2, "ms_per_step": round(bms, 4), "value": round(args.batch / (bms * 1e-3), 1),
                    "output_equals_single_branch": bool(torch.equal(out_t, whole))}

        def in_flight():
            # a second copy of the network (own tensors, graph and stream) takes every other step and nothing joins
            # the two chains until the end of the timed region; reported beside `value`, never as `value`
            from nart_amd.runner import PipelinedExecutor
            pipe = PipelinedExecutor(lambda: build(args.batch), depth=2, fuse_add=not args.no_fuse, first=ex)
            pipe.execs[1].set_input(x)
            torch.cuda.synchronize()
            for _ in range(10):
                pipe.submit()
            pipe.wait()
            n = min(args.steps, 50)
            t0 = time.perf_counter()
            for _ in range(n):
                pipe.submit()
            pipe.wait()
            pms = (time.perf_counter() - t0) * 1e3 / n
            same = torch.equal(pipe.execs[1].buf[case.output.name], ex.buf[case.output.name])
            return {"batches_in_flight": 2, "ms_per_step": round(pms, 4), "value": round(args.batch / (pms * 1e-3), 1),
                    "conv_tops_whole_step": round(case.conv_ops() / (pms * 1e-3) / 1e12, 2),
                    "timer": "host clock around the K submissions and the final synchronisation",
                    "outputs_equal_single_stream": bool(same)}
        if args.batch >= 2:
            extra("two_branch_graph", two_branch)
        extra("two_batches_in_flight", in_flight)

    if not args.no_extras and not args.no_graph:
        extra("library_int8_gemm", lambda: library_gemm(case, ex, kt))

    if not args.no_extras and args.workload == "resnet50":
        extra("module_path", lambda: module_path(build, args.batch, 50))
        others = {}
        for key, bld, b, inner_w, rows in (
                ("conv_cfg0_n1", builders["conv"], 1, 20, (0,)),
                ("conv_cfg0_n64", builders["conv"], 64, 20, (0, 63)),
                ("fc_cfg1_m128", builders["fc"], 128, 20, (0, 127)),
                ("resnet18_cfg2_n1", builders["resnet18"], 1, 1, (0,)),
                ("resnet18_cfg2_n32", builders["resnet18"], 32, 1, (0, 31)),
                ("mobilenetv2_cfg3_n64", builders["mobilenetv2"], 64, 1, (0,))):
            try:
                others[key] = measure_workload(bld, b, inner_w, args.kernel_reps, rows)
            except Exception as e:  # noqa: BLE001
                others[key] = {"error": repr(e)}
        res["other_workloads"] = others

    if not args.no_cpu:
        i0 = {"x": x[:1], "y": y[:1]}
        extra("cpu_baseline", lambda: cpu_baseline(build, i0))
    print(json.dumps(res))


if __name__ == "__main__":
    main()
