"""Runs a Case (nart_amd/cases.py) on the GPU through the hipq C ABI.

This is the Python-side counterpart of the reference's parade: a flat list of prepared operators that
`run()` launches in order on the current HIP stream (art/src/parade.c:184-197).  `capture()` records one
pass into a HIP graph so that a launch-bound step replays without per-kernel host overhead.
All device tensors are channels-last with padded channel stride (see include/hipq.h).
"""
import numpy as np
import torch

from . import hipq


class HipqExecutor:
    """fuse_add: a convolution whose only consumer is a two-input add is launched with the add fused into its
    epilogue (hipq_conv2d_run_add); the convolution's own output tensor is then never materialised."""

    def __init__(self, case, fuse_add=False):
        self.case = case
        self.fused = {}      # conv output name -> the add node that absorbs it
        if fuse_add:
            uses = {}
            for node in case.nodes:
                for i in node.inputs:
                    uses.setdefault(i, []).append(node)
            for node in case.nodes:
                u = uses.get(node.output, [])
                if (node.kind == "conv" and node.attrs["group"] == 1 and not node.attrs["relu"] and len(u) == 1
                        and u[0].kind == "add" and u[0].inputs[0] != u[0].inputs[1] and node.output != case.output.name
                        and not any(a is u[0] for a in self.fused.values())):  # one convolution per add
                    self.fused[node.output] = u[0]  # launched at the add's position: both operands exist by then
        self._pending = {}   # id(add node) -> the deferred convolution
        self.buf = {}        # tensor name -> device tensor
        self.steps = []      # (label, kernel name, callable, algorithmic ops, compulsory bytes)
        self.plans = []
        self.graph = None
        T = case.tensors
        inp = case.input
        if inp.dtype == "f32":
            self.buf[inp.name] = torch.zeros(inp.shape, dtype=torch.float32, device="cuda")
        else:
            N, C, H, W = inp.shape
            self.buf[inp.name] = torch.zeros((N, H, W, hipq.channel_stride(C)), dtype=torch.uint8, device="cuda")
        for node in case.nodes:
            y = T[node.output]
            xs = [T[i] for i in node.inputs]
            N, C, H, W = y.shape
            if y.dtype == "f32":
                out = torch.zeros(y.shape, dtype=torch.float32, device="cuda")
            else:
                out = torch.zeros((N, H, W, hipq.channel_stride(C)), dtype=torch.uint8, device="cuda")
            self.buf[y.name] = out
            ins = [self.buf.get(i) for i in node.inputs]
            a = node.attrs
            if node.kind == "quantize":
                fn = (lambda i=ins[0], o=out, y=y: hipq.quantize_u8(i, o, y.alpha, y.zp))
                self._add(node, "quantize_u8_kernel", fn, 0, 5 * int(np.prod(y.shape)))
            elif node.kind == "dequantize":
                x = xs[0]
                fn = (lambda i=ins[0], o=out, x=x: hipq.dequantize_u8(i, o, x.alpha, x.zp))
                self._add(node, "dequantize_u8_kernel", fn, 0, 5 * int(np.prod(y.shape)))
            elif node.kind == "conv":
                x = xs[0]
                plan = hipq.Conv2d(x.shape, case.weights[a["w"]], case.weights[a["b"]], a["pad"], a["stride"],
                                   a["group"], x.alpha, x.zp, a["walpha"], a["wzp"], y.alpha, y.zp, relu=a["relu"])
                self.plans.append(plan)
                nbytes = int(np.prod(x.shape)) + int(np.prod(y.shape)) + case.weights[a["w"]].size + 4 * a["K"]
                if node.output in self.fused and plan.kernel.startswith("conv_mfma"):
                    add = self.fused[node.output]
                    other = [i for i in add.inputs if i != node.output][0]
                    res_first = add.inputs[0] == other
                    ot, st = T[other], T[add.output]
                    self._pending[id(add)] = (plan, ins[0], other, res_first, ot, st, nbytes + int(np.prod(y.shape)))
                    del self.buf[y.name]  # never materialised
                    continue
                self.fused.pop(node.output, None)
                fn = (lambda p=plan, i=ins[0], o=out: p(i, o))
                self._add(node, plan.kernel, fn, plan.ops, nbytes)
                self.steps[-1]["plan"] = plan
            elif node.kind == "ip":
                x = xs[0]
                Nn, Cc, Hh, Ww = x.shape
                w = np.ascontiguousarray(case.weights[a["w"]])
                cs = hipq.channel_stride(Cc)
                if Hh * Ww > 1 or cs != Cc:
                    w2 = np.empty((a["K"], Hh * Ww * cs), np.uint8)
                    hipq.check(hipq.lib().hipq_ip_reorder_weights(w.ctypes.data, w2.ctypes.data, a["K"], Cc, Hh, Ww, cs,
                                                                  a["wzp"]))
                    w = w2
                kd = Hh * Ww * cs
                plan = hipq.Conv2d((Nn, kd, 1, 1), w.reshape(a["K"], kd, 1, 1), case.weights[a["b"]], 0, 1, 1, x.alpha,
                                   x.zp, a["walpha"], a["wzp"], y.alpha, y.zp, in_cs=kd)
                self.plans.append(plan)
                fn = (lambda p=plan, i=ins[0], o=out: p(i, o))
                self._add(node, plan.kernel, fn, 2 * Nn * a["K"] * Cc * Hh * Ww,
                          Nn * Cc * Hh * Ww + Nn * a["K"] + a["K"] * Cc * Hh * Ww + 4 * a["K"])
            elif node.kind == "pool":
                x = xs[0]
                fn = (lambda i=ins[0], o=out, x=x, y=y, a=a: hipq.pool_u8(i, o, x.shape[1], a["k"], a["pad"], a["stride"],
                                                                         a["method"], x.alpha, x.zp, y.alpha, y.zp))
                self._add(node, "pool_u8_kernel", fn, 0, int(np.prod(x.shape)) + int(np.prod(y.shape)))
            elif node.kind == "add" and id(node) in self._pending:
                plan, xin, other, res_first, ot, st, nbytes = self._pending.pop(id(node))
                fn = (lambda p=plan, i=xin, r=self.buf[other], rf=res_first, ot=ot, st=st, o=out:
                      p.run_add(i, r, rf, ot.alpha, ot.zp, st.alpha, st.zp, o))
                self.steps.append({"label": node.output, "kind": "conv+add", "kernel": plan.kernel + "+add", "fn": fn,
                                   "ops": plan.ops, "bytes": nbytes, "plan": plan})
            elif node.kind == "add":
                fn = (lambda i=ins, o=out, xs=xs, y=y: hipq.add_u8(i[0], i[1], o, xs[0].alpha, xs[0].zp, xs[1].alpha,
                                                                 xs[1].zp, y.alpha, y.zp))
                self._add(node, "add_u8_kernel", fn, 0, 3 * int(np.prod(y.shape)))
            else:
                raise ValueError("unknown node kind " + node.kind)

    def _add(self, node, kernel, fn, ops, nbytes):
        self.steps.append({"label": node.output, "kind": node.kind, "kernel": kernel, "fn": fn, "ops": ops,
                           "bytes": nbytes})

    # ---- data in / out ---------------------------------------------------------------------------
    def set_input(self, x):
        inp = self.case.input
        if inp.dtype == "f32":
            self.buf[inp.name].copy_(torch.from_numpy(np.ascontiguousarray(x, np.float32)))
        else:
            self.buf[inp.name].copy_(hipq.to_device_nhwc(x))

    def fetch(self, name):
        t = self.case.tensors[name]
        if t.dtype == "f32":
            return self.buf[name].cpu().numpy()
        return hipq.from_device_nhwc(self.buf[name], t.shape[1])

    def output(self):
        return self.fetch(self.case.output.name)

    # ---- execution -------------------------------------------------------------------------------
    def run(self):
        for s in self.steps:
            s["fn"]()

    # ---- tuning ----------------------------------------------------------------------------------
    TILES = (0, 2, 3, 4)   # 128x128, 128x64, 64x128, 64x64 (include/hipq.h: hipq_conv2d_plan_select)
    STAGES = (2, 3, 4)

    def _time_window(self, lo, hi, reps):
        """Replays steps[lo:hi] from a HIP graph `reps` times; returns microseconds per replay."""
        torch.cuda.synchronize()
        g = torch.cuda.CUDAGraph()
        with torch.cuda.graph(g):
            for s in self.steps[lo:hi]:
                s["fn"]()
        for _ in range(3):
            g.replay()
        torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(reps):
            g.replay()
        e1.record()
        torch.cuda.synchronize()
        return e0.elapsed_time(e1) / reps * 1e3

    def tune(self, reps=20, before=2, after=1, verbose=False):
        """Per-layer search over the MFMA convolution's tile shapes and load stages, timed inside the network: each
        candidate is measured as part of a replayed window of its neighbouring operators, because a kernel timed
        alone on warm inputs ranks the variants differently from the same kernel between its producer and its
        consumer.  Every variant computes the same bytes; only the launch shape changes."""
        self.run()
        torch.cuda.synchronize()
        chosen = {}
        for k, s in enumerate(self.steps):
            plan = s.get("plan")
            if plan is None or not plan.kernel.startswith("conv_mfma") or "_c4" in plan.kernel or "_wzp" in plan.kernel:
                continue
            if plan.desc.in_cs % 64 and not (plan.desc.R == 1 and plan.desc.S == 1):
                continue  # the generic-addressing kernel has a single variant
            if plan.kernel.endswith("pointwise") and s["kind"] != "conv+add":
                continue  # the pointwise kernel has no tile or stages (the fused add runs a tile kernel)
            lo, hi = max(0, k - before), min(len(self.steps), k + 1 + after)
            base = self._time_window(lo, hi, reps)
            best, best_t = (-1, 0), base
            for tile in self.TILES:
                for st in self.STAGES:
                    plan.select(tile, st)
                    t = min(self._time_window(lo, hi, reps) for _ in range(2))
                    if t < best_t * 0.985:  # only move for a clear win
                        best, best_t = (tile, st), t
            if best[0] >= 0:
                plan.select(*best)
            else:  # back to the built-in choice
                plan.select(plan._tile0, 0)
            s["kernel"] = plan.kernel + ("+add" if s["kind"] == "conv+add" else "")
            chosen[s["label"]] = (best, round(base, 2), round(best_t, 2))
            if verbose:
                print("tune %-12s %-28s window %.1f -> %.1f us  choice %s" % (s["label"], plan.kernel, base, best_t, best), flush=True)
        return chosen

    def capture(self):
        """Record one pass into a HIP graph (kernel nodes only: no memsets, no allocations)."""
        self.run()
        torch.cuda.synchronize()
        g = torch.cuda.CUDAGraph()
        with torch.cuda.graph(g):
            self.run()
        self.graph = g
        return g

    def replay(self):
        self.graph.replay()
