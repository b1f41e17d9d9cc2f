"""Runs a Case (nart_amd/cases.py) on the GPU through the hipq C ABI.

This is the Python-side counterpart of the reference's parade: a flat list of prepared operators that
`run()` launches in order on the current HIP stream (art/src/parade.c:184-197).  `capture()` records one
pass into a HIP graph so that a launch-bound step replays without per-kernel host overhead.
All device tensors are channels-last with padded channel stride (see include/hipq.h).
"""
import time

import numpy as np
import torch

from . import hipq


class HipqExecutor:
    """fuse_add: a convolution whose only consumer is a two-input add is launched with the add fused into its
    epilogue (hipq_conv2d_run_add); the convolution's own output tensor is then never materialised."""

    def __init__(self, case, fuse_add=False, share=None):
        """share = (parent, first): every tensor of this executor is the batch slice [first, first + N) of the
        parent executor's tensor of the same name (the batch is the outermost dimension of both layouts, so the
        slice is contiguous).  The parent runs the same network at a larger batch; nothing is allocated here."""
        self.case = case
        self.share = share
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
        self.pooled = {}     # conv output name -> the max-pooling node computed inside the convolution's kernel
        self.blocks = {}     # id(add node) -> (reduce, mid, widen conv nodes) of an identity bottleneck block run as one kernel
        self.in_block = {}   # id(conv node) -> the add node of its block
        self.tails = {}      # id(add node) -> (mid, widen, next or None): the block from its 3x3 layer on as one kernel
        self.duals = {}      # id(add node) -> (widen, shortcut): both 1x1 convolutions and the add as one kernel
        self.dequantized = {}  # fully-connected output name -> the dequantize node computed in the layer's epilogue
        self.chained = {}    # add output name -> the 1x1 convolution node computed inside the fused add's kernel
        self._early = {}     # id(conv node) -> its plan, created ahead of its turn (when an add looked at it)
        self._pending = {}   # id(add node) -> the deferred convolution
        self.buf = {}        # tensor name -> device tensor
        self.steps = []      # (label, kernel name, callable, algorithmic ops, compulsory bytes)
        self.plans = []
        self.graph = None
        T = case.tensors
        inp = case.input
        self.buf[inp.name] = self._tensor(inp)
        def conv_plan(node):
            a, x, y = node.attrs, T[node.inputs[0]], T[node.output]
            plan = self._early.pop(id(node), None)
            if plan is None:
                plan = hipq.Conv2d(x.shape, case.weights[a["w"]], case.weights[a["b"]], a["pad"], a["stride"],
                                   a["group"], x.alpha, x.zp, a["walpha"], a["wzp"], y.alpha, y.zp, relu=a["relu"])
            nbytes = int(np.prod(x.shape)) + int(np.prod(y.shape)) + case.weights[a["w"]].size + 4 * a["K"]
            return plan, nbytes

        if fuse_add:
            self._find_blocks(conv_plan)
        done = set()  # nodes computed inside an earlier node's kernel
        for node in case.nodes:
            if id(node) in done:
                continue
            y = T[node.output]
            xs = [T[i] for i in node.inputs]
            N, C, H, W = y.shape
            out = self._tensor(y)
            self.buf[y.name] = out
            ins = [self.buf.get(i) for i in node.inputs]
            a = node.attrs
            if node.kind == "quantize":
                fn = (lambda i=ins[0], o=out, y=y: hipq.quantize_u8(i, o, y.alpha, y.zp))
                self._add(node, "quantize_u8_kernel", fn, 0, 5 * int(np.prod(y.shape)))
            elif node.kind == "dequantize" and id(node) in self._pending:
                plan, xin, ops, nbytes, xname = self._pending.pop(id(node))
                fn = (lambda p=plan, i=xin, o=out: p.run_dequant(i, o))
                self.steps.append({"label": node.output, "kind": "ip+dequantize", "kernel": plan.kernel + "+dequantize", "fn": fn,
                                   "ops": ops, "bytes": nbytes, "plan": plan})
            elif node.kind == "dequantize":
                x = xs[0]
                fn = (lambda i=ins[0], o=out, x=x: hipq.dequantize_u8(i, o, x.alpha, x.zp))
                self._add(node, "dequantize_u8_kernel", fn, 0, 5 * int(np.prod(y.shape)))
            elif node.kind == "conv" and id(node) in self.in_block:
                self.buf.pop(y.name, None)  # computed inside the block's kernel, never materialised
                continue
            elif node.kind == "add" and id(node) in self.blocks:
                c1, c2, c3 = self.blocks[id(node)]
                plans = [self._early.pop(id(c)) for c in (c1, c2, c3)]
                self.plans += plans
                xin = self.buf[c1.inputs[0]]
                res_first = node.inputs[0] == c1.inputs[0]
                nb = 2 * int(np.prod(y.shape)) + sum(case.weights[c.attrs["w"]].size + 4 * c.attrs["K"] for c in (c1, c2, c3))
                # the 1x1 convolution that reads the sum (the first layer of the next stage) in the same kernel
                nxt = None
                for nd in case.nodes:
                    na = nd.attrs
                    if (nd.kind == "conv" and nd.inputs[0] == node.output and na["k"] == 1 and na["stride"] == 1
                            and na["pad"] == 0 and na["group"] == 1 and nd.output != case.output.name
                            and id(nd) not in self.in_block and nd.output not in self.fused):
                        p2, nb2 = conv_plan(nd)
                        if hipq.bottleneck_conv_fusable(plans[0], plans[1], plans[2], res_first, y.alpha, y.zp, p2):
                            nxt = (nd, p2, nb2)
                            break
                        self._early[id(nd)] = p2
                if nxt is not None:
                    nd, p2, nb2 = nxt
                    y2 = self._tensor(T[nd.output])
                    if y2 is None:
                        raise RuntimeError("shared executor: %s is fused away in the parent but not here" % nd.output)
                    self.buf[nd.output] = y2
                    self.plans.append(p2)
                    self.chained[node.output] = nd
                    done.add(id(nd))
                    fn = (lambda ps=plans, i=xin, rf=res_first, y=y, o=out, p2=p2, y2=y2:
                          hipq.bottleneck_run_conv(ps[0], ps[1], ps[2], i, rf, y.alpha, y.zp, o, p2, y2))
                    self.steps.append({"label": node.output, "kind": "block+conv", "kernel": "conv_mfma_i8_bottleneck+conv", "fn": fn,
                                       "ops": sum(p.ops for p in plans) + p2.ops, "bytes": nb + nb2 - int(np.prod(y.shape)),
                                       "plan": plans[0]})
                    continue
                fn = (lambda ps=plans, i=xin, rf=res_first, y=y, o=out: hipq.bottleneck_run(ps[0], ps[1], ps[2], i, rf, y.alpha, y.zp, o))
                self.steps.append({"label": node.output, "kind": "block", "kernel": "conv_mfma_i8_bottleneck", "fn": fn,
                                   "ops": sum(p.ops for p in plans), "bytes": nb, "plan": plans[0]})
            elif node.kind == "add" and id(node) in self.duals:
                cm, cs = self.duals[id(node)]
                pm, ps = self._early.pop(id(cm)), self._early.pop(id(cs))
                self.plans += [pm, ps]
                sc_first = node.inputs[0] == cs.output
                fn = (lambda pm=pm, ps=ps, i=self.buf[cm.inputs[0]], j=self.buf[cs.inputs[0]], sf=sc_first, y=y, o=out:
                      hipq.run_add2(pm, i, ps, j, sf, y.alpha, y.zp, o))
                nb = (int(np.prod(T[cm.inputs[0]].shape)) + int(np.prod(T[cs.inputs[0]].shape)) + int(np.prod(y.shape))
                      + sum(case.weights[c.attrs["w"]].size + 4 * c.attrs["K"] for c in (cm, cs)))
                self.steps.append({"label": node.output, "kind": "conv+conv+add", "kernel": "conv_mfma_i8_wreg_dual+add", "fn": fn,
                                   "ops": pm.ops + ps.ops, "bytes": nb, "plan": pm})
            elif node.kind == "add" and id(node) in self.tails:
                c2, c3, nxt = self.tails[id(node)]
                convs = [c for c in (c2, c3, nxt) if c is not None]
                plans = [self._early.pop(id(c)) for c in convs]
                self.plans += plans
                other = [i for i in node.inputs if i != c3.output][0]
                res_first = node.inputs[0] == other
                ot = T[other]
                y2 = None
                if nxt is not None:
                    y2 = self._tensor(T[nxt.output])
                    if y2 is None:
                        raise RuntimeError("shared executor: %s is fused away in the parent but not here" % nxt.output)
                    self.buf[nxt.output] = y2
                    self.chained[node.output] = nxt
                    done.add(id(nxt))
                fn = (lambda ps=plans, i=self.buf[c2.inputs[0]], r=self.buf[other], rf=res_first, ot=ot, y=y, o=out, y2=y2:
                      hipq.bottleneck_tail_run(ps[0], ps[1], i, r, rf, ot.alpha, ot.zp, y.alpha, y.zp, o,
                                               ps[2] if len(ps) > 2 else None, y2))
                nb = (int(np.prod(T[c2.inputs[0]].shape)) + 2 * int(np.prod(y.shape)) + (int(np.prod(T[nxt.output].shape)) if nxt else 0)
                      + sum(case.weights[c.attrs["w"]].size + 4 * c.attrs["K"] for c in convs))
                self.steps.append({"label": node.output, "kind": "block tail", "kernel": "conv_mfma_i8_bottleneck_tail" + ("+conv" if nxt else ""),
                                   "fn": fn, "ops": sum(p.ops for p in plans), "bytes": nb, "plan": plans[0]})
            elif node.kind == "conv":
                x = xs[0]
                plan, nbytes = conv_plan(node)
                self.plans.append(plan)
                u = [nd for nd in case.nodes if node.output in nd.inputs]
                if (fuse_add and len(u) == 1 and u[0].kind == "pool" and u[0].attrs["method"] == 0
                        and node.output != case.output.name):
                    # the stem: a 3x3 / stride 2 / pad 1 max pooling with the convolution's own scale runs inside the
                    # convolution's kernel (hipq_conv2d_run_maxpool); the convolution's output is never materialised
                    pa, pt = u[0].attrs, T[u[0].output]
                    if plan.maxpool_fusable(pt.shape[2], pt.shape[3], pa["k"], pa["stride"], pa["pad"], y.alpha, y.zp,
                                            pt.alpha, pt.zp):
                        self.pooled[node.output] = u[0]
                        self._pending[id(u[0])] = (plan, ins[0], nbytes - int(np.prod(y.shape)) + int(np.prod(pt.shape)))
                        self.buf.pop(y.name, None)
                        continue
                if node.output in self.fused and plan.kernel.startswith("conv_mfma"):
                    add = self.fused[node.output]
                    other = [i for i in add.inputs if i != node.output][0]
                    res_first = add.inputs[0] == other
                    ot, st = T[other], T[add.output]
                    self._pending[id(add)] = (plan, ins[0], other, res_first, ot, st, nbytes + int(np.prod(y.shape)))
                    self.buf.pop(y.name, None)  # never materialised
                    continue
                self.fused.pop(node.output, None)
                if out is None:
                    raise RuntimeError("shared executor: %s is fused away in the parent but not here" % y.name)
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
                ip_ops = 2 * Nn * a["K"] * Cc * Hh * Ww
                ip_bytes = Nn * Cc * Hh * Ww + Nn * a["K"] + a["K"] * Cc * Hh * Ww + 4 * a["K"]
                u = [nd for nd in case.nodes if node.output in nd.inputs]
                if (fuse_add and len(u) == 1 and u[0].kind == "dequantize" and node.output != case.output.name
                        and plan.dequant_fusable(y.alpha, y.zp)):
                    # the dequantize that reads the layer runs in its epilogue (hipq_conv2d_run_dequant); the bytes are never written
                    self.dequantized[node.output] = u[0]
                    self._pending[id(u[0])] = (plan, ins[0], ip_ops, ip_bytes + 3 * Nn * a["K"], node.inputs[0])
                    self.buf.pop(y.name, None)
                    continue
                fn = (lambda p=plan, i=ins[0], o=out: p(i, o))
                self._add(node, plan.kernel, fn, ip_ops, ip_bytes)
            elif node.kind == "pool" and id(node) in self._pending:
                plan, xin, nbytes = self._pending.pop(id(node))
                # the 1x1 convolutions that read the pooled tensor (the first layer of the first block, its projection
                # shortcut) in the same kernel
                cands = []
                for nd in case.nodes:
                    na = nd.attrs
                    if (nd.kind == "conv" and nd.inputs[0] == node.output and na["k"] == 1 and na["stride"] == 1
                            and na["pad"] == 0 and na["group"] == 1 and nd.output != case.output.name
                            and id(nd) not in self.in_block and nd.output not in self.fused and len(cands) < 2):
                        p2, nb2 = conv_plan(nd)
                        cands.append((nd, p2, nb2))
                OHp, OWp = y.shape[2], y.shape[3]
                nxt = []
                if len(cands) == 2 and plan.maxpool_conv_fusable(OHp, OWp, cands[0][1], cands[1][1]):
                    nxt = cands
                else:
                    for c in cands:
                        if not nxt and plan.maxpool_conv_fusable(OHp, OWp, c[1]):
                            nxt = [c]
                for c in cands:
                    if not any(c is k for k in nxt):
                        self._early[id(c[0])] = c[1]
                if nxt:
                    ys = []
                    for nd, p2, nb2 in nxt:
                        y2 = self._tensor(T[nd.output])
                        if y2 is None:
                            raise RuntimeError("shared executor: %s is fused away in the parent but not here" % nd.output)
                        self.buf[nd.output] = y2
                        self.plans.append(p2)
                        done.add(id(nd))
                        ys.append(y2)
                    self.chained[node.output] = nxt[0][0]
                    p2, pb = nxt[0][1], (nxt[1][1] if len(nxt) == 2 else None)
                    yb = ys[1] if len(nxt) == 2 else None
                    fn = (lambda p=plan, i=xin, o=out, p2=p2, y2=ys[0], pb=pb, yb=yb: p.run_maxpool_conv(i, o, p2, y2, nxt2=pb, y_next2=yb))
                    self.steps.append({"label": node.output, "kind": "conv+pool+conv", "kernel": "conv_mfma_i8_stem+maxpool" + "+conv" * len(nxt),
                                       "fn": fn, "ops": plan.ops + sum(c[1].ops for c in nxt),
                                       "bytes": nbytes + sum(c[2] - int(np.prod(y.shape)) for c in nxt), "plan": plan})
                    continue
                fn = (lambda p=plan, i=xin, o=out: p.run_maxpool(i, o))
                self.steps.append({"label": node.output, "kind": "conv+pool", "kernel": "conv_mfma_i8_stem+maxpool", "fn": fn,
                                   "ops": plan.ops, "bytes": nbytes, "plan": plan})
            elif node.kind == "pool":
                x = xs[0]
                fn = (lambda i=ins[0], o=out, x=x, y=y, a=a: hipq.pool_u8(i, o, x.shape[1], a["k"], a["pad"], a["stride"],
                                                                         a["method"], x.alpha, x.zp, y.alpha, y.zp))
                self._add(node, "pool_u8_kernel", fn, 0, int(np.prod(x.shape)) + int(np.prod(y.shape)))
            elif node.kind == "add" and id(node) in self._pending:
                plan, xin, other, res_first, ot, st, nbytes = self._pending.pop(id(node))
                # the 1x1 convolution that reads the sum (the first layer of the next block) in the same kernel
                nxt = None
                for nd in case.nodes:
                    na = nd.attrs
                    if (nd.kind == "conv" and nd.inputs[0] == node.output and na["k"] == 1 and na["stride"] == 1
                            and na["pad"] == 0 and na["group"] == 1 and nd.output != case.output.name
                            and id(nd) not in self.in_block):
                        p2, nb2 = conv_plan(nd)
                        if plan.add_conv_fusable(res_first, ot.alpha, ot.zp, st.alpha, st.zp, p2):
                            nxt = (nd, p2, nb2)
                            break
                        self._early[id(nd)] = p2
                if nxt is not None:
                    nd, p2, nb2 = nxt
                    y2 = self._tensor(T[nd.output])
                    if y2 is None:
                        raise RuntimeError("shared executor: %s is fused away in the parent but not here" % nd.output)
                    self.buf[nd.output] = y2
                    self.plans.append(p2)
                    self.chained[node.output] = nd
                    done.add(id(nd))
                    fn = (lambda p=plan, i=xin, r=self.buf[other], rf=res_first, ot=ot, st=st, o=out, p2=p2, y2=y2:
                          p.run_add_conv(i, r, rf, ot.alpha, ot.zp, st.alpha, st.zp, o, p2, y2))
                    self.steps.append({"label": node.output, "kind": "conv+add+conv", "kernel": "conv_mfma_i8_expand+add+conv",
                                       "fn": fn, "ops": plan.ops + p2.ops, "bytes": nbytes + nb2 - int(np.prod(st.shape)),
                                       "plan": plan})
                    continue
                fn = (lambda p=plan, i=xin, r=self.buf[other], rf=res_first, ot=ot, st=st, o=out:
                      p.run_add(i, r, rf, ot.alpha, ot.zp, st.alpha, st.zp, o))
                self.steps.append({"label": node.output, "kind": "conv+add", "kernel": plan.kernel_add or plan.kernel + "+add", "fn": fn,
                                   "ops": plan.ops, "bytes": nbytes, "plan": plan})
            elif node.kind == "add":
                fn = (lambda i=ins, o=out, xs=xs, y=y: hipq.add_u8(i[0], i[1], o, xs[0].alpha, xs[0].zp, xs[1].alpha,
                                                                 xs[1].zp, y.alpha, y.zp))
                self._add(node, "add_u8_kernel", fn, 0, 3 * int(np.prod(y.shape)))
            else:
                raise ValueError("unknown node kind " + node.kind)

    def _find_blocks(self, conv_plan):
        """Identity bottleneck blocks - 1x1, 3x3, 1x1 and the add of the last one's output with the first one's input,
        every intermediate tensor read by nobody else - that hipq_bottleneck_run computes in one launch."""
        case = self.case
        T = case.tensors
        prod = {n.output: n for n in case.nodes}
        uses = {}
        for n in case.nodes:
            for i in n.inputs:
                uses.setdefault(i, []).append(n)

        def only_conv(name, k, strides=(1,)):
            n = prod.get(name)
            if (n is None or n.kind != "conv" or n.attrs["k"] != k or n.attrs["stride"] not in strides or n.attrs["group"] != 1
                    or n.attrs["relu"] or len(uses.get(name, [])) != 1 or name == case.output.name):
                return None
            return n
        for add in case.nodes:
            if add.kind != "add" or len(add.inputs) != 2 or add.inputs[0] == add.inputs[1]:
                continue
            for ci in (0, 1):
                c3 = only_conv(add.inputs[ci], 1)
                c2 = only_conv(c3.inputs[0], 3) if c3 else None
                c1 = only_conv(c2.inputs[0], 1) if c2 else None
                if c1 is None or c1.inputs[0] != add.inputs[1 - ci] or any(id(c) in self.in_block for c in (c1, c2, c3)):
                    continue
                if T[c1.inputs[0]].dtype != "u8" or c1.attrs["pad"] != 0 or c3.attrs["pad"] != 0 or c2.attrs["pad"] != 1:
                    continue
                plans = [conv_plan(c)[0] for c in (c1, c2, c3)]
                st = T[add.output]
                if hipq.bottleneck_fusable(plans[0], plans[1], plans[2], ci == 1, st.alpha, st.zp):
                    self.blocks[id(add)] = (c1, c2, c3)
                    for c, p in zip((c1, c2, c3), plans):
                        self.in_block[id(c)] = add
                        self._early[id(c)] = p
                        self.fused.pop(c.output, None)
                    break
                for c, p in zip((c1, c2, c3), plans):
                    self._early.setdefault(id(c), p)  # keep the plans for the operators' own turns
            if id(add) in self.blocks:
                continue
            # a block with a projection shortcut: both inputs of the add are 1x1 convolutions read by nobody else
            pair = [prod.get(i) for i in add.inputs]
            if all(n is not None and n.kind == "conv" and n.attrs["k"] == 1 and n.attrs["group"] == 1 and not n.attrs["relu"]
                   and n.attrs["pad"] == 0 and len(uses.get(n.output, [])) == 1 and n.output != case.output.name
                   and id(n) not in self.in_block for n in pair):
                plans = [conv_plan(n)[0] for n in pair]
                st = T[add.output]
                for mi in (0, 1):
                    if hipq.add2_fusable(plans[mi], plans[1 - mi], mi == 1, st.alpha, st.zp):
                        self.duals[id(add)] = (pair[mi], pair[1 - mi])
                        break
                for n, pl in zip(pair, plans):
                    self._early[id(n)] = pl
                    if id(add) in self.duals:
                        self.in_block[id(n)] = add
                        self.fused.pop(n.output, None)
                if id(add) in self.duals:
                    continue
            # the block from its 3x3 layer on, with any residual, and the 1x1 layer that reads the sum
            for ci in (0, 1):
                c3 = only_conv(add.inputs[ci], 1)
                c2 = only_conv(c3.inputs[0], 3, (1, 2)) if c3 else None
                if c2 is None or any(id(c) in self.in_block for c in (c2, c3)) or c3.attrs["pad"] != 0 or c2.attrs["pad"] != 1:
                    continue
                p2, p3 = conv_plan(c2)[0], conv_plan(c3)[0]
                st, ot = T[add.output], T[add.inputs[1 - ci]]
                nxt, pn = None, None
                for nd in uses.get(add.output, []):
                    na = nd.attrs
                    if (nd.kind == "conv" and na["k"] == 1 and na["stride"] == 1 and na["pad"] == 0 and na["group"] == 1
                            and not na["relu"] and nd.output != case.output.name and id(nd) not in self.in_block
                            and not any(t[2] is nd for t in self.tails.values())):
                        cand = conv_plan(nd)[0]
                        self._early[id(nd)] = cand
                        if hipq.bottleneck_tail_fusable(p2, p3, ci == 1, ot.alpha, ot.zp, st.alpha, st.zp, cand):
                            nxt, pn = nd, cand
                            break
                if nxt is not None or hipq.bottleneck_tail_fusable(p2, p3, ci == 1, ot.alpha, ot.zp, st.alpha, st.zp):
                    self.tails[id(add)] = (c2, c3, nxt)
                    for c, pl in ((c2, p2), (c3, p3)):
                        self.in_block[id(c)] = add
                        self._early[id(c)] = pl
                        self.fused.pop(c.output, None)
                    break
                self._early.setdefault(id(c2), p2)
                self._early.setdefault(id(c3), p3)

    def _tensor(self, t):
        N, C, H, W = t.shape
        if self.share is not None:
            parent, first = self.share
            whole = parent.buf.get(t.name)
            return None if whole is None else whole[first:first + N]  # None: fused away in the parent as well
        if t.dtype == "f32":
            return torch.zeros(t.shape, dtype=torch.float32, device="cuda")
        return torch.zeros((N, H, W, hipq.channel_stride(C)), dtype=torch.uint8, device="cuda")

    def _add(self, node, kernel, fn, ops, nbytes):
        self.steps.append({"label": node.output, "kind": node.kind, "kernel": kernel, "fn": fn, "ops": ops,
                           "bytes": nbytes})

    # ---- data in / out ---------------------------------------------------------------------------
    @property
    def elided(self):
        """Names of the tensors that are never materialised (absorbed into a fused kernel)."""
        return set(self.fused) | set(self.pooled) | set(self.dequantized) | {c.output for cs in self.blocks.values() for c in cs} | {c.output for cs in self.tails.values() for c in cs[:2]} | {c.output for cs in self.duals.values() for c in cs}

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
            if "expand" in s["kernel"] or "_stream_" in s["kernel"]:
                continue  # neither have these two; naming a tile would take the layer away from them for good
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
            s["kernel"] = (plan.kernel_add or plan.kernel + "+add") if s["kind"] == "conv+add" else plan.kernel
            chosen[s["label"]] = (best, round(base, 2), round(best_t, 2))
            if verbose:
                print("tune %-12s %-28s window %.1f -> %.1f us  choice %s" % (s["label"], plan.kernel, base, best_t, best), flush=True)
        return chosen

    def capture(self, passes=1):
        """Record `passes` passes into a HIP graph (kernel nodes only: no memsets, no allocations).  A network of one or
        two kernels is shorter than a graph launch: its callers record several passes per graph."""
        self.run()
        torch.cuda.synchronize()
        g = torch.cuda.CUDAGraph()
        with torch.cuda.graph(g):
            for _ in range(passes):
                self.run()
        self.graph = g
        return g

    def replay(self):
        self.graph.replay()


class BranchedExecutor:
    """One pass over a batch run as `branches` part-batches side by side, each on a stream of its own.

    Every operator of the path treats the images of a batch independently, and the batch is the outermost dimension
    of every device tensor, so a part-batch is a contiguous slice of the whole batch's tensors: the part executors
    share the parent's buffers (HipqExecutor(share=...)) and the parent's input / output stay the interface.
    Two chains of kernels that do not depend on each other let the GPU start one chain's next kernel while the other
    chain's current kernel drains its last work-groups, and the chains drift apart so that kernels bound by
    different units (HBM, LDS, matrix cores) overlap; the arithmetic, and so every output byte, is unchanged.
    The reference has no counterpart: its parade is one sequential op list (art/src/parade.c:184-197)."""

    def __init__(self, parent, build, branches=2):
        N = parent.case.input.shape[0]
        if branches < 2 or N < branches:
            raise ValueError("branches must be between 2 and the batch size")
        self.parent = parent
        bounds = [N * b // branches for b in range(branches + 1)]
        self.parts = [HipqExecutor(build(hi - lo), fuse_add=bool(parent.fused), share=(parent, lo))
                      for lo, hi in zip(bounds[:-1], bounds[1:])]
        for p in self.parts:
            # a part may cut its launches differently (a kernel that serves two operators at the parent's size need not
            # at the part's), but it must materialise exactly the parent's tensors: they are slices of the same buffers
            if p.elided != parent.elided or set(p.buf) != set(parent.buf):
                raise RuntimeError("part-batch executor materialises other tensors than its parent")
        self.side = [torch.cuda.Stream() for _ in self.parts[1:]]  # default priority
        self.graph = None

    def run(self):
        cur = torch.cuda.current_stream()
        for s in self.side:
            s.wait_stream(cur)
        self.parts[0].run()
        for s, p in zip(self.side, self.parts[1:]):
            with torch.cuda.stream(s):
                p.run()
        for s in self.side:
            cur.wait_stream(s)

    def capture(self):
        """One HIP graph with a branch per part-batch (kernel nodes and the fork / join dependencies only)."""
        self.run()
        torch.cuda.synchronize()
        g = torch.cuda.CUDAGraph()
        with torch.cuda.graph(g):
            self.run()
        self.graph = g
        return g

    def replay(self):
        self.graph.replay()


class PipelinedExecutor:
    """`depth` independent copies of one network (own tensors, own HIP graph, own stream each) that take consecutive
    batches in turn, so that `depth` batches are in flight at once: `submit()` replays the next copy's graph and returns
    its executor without waiting; the caller synchronises (`wait()`) before it reads a copy's output or refills its
    input.  One chain of dependent kernels leaves the GPU partly idle while each kernel ramps up and drains; a second,
    unrelated chain fills those gaps, and because the chains are never joined they drift into complementary phases
    (an HBM-bound layer of one batch beside a latency-bound layer of the other).  More than two chains add nothing.
    The reference has no counterpart inside one parade; its equivalent is two parades on two workspaces, which
    nart_promark -p 2 drives the same way through the `hip` module."""

    def __init__(self, build, depth=2, fuse_add=True, first=None):
        if depth < 1:
            raise ValueError("depth must be at least 1")
        self.execs = [first if (k == 0 and first is not None) else HipqExecutor(build(), fuse_add=fuse_add)
                      for k in range(depth)]
        self.turn = 0
        cur = torch.cuda.current_stream()
        for ex in self.execs:
            if ex.graph is None:
                ex.capture()
        # The runtime multiplexes HIP streams over a few hardware queues (4 by default), and two streams that share a
        # queue run their kernels one after the other.  Which queue a new stream gets depends on how many streams the
        # process created before, so with two copies a few candidate partners are timed and the best one is kept.
        cands = [torch.cuda.Stream() for _ in range(depth if depth != 2 else 4)]  # default priority
        for st in cands:
            st.wait_stream(cur)
        self.streams = cands[:depth]
        if depth == 2:
            best = None
            for partner in cands[1:]:
                self.streams = [cands[0], partner]
                self._burst(4)
                t0 = time.perf_counter()
                self._burst(8)
                t = time.perf_counter() - t0
                if best is None or t < best[0]:
                    best = (t, partner)
            self.streams = [cands[0], best[1]]
            self.turn = 0

    def _burst(self, n):
        for _ in range(n):
            self.submit()
        self.wait()

    def submit(self):
        k = self.turn
        self.turn = (k + 1) % len(self.execs)
        with torch.cuda.stream(self.streams[k]):
            self.execs[k].replay()
        return self.execs[k]

    def wait(self):
        for st in self.streams:
            st.synchronize()
