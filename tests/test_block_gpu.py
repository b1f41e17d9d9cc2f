"""GPU parity of hipq_bottleneck_run - an identity bottleneck block (1x1, 3x3, 1x1, residual add) in one launch - against
the CPU oracle's four operators, bit for bit, through the C ABI."""
import math
import sys
import time

import numpy as np
import pytest

pytestmark = pytest.mark.gpu

torch = pytest.importorskip("torch")

from oracle import orc  # noqa: E402  (checker only)
from nart_amd import hipq  # noqa: E402


def make_block(rng, N, CW, H, W, ozps=(0, 0, None)):
    """Seeded tensors and quantisation parameters of one identity block: widths CW -> CW/4 -> CW/4 -> CW."""
    CM = CW // 4
    xa, xz = 0.05, int(rng.integers(0, 256))
    x = rng.integers(0, 256, (N, CW, H, W), dtype=np.uint8)
    layers = []
    ia, iz = xa, xz
    for (K, C, k), oz in zip(((CM, CW, 1), (CM, CM, 3), (CW, CM, 1)), ozps):
        w = rng.integers(1, 256, (K, C, k, k), dtype=np.uint8)
        sigma = 74.0 * 74.0 * math.sqrt(C * k * k)
        b = rng.integers(-int(sigma), int(sigma) + 1, K).astype(np.int32)
        oa = float(np.float32(ia * rng.uniform(0.75, 1.35)))
        wa = float(np.float32(oa * 40.0 / (ia * sigma)))
        oz = int(rng.integers(96, 160)) if oz is None else oz
        layers.append(dict(w=w, b=b, pad=k // 2, q=(ia, iz, wa, 128, oa, oz)))
        ia, iz = oa, oz
    sa = float(np.float32(math.hypot(ia, xa) * 1.1))
    return x, (xa, xz), layers, (sa, int(rng.integers(0, 40)))


def oracle_block(x, xq, layers, sq, res_first):
    t = x
    for L in layers:
        t = orc.conv2d_u8(t, L["w"], L["b"], L["pad"], 1, 1, *L["q"])
    q3 = layers[2]["q"]
    if res_first:
        return orc.add_u8(x, t, xq[0], xq[1], q3[4], q3[5], sq[0], sq[1])
    return orc.add_u8(t, x, q3[4], q3[5], xq[0], xq[1], sq[0], sq[1])


def plans_of(x, layers, stride=1):
    """stride: of the first layer (a 3x3 / pad 1 layer when it is 2)."""
    shape = x.shape
    plans = []
    for L in layers:
        st = stride if not plans else 1
        p = hipq.Conv2d(shape, L["w"], L["b"], L["pad"], st, 1, *L["q"])
        plans.append(p)
        if len(plans) == 1:
            p.special(2)  # the block kernel wherever it applies, not only where the built-in rule uses it
        shape = (shape[0], L["w"].shape[0], (shape[2] - 1) // st + 1, (shape[3] - 1) // st + 1)
    return plans


CASES = [  # N, CW, H, W
    (2, 1024, 14, 14), (1, 512, 28, 28), (1, 256, 28, 35), (3, 1024, 7, 7), (2, 512, 14, 7), (1, 256, 7, 14), (1, 1024, 21, 14),
]


@pytest.mark.parametrize("case", CASES, ids=lambda c: "x".join(map(str, c)))
def test_bottleneck_block(case):
    N, CW, H, W = case
    rng = np.random.default_rng(1000 + CW + H)
    for res_first, ozps in ((False, (0, 0, None)), (True, (7, 200, None))):
        x, xq, layers, sq = make_block(rng, N, CW, H, W, ozps)
        plans = plans_of(x, layers)
        print("block case", case, res_first, [p.kernel for p in plans], flush=True)
        assert hipq.bottleneck_fusable(*plans, res_first, sq[0], sq[1]), hipq.lib().hipq_last_error()
        want = oracle_block(x, xq, layers, sq, res_first)
        xd = hipq.to_device_nhwc(x)
        y = torch.zeros_like(xd)
        hipq.bottleneck_run(*plans, xd, res_first, sq[0], sq[1], y)
        torch.cuda.synchronize()
        got = hipq.from_device_nhwc(y, CW)
        bad = got != want
        assert not bad.any(), (case, res_first, int(bad.sum()), np.argwhere(bad)[:8].tolist())
        # the three existing entry points give the same bytes
        t1 = plans[0](xd)
        t2 = plans[1](t1)
        y2 = torch.zeros_like(xd)
        plans[2].run_add(t2, xd, res_first, xq[0], xq[1], sq[0], sq[1], y2)
        torch.cuda.synchronize()
        assert torch.equal(y, y2)
        # the same with the next stage's first layer (CW -> CW / 2) computed in the kernel as well
        CN = CW // 2
        wn = rng.integers(1, 256, (CN, CW, 1, 1), dtype=np.uint8)
        sigma = 74.0 * 74.0 * math.sqrt(CW)
        bn = rng.integers(-int(sigma), int(sigma) + 1, CN).astype(np.int32)
        oan = float(np.float32(sq[0] * rng.uniform(0.75, 1.35)))
        qn = (sq[0], sq[1], float(np.float32(oan * 40.0 / (sq[0] * sigma))), 128, oan, int(rng.integers(20, 60)))
        pn = hipq.Conv2d((N, CW, H, W), wn, bn, 0, 1, 1, *qn, relu=res_first)
        assert hipq.bottleneck_conv_fusable(*plans, res_first, sq[0], sq[1], pn), hipq.lib().hipq_last_error()
        y3, yn = torch.zeros_like(xd), torch.zeros((N, H, W, CN), dtype=torch.uint8, device="cuda")
        hipq.bottleneck_run_conv(*plans, xd, res_first, sq[0], sq[1], y3, pn, yn)
        torch.cuda.synchronize()
        assert torch.equal(y3, y)
        wantn = orc.conv2d_u8(want, wn, bn, 0, 1, 1, *qn)
        if res_first:
            wantn = np.maximum(wantn, qn[5]).astype(np.uint8)
        gotn = hipq.from_device_nhwc(yn, CN)
        bad = gotn != wantn
        assert not bad.any(), (case, "next layer", int(bad.sum()), np.argwhere(bad)[:8].tolist())
        assert len(np.unique(wantn)) > 8


TAIL_CASES = [  # N, CW, H, W: patches of 8 x 8, 4 x 14 and 7 x 7 pixels; 64, 128 and 256 middle channels
    (1, 256, 16, 24), (2, 512, 8, 28), (2, 256, 14, 21), (1, 1024, 8, 8), (1, 512, 56, 8), (3, 256, 4, 14), (1, 1024, 7, 7),
]


def make_tail(rng, N, CW, H, W, relu_next, wide_next=False, in_hw=None):
    """The block from its 3x3 layer on: t1 [N, CM, H, W] -> 3x3 -> 1x1 to CW -> add(., residual) -> 1x1 back to CM (to
    2 CM with wide_next: the first layer of the next stage).  in_hw: the size of t1 where the 3x3 layer has stride 2 and
    H x W is its output."""
    CM = CW // 4
    CN = 2 * CM if wide_next else CM
    t1 = rng.integers(0, 256, (N, CM) + tuple(in_hw or (H, W)), dtype=np.uint8)
    res = rng.integers(0, 256, (N, CW, H, W), dtype=np.uint8)
    ia, iz = 0.04, int(rng.integers(0, 256))
    layers = []
    for (K, C, k), oz in zip(((CM, CM, 3), (CW, CM, 1)), (int(rng.integers(0, 30)), None)):
        w = rng.integers(1, 256, (K, C, k, k), dtype=np.uint8)
        sigma = 74.0 * 74.0 * math.sqrt(C * k * k)
        b = rng.integers(-int(sigma), int(sigma) + 1, K).astype(np.int32)
        oa = float(np.float32(ia * rng.uniform(0.75, 1.35)))
        wa = float(np.float32(oa * 40.0 / (ia * sigma)))
        oz = int(rng.integers(96, 160)) if oz is None else oz
        layers.append(dict(w=w, b=b, pad=k // 2, q=(ia, iz, wa, 128, oa, oz)))
        ia, iz = oa, oz
    ra, rz = float(np.float32(ia * rng.uniform(0.6, 1.6))), int(rng.integers(0, 256))
    sa, sz = float(np.float32(math.hypot(ia, ra) * 1.1)), int(rng.integers(0, 40))
    w = rng.integers(1, 256, (CN, CW, 1, 1), dtype=np.uint8)
    sigma = 74.0 * 74.0 * math.sqrt(CW)
    b = rng.integers(-int(sigma), int(sigma) + 1, CN).astype(np.int32)
    oa = float(np.float32(sa * rng.uniform(0.75, 1.35)))
    nxt = dict(w=w, b=b, pad=0, q=(sa, sz, float(np.float32(oa * 40.0 / (sa * sigma))), 128, oa, int(rng.integers(20, 60))), relu=relu_next)
    return t1, res, layers, (ra, rz), (sa, sz), nxt


@pytest.mark.parametrize("case", TAIL_CASES, ids=lambda c: "x".join(map(str, c)))
def test_bottleneck_tail(case):
    """hipq_bottleneck_tail_run == 3x3 convolution, widening convolution, add with any residual and - chained - the next
    1x1 convolution run one by one by the oracle: both operand orders of the add, with and without the chained layer, a
    ReLU on the chained layer, a chained layer of twice the channels, every patch shape and channel count."""
    N, CW, H, W = case
    CM = CW // 4
    rng = np.random.default_rng(2000 + CW + H)
    for res_first, chain, relu_next, wide in ((False, True, False, False), (True, True, True, False), (True, False, False, False),
                                              (False, True, True, True)):
        t1, res, layers, rq, sq, nx = make_tail(rng, N, CW, H, W, relu_next, wide)
        plans = plans_of(t1, layers)
        pn = hipq.Conv2d((N, CW, H, W), nx["w"], nx["b"], 0, 1, 1, *nx["q"])
        print("tail case", case, res_first, chain, relu_next, [p.kernel for p in plans], flush=True)
        assert hipq.bottleneck_tail_fusable(plans[0], plans[1], res_first, rq[0], rq[1], sq[0], sq[1], pn if chain else None)
        t = orc.conv2d_u8(t1, layers[0]["w"], layers[0]["b"], 1, 1, 1, *layers[0]["q"])
        c = orc.conv2d_u8(t, layers[1]["w"], layers[1]["b"], 0, 1, 1, *layers[1]["q"])
        q3 = layers[1]["q"]
        want = orc.add_u8(res, c, rq[0], rq[1], q3[4], q3[5], sq[0], sq[1]) if res_first else orc.add_u8(c, res, q3[4], q3[5], rq[0], rq[1], sq[0], sq[1])
        xd, rd = hipq.to_device_nhwc(t1), hipq.to_device_nhwc(res)
        y = torch.zeros_like(rd)
        yn = torch.zeros((N, H, W, nx["w"].shape[0]), dtype=torch.uint8, device="cuda") if chain else None
        hipq.bottleneck_tail_run(plans[0], plans[1], xd, rd, res_first, rq[0], rq[1], sq[0], sq[1], y, pn if chain else None, yn,
                                 next_relu=relu_next)
        torch.cuda.synchronize()
        got = hipq.from_device_nhwc(y, CW)
        bad = got != want
        assert not bad.any(), (case, res_first, chain, int(bad.sum()), np.argwhere(bad)[:8].tolist())
        if chain:
            wantn = orc.conv2d_u8(want, nx["w"], nx["b"], 0, 1, 1, *nx["q"])
            if relu_next:
                wantn = np.maximum(wantn, nx["q"][5]).astype(np.uint8)
            gotn = hipq.from_device_nhwc(yn, nx["w"].shape[0])
            bad = gotn != wantn
            assert not bad.any(), (case, "next layer", relu_next, int(bad.sum()), np.argwhere(bad)[:8].tolist())


@pytest.mark.parametrize("case", [(2, 512, 28, 28, 56, 56), (1, 512, 8, 16, 15, 32), (2, 512, 7, 14, 13, 27), (1, 512, 4, 14, 8, 28)],
                         ids=lambda c: "x".join(map(str, c)))
def test_bottleneck_tail_with_a_strided_3x3_layer(case):
    """The first block of a stage: the 3x3 layer has stride 2 (even and odd input sizes, every patch shape), the residual is
    any tensor of the output's size (the projection shortcut), with and without the chained layer."""
    N, CW, H, W, IH, IW = case
    CM = CW // 4
    rng = np.random.default_rng(2500 + H + IW)
    for res_first, chain, wide in ((False, True, False), (True, False, False), (True, True, True)):
        t1, res, layers, rq, sq, nx = make_tail(rng, N, CW, H, W, False, wide, (IH, IW))
        plans = plans_of(t1, layers, stride=2)
        pn = hipq.Conv2d((N, CW, H, W), nx["w"], nx["b"], 0, 1, 1, *nx["q"])
        print("strided tail case", case, res_first, chain, wide, [p.kernel for p in plans], flush=True)
        assert hipq.bottleneck_tail_fusable(plans[0], plans[1], res_first, rq[0], rq[1], sq[0], sq[1], pn if chain else None)
        t = orc.conv2d_u8(t1, layers[0]["w"], layers[0]["b"], 1, 2, 1, *layers[0]["q"])
        assert t.shape[2:] == (H, W)
        c = orc.conv2d_u8(t, layers[1]["w"], layers[1]["b"], 0, 1, 1, *layers[1]["q"])
        q3 = layers[1]["q"]
        want = orc.add_u8(res, c, rq[0], rq[1], q3[4], q3[5], sq[0], sq[1]) if res_first else orc.add_u8(c, res, q3[4], q3[5], rq[0], rq[1], sq[0], sq[1])
        xd, rd = hipq.to_device_nhwc(t1), hipq.to_device_nhwc(res)
        y = torch.zeros_like(rd)
        yn = torch.zeros((N, H, W, nx["w"].shape[0]), dtype=torch.uint8, device="cuda") if chain else None
        hipq.bottleneck_tail_run(plans[0], plans[1], xd, rd, res_first, rq[0], rq[1], sq[0], sq[1], y, pn if chain else None, yn)
        torch.cuda.synchronize()
        got = hipq.from_device_nhwc(y, CW)
        bad = got != want
        assert not bad.any(), (case, res_first, chain, int(bad.sum()), np.argwhere(bad)[:8].tolist())
        if chain:
            wantn = orc.conv2d_u8(want, nx["w"], nx["b"], 0, 1, 1, *nx["q"])
            gotn = hipq.from_device_nhwc(yn, nx["w"].shape[0])
            bad = gotn != wantn
            assert not bad.any(), (case, "next layer", int(bad.sum()), np.argwhere(bad)[:8].tolist())
    # 64 or 256 middle channels with a strided 3x3 layer go through the separate entry points
    t1, res, layers, rq, sq, nx = make_tail(rng, 1, 256, 8, 8, False, False, (16, 16))
    plans = plans_of(t1, layers, stride=2)
    assert not hipq.bottleneck_tail_fusable(plans[0], plans[1], False, rq[0], rq[1], sq[0], sq[1])


def test_bottleneck_refusals():
    """What the one-launch forms do not serve is refused by the predicates and fails loudly in the run entry points."""
    rng = np.random.default_rng(7)
    x, xq, layers, sq = make_block(rng, 1, 256, 10, 14)  # a height that is no multiple of 7
    plans = plans_of(x, layers)
    assert not hipq.bottleneck_fusable(*plans, False, sq[0], sq[1])
    xd = hipq.to_device_nhwc(x)
    with pytest.raises(hipq.HipqError, match="do not run as one kernel"):
        hipq.bottleneck_run(*plans, xd, False, sq[0], sq[1], torch.zeros_like(xd))
    x, xq, layers, sq = make_block(rng, 1, 256, 14, 14)
    plans = plans_of(x, layers)
    xd = hipq.to_device_nhwc(x)
    with pytest.raises(hipq.HipqError, match="cannot overwrite"):
        hipq.bottleneck_run(*plans, xd, False, sq[0], sq[1], xd)
    assert not hipq.bottleneck_fusable(*plans, False, sq[0], sq[1], obits=7)
    # the tail form: a stride-2 3x3 layer, and a chained layer that reads the sum with another zero point
    t1, res, tl, rq, sq2, nx = make_tail(rng, 1, 256, 16, 16, False)
    p2s = hipq.Conv2d(t1.shape, tl[0]["w"], tl[0]["b"], 1, 2, 1, *tl[0]["q"]).special(2)
    p3 = hipq.Conv2d((1, 64, 8, 8), tl[1]["w"], tl[1]["b"], 0, 1, 1, *tl[1]["q"])
    assert not hipq.bottleneck_tail_fusable(p2s, p3, False, rq[0], rq[1], sq2[0], sq2[1])
    plans = plans_of(t1, tl)
    q = list(nx["q"])
    q[1] = (q[1] + 1) % 256
    pn = hipq.Conv2d((1, 256, 16, 16), nx["w"], nx["b"], 0, 1, 1, *q)
    assert hipq.bottleneck_tail_fusable(plans[0], plans[1], False, rq[0], rq[1], sq2[0], sq2[1])
    assert not hipq.bottleneck_tail_fusable(plans[0], plans[1], False, rq[0], rq[1], sq2[0], sq2[1], pn)
    xd, rd = hipq.to_device_nhwc(t1), hipq.to_device_nhwc(res)
    with pytest.raises(hipq.HipqError, match="do not run as one kernel"):
        hipq.bottleneck_tail_run(plans[0], plans[1], xd, rd, False, rq[0], rq[1], sq2[0], sq2[1], torch.zeros_like(rd), pn, torch.zeros_like(xd))


def time_tail(N, CW, HW, reps=50):
    rng = np.random.default_rng(6)
    t1, res, layers, rq, sq, nx = make_tail(rng, N, CW, HW, HW, False)
    plans = plans_of(t1, layers)
    pn = hipq.Conv2d((N, CW, HW, HW), nx["w"], nx["b"], 0, 1, 1, *nx["q"])
    xd, rd = hipq.to_device_nhwc(t1), hipq.to_device_nhwc(res)
    y, yn, t = torch.zeros_like(rd), torch.zeros_like(xd), torch.zeros_like(xd)
    fusable = plans[1].add_conv_fusable(False, rq[0], rq[1], sq[0], sq[1], pn)

    def fused():
        hipq.bottleneck_tail_run(plans[0], plans[1], xd, rd, False, rq[0], rq[1], sq[0], sq[1], y, pn, yn)

    def separate():
        plans[0](xd, t)
        if fusable:
            plans[1].run_add_conv(t, rd, False, rq[0], rq[1], sq[0], sq[1], y, pn, yn)
        else:
            plans[1].run_add(t, rd, False, rq[0], rq[1], sq[0], sq[1], y)
            pn(y, yn)

    out = {}
    for name, fn in (("fused", fused), ("separate", separate)):
        fn()
        torch.cuda.synchronize()
        g = torch.cuda.CUDAGraph()
        with torch.cuda.graph(g):
            for _ in range(10):
                fn()
        for _ in range(3):
            g.replay()
        torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(reps):
            g.replay()
        e1.record()
        torch.cuda.synchronize()
        out[name] = e0.elapsed_time(e1) / reps / 10 * 1e3
    print("tail N=%d CW=%d %dx%d: fused %.1f us, separate (%s, %s) %.1f us" % (
        N, CW, HW, HW, out["fused"], plans[0].kernel, "expand+add+conv" if fusable else "add, conv", out["separate"]), flush=True)


WREG_CASES = [  # N, C, H, W, K, kernel, stride: 1x1 and 3x3 layers of the 14x14 and 7x7 stages
    (2, 1024, 14, 14, 256, 1, 1), (1, 2048, 7, 7, 512, 1, 1), (3, 512, 7, 7, 2048, 1, 1), (2, 512, 28, 28, 1024, 1, 2),
    (1, 256, 9, 13, 128, 1, 1), (2, 1024, 14, 14, 2048, 1, 2), (2, 512, 7, 7, 512, 3, 1), (1, 256, 28, 28, 256, 3, 2),
    (2, 128, 14, 21, 128, 3, 1), (1, 512, 14, 14, 512, 3, 2), (1, 128, 56, 28, 128, 3, 2), (2, 256, 14, 14, 256, 3, 1),
]


@pytest.mark.parametrize("case", WREG_CASES, ids=lambda c: "x".join(map(str, c)))
def test_register_fed_convolution(case):
    """conv_wreg_kernel (special(3)) against the oracle's convolution and, for 1x1 layers, convolution + add."""
    N, C, H, W, K, k, st = case
    rng = np.random.default_rng(3000 + C + K + k)
    x = rng.integers(0, 256, (N, C, H, W), dtype=np.uint8)
    w = rng.integers(1, 256, (K, C, k, k), dtype=np.uint8)
    sigma = 74.0 * 74.0 * math.sqrt(C * k * k)
    b = rng.integers(-int(sigma), int(sigma) + 1, K).astype(np.int32)
    for relu in (False, True):
        ia, iz = 0.03, int(rng.integers(0, 256))
        oa = float(np.float32(ia * rng.uniform(0.75, 1.35)))
        q = (ia, iz, float(np.float32(oa * 40.0 / (ia * sigma))), 128, oa, int(rng.integers(0, 200)))
        plan = hipq.Conv2d(x.shape, w, b, k // 2, st, 1, *q, relu=relu).special(3)
        print("register-fed case", case, relu, plan.kernel, flush=True)
        assert plan.kernel == "conv_mfma_i8_wreg", plan.kernel
        want = orc.conv2d_u8(x, w, b, k // 2, st, 1, *q)
        if relu:
            want = np.maximum(want, q[5]).astype(np.uint8)
        xd = hipq.to_device_nhwc(x)
        y = plan(xd)
        torch.cuda.synchronize()
        got = hipq.from_device_nhwc(y, K)
        bad = got != want
        assert not bad.any(), (case, relu, int(bad.sum()), np.argwhere(bad)[:8].tolist())
        if k == 1 and not relu:
            for res_first in (False, True):
                res = rng.integers(0, 256, want.shape, dtype=np.uint8)
                ra, rz = float(np.float32(oa * rng.uniform(0.6, 1.6))), int(rng.integers(0, 256))
                sa, sz = float(np.float32(math.hypot(oa, ra) * 1.1)), int(rng.integers(0, 40))
                assert plan.kernel_add == "conv_mfma_i8_wreg+add", plan.kernel_add
                wanta = orc.add_u8(res, want, ra, rz, q[4], q[5], sa, sz) if res_first else orc.add_u8(want, res, q[4], q[5], ra, rz, sa, sz)
                ya = torch.zeros_like(y)
                plan.run_add(xd, hipq.to_device_nhwc(res), res_first, ra, rz, sa, sz, ya)
                torch.cuda.synchronize()
                gota = hipq.from_device_nhwc(ya, K)
                assert np.array_equal(gota, wanta), (case, "add", res_first, int((gota != wanta).sum()))


ADD2_CASES = [  # N, C (widening layer's input channels), output H, W, K, the shortcut's stride
    (2, 256, 14, 14, 1024, 2), (3, 512, 7, 7, 2048, 2), (1, 256, 9, 13, 384, 1), (2, 512, 14, 7, 1024, 1),
]


@pytest.mark.parametrize("case", ADD2_CASES, ids=lambda c: "x".join(map(str, c)))
def test_widening_convolution_shortcut_and_add(case):
    """hipq_conv2d_run_add2: the widening 1x1 convolution of a block, its projection shortcut (1x1, stride 1 or 2, from the
    block's input) and the add, against the oracle's three operators; both operand orders."""
    N, C, H, W, K, st = case
    rng = np.random.default_rng(4000 + C + K + st)
    x = rng.integers(0, 256, (N, C, H, W), dtype=np.uint8)
    xs = rng.integers(0, 256, (N, 2 * C, H * st - (st - 1), W * st - (st - 1)), dtype=np.uint8)

    def layer(Cin):
        w = rng.integers(1, 256, (K, Cin, 1, 1), dtype=np.uint8)
        sigma = 74.0 * 74.0 * math.sqrt(Cin)
        b = rng.integers(-int(sigma), int(sigma) + 1, K).astype(np.int32)
        ia, iz = float(np.float32(rng.uniform(0.02, 0.06))), int(rng.integers(0, 256))
        oa = float(np.float32(ia * rng.uniform(0.75, 1.35)))
        return w, b, (ia, iz, float(np.float32(oa * 40.0 / (ia * sigma))), 128, oa, int(rng.integers(96, 160)))
    w, b, q = layer(C)
    ws_, bs, qs = layer(2 * C)
    pm = hipq.Conv2d(x.shape, w, b, 0, 1, 1, *q).special(2)
    ps = hipq.Conv2d(xs.shape, ws_, bs, 0, st, 1, *qs)
    want_m = orc.conv2d_u8(x, w, b, 0, 1, 1, *q)
    want_s = orc.conv2d_u8(xs, ws_, bs, 0, st, 1, *qs)
    assert want_m.shape == want_s.shape
    xd, xsd = hipq.to_device_nhwc(x), hipq.to_device_nhwc(xs)
    for sc_first in (False, True):
        sa, sz = float(np.float32(math.hypot(q[4], qs[4]) * 1.1)), int(rng.integers(0, 40))
        print("add2 case", case, sc_first, pm.kernel, ps.kernel, flush=True)
        assert hipq.add2_fusable(pm, ps, sc_first, sa, sz)
        want = orc.add_u8(want_s, want_m, qs[4], qs[5], q[4], q[5], sa, sz) if sc_first else orc.add_u8(want_m, want_s, q[4], q[5], qs[4], qs[5], sa, sz)
        y = pm.empty_output()
        hipq.run_add2(pm, xd, ps, xsd, sc_first, sa, sz, y)
        torch.cuda.synchronize()
        got = hipq.from_device_nhwc(y, K)
        bad = got != want
        assert not bad.any(), (case, sc_first, int(bad.sum()), np.argwhere(bad)[:8].tolist())
    # a shortcut with other output channels is refused
    w3 = rng.integers(1, 256, (K + 128, 2 * C, 1, 1), dtype=np.uint8)
    p3 = hipq.Conv2d(xs.shape, w3, None, 0, st, 1, *qs)
    assert not hipq.add2_fusable(pm, p3, False, 0.1, 0)
    with pytest.raises(hipq.HipqError, match="do not run as one kernel"):
        hipq.run_add2(pm, xd, p3, xsd, False, 0.1, 0, pm.empty_output())


def time_layers():
    """Every convolution of the 28x28-and-smaller stages of ResNet-50 at batch 64: the built-in kernel against special(3)."""
    rng = np.random.default_rng(9)
    layers = [  # C, H, K, k, stride, with add
        (256, 56, 128, 1, 1, False), (128, 56, 128, 3, 2, False), (256, 56, 512, 1, 2, False), (512, 28, 128, 1, 1, False),
        (512, 28, 256, 1, 1, False), (256, 28, 256, 3, 2, False), (512, 28, 1024, 1, 2, False), (256, 14, 1024, 1, 1, True),
        (1024, 14, 256, 1, 1, False), (256, 14, 256, 3, 1, False), (1024, 14, 512, 1, 1, False), (512, 14, 512, 3, 2, False),
        (1024, 14, 2048, 1, 2, False), (512, 7, 2048, 1, 1, True), (2048, 7, 512, 1, 1, False), (512, 7, 512, 3, 1, False),
    ]
    for C, HW, K, k, st, add in layers:
        N = 64
        x = torch.randint(0, 256, (N, HW, HW, C), dtype=torch.uint8, device="cuda")
        w = rng.integers(1, 256, (K, C, k, k), dtype=np.uint8)
        sigma = 74.0 * 74.0 * math.sqrt(C * k * k)
        b = rng.integers(-int(sigma), int(sigma) + 1, K).astype(np.int32)
        q = (0.03, 120, float(np.float32(40.0 / sigma)), 128, 0.03, 0 if not add else 128)
        out = {}
        for mode in (1, 3):
            plan = hipq.Conv2d((N, C, HW, HW), w, b, k // 2, st, 1, *q).special(mode)
            y = plan.empty_output()
            res = torch.randint(0, 256, y.shape, dtype=torch.uint8, device="cuda")
            fn = (lambda: plan.run_add(x, res, False, 0.04, 100, 0.06, 0, y)) if add else (lambda: plan(x, y))
            fn()
            torch.cuda.synchronize()
            g = torch.cuda.CUDAGraph()
            with torch.cuda.graph(g):
                for _ in range(10):
                    fn()
            for _ in range(3):
                g.replay()
            torch.cuda.synchronize()
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record()
            for _ in range(20):
                g.replay()
            e1.record()
            torch.cuda.synchronize()
            out[mode] = (e0.elapsed_time(e1) / 200 * 1e3, plan.kernel_add if add else plan.kernel)
        print("layer C=%4d %2dx%2d K=%4d k=%d s=%d add=%d: %-34s %6.1f us | %-22s %6.1f us" % (
            C, HW, HW, K, k, st, add, out[1][1], out[1][0], out[3][1], out[3][0]), flush=True)


def time_block(N, CW, HW, reps=50):
    rng = np.random.default_rng(5)
    x, xq, layers, sq = make_block(rng, N, CW, HW, HW)
    plans = plans_of(x, layers)
    xd = hipq.to_device_nhwc(x)
    y = torch.zeros_like(xd)
    t1, t2 = plans[0].empty_output(), plans[1].empty_output()

    def fused():
        hipq.bottleneck_run(*plans, xd, False, sq[0], sq[1], y)

    def separate():
        plans[0](xd, t1)
        plans[1](t1, t2)
        plans[2].run_add(t2, xd, False, xq[0], xq[1], sq[0], sq[1], y)

    out = {}
    for name, fn in (("fused", fused), ("separate", separate)):
        fn()
        torch.cuda.synchronize()
        g = torch.cuda.CUDAGraph()
        with torch.cuda.graph(g):
            for _ in range(10):
                fn()
        for _ in range(3):
            g.replay()
        torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(reps):
            g.replay()
        e1.record()
        torch.cuda.synchronize()
        out[name] = e0.elapsed_time(e1) / reps / 10 * 1e3
    print("block N=%d CW=%d %dx%d: fused %.1f us, separate (%s) %.1f us" % (
        N, CW, HW, HW, out["fused"], " + ".join([plans[0].kernel, plans[1].kernel, plans[2].kernel_add]), out["separate"]), flush=True)


if __name__ == "__main__":
    for N, CW, HW in ((64, 1024, 14), (64, 512, 28), (64, 256, 56)):
        time_block(N, CW, HW)
    for N, CW, HW in ((64, 1024, 14), (64, 512, 28), (64, 256, 56)):
        time_tail(N, CW, HW)
    time_layers()
