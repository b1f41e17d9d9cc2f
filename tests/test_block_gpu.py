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


def plans_of(x, layers):
    shape = x.shape
    plans = []
    for L in layers:
        p = hipq.Conv2d(shape, L["w"], L["b"], L["pad"], 1, 1, *L["q"])
        plans.append(p)
        if len(plans) == 1:
            p.special(2)  # the block kernel wherever it applies, not only where the built-in rule uses it
        shape = (shape[0], L["w"].shape[0], shape[2], shape[3])
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
