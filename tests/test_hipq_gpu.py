"""GPU parity of the hipq kernels against the CPU oracle, through the C ABI (ctypes -> libhipq.so).

Bar: bit-exact uint8 outputs AND bit-exact int32 accumulators for conv / ip; bit-exact bytes for add,
eltwise, relu, pool and quantize (the kernel uses IEEE fp32 divide, so the 1-LSB allowance is not
needed); bit-exact fp32 for dequantize.
"""
import json
import os

import numpy as np
import pytest

pytestmark = pytest.mark.gpu

torch = pytest.importorskip("torch")

from oracle import orc  # noqa: E402  (checker only)
from nart_amd import hipq  # noqa: E402

HERE = os.path.dirname(os.path.abspath(__file__))


def rand_q(rng, lo=1e-3, hi=1e-1):
    return float(np.float32(np.exp(rng.uniform(np.log(lo), np.log(hi)))))


def run_conv(x, w, b, pad, stride, group, q, relu=False, want_acc=True):
    plan = hipq.Conv2d(x.shape, w, b, pad, stride, group, *q, relu=relu)
    xd = hipq.to_device_nhwc(x)
    acc = torch.zeros((x.shape[0], plan.OH, plan.OW, plan.desc.out_cs), dtype=torch.int32, device="cuda") if want_acc else None
    yd = plan(xd, acc=acc)
    torch.cuda.synchronize()
    y = hipq.from_device_nhwc(yd, w.shape[0])
    a = acc.cpu().numpy()[..., :w.shape[0]].transpose(0, 3, 1, 2) if want_acc else None
    return y, a, plan.kernel


def check_conv(x, w, b, pad, stride, group, q, tag=""):
    print("conv case", tag, x.shape, w.shape, pad, stride, group, q, flush=True)
    want_y, want_acc = orc.conv2d_u8(x, w, b, pad, stride, group, *q, return_acc=True)
    y, acc, kern = run_conv(x, w, b, pad, stride, group, q)
    assert np.array_equal(acc, want_acc), (tag, kern, "accumulators differ", int((acc != want_acc).sum()))
    assert np.array_equal(y, want_y), (tag, kern, "outputs differ", int((y != want_y).sum()))
    return kern


with open(os.path.join(HERE, "golden", "conv_kat.json")) as f:
    KATS = json.load(f)["cases"]


@pytest.mark.parametrize("c", KATS, ids=lambda c: c["id"])
def test_conv_known_answers_on_gpu(c):
    """The reference's recorded checksums, reproduced by the HIP kernels (config 1 is the first)."""
    from test_oracle import kat_case
    x, w, b = kat_case(c)
    y, _, kern = run_conv(x, w, b, c["pad"], c["stride"], c["group"], (0.02, c["izp"], 0.005, 128, 0.05, c["ozp"]),
                          want_acc=False)
    assert "%016x" % orc.fnv1a64(y) == c["fnv"], kern


def test_conv_mfma_shapes():
    rng = np.random.default_rng(11)
    kerns = set()
    cases = [  # N, C, H, W, K, R, S, pad, stride
        (2, 64, 14, 14, 64, 3, 3, 1, 1), (1, 64, 9, 11, 128, 1, 1, 0, 1), (3, 32, 10, 7, 48, 3, 3, 1, 2),
        (1, 16, 12, 12, 24, 5, 3, 1, 1), (2, 128, 7, 7, 256, 1, 1, 0, 2), (1, 48, 8, 8, 200, 3, 3, 0, 1),
        (1, 3, 33, 29, 64, 7, 7, 3, 2), (2, 3, 16, 16, 16, 3, 3, 1, 1), (1, 1, 9, 9, 8, 5, 5, 2, 1),
        (1, 20, 6, 6, 10, 3, 3, 1, 1), (1, 256, 4, 4, 64, 3, 3, 1, 1), (5, 24, 5, 5, 40, 1, 1, 0, 1),
    ]
    for i, (N, C, H, W, K, R, S, pad, st) in enumerate(cases):
        x = rng.integers(0, 256, (N, C, H, W), dtype=np.uint8)
        w = rng.integers(0, 256, (K, C, R, S), dtype=np.uint8)
        b = rng.integers(-30000, 30000, K).astype(np.int32)
        for wzp in (128, int(rng.integers(0, 256))):
            q = (rand_q(rng), int(rng.integers(0, 256)), rand_q(rng), wzp, rand_q(rng, 1e-2, 1.0), int(rng.integers(0, 256)))
            kerns.add(check_conv(x, w, b, pad, st, 1, q, tag="mfma%d" % i))
    assert any("mfma" in k and "_wzp" in k for k in kerns) and any("_c4" in k for k in kerns), kerns


def test_conv_edge_cases():
    rng = np.random.default_rng(12)
    # extreme values: all-255 activations against all-0 / all-255 weights, zero points at both ends
    for xv, wv, izp, wzp in ((255, 255, 0, 0), (255, 0, 0, 255), (0, 255, 255, 0), (0, 0, 255, 255)):
        x = np.full((1, 64, 6, 6), xv, np.uint8)
        w = np.full((64, 64, 3, 3), wv, np.uint8)
        check_conv(x, w, None, 1, 1, 1, (0.01, izp, 0.01, wzp, 0.9, 3), tag="extreme")
    # no bias, asymmetric padding and stride, ragged pixel count (not a multiple of any tile)
    x = rng.integers(0, 256, (1, 32, 13, 5), dtype=np.uint8)
    w = rng.integers(0, 256, (33, 32, 3, 2), dtype=np.uint8)
    check_conv(x, w, None, (2, 0), (2, 1), 1, (0.02, 7, 0.005, 128, 0.05, 0), tag="ragged")
    # accumulator wrap-around: 4608 taps of (255-0)*(255-0) stay below 2^31, so force it with a huge bias
    x = np.full((1, 512, 3, 3), 255, np.uint8)
    w = np.full((16, 512, 3, 3), 255, np.uint8)
    b = np.full(16, 2**31 - 1000, np.int32)
    check_conv(x, w, b, 1, 1, 1, (0.01, 0, 0.01, 0, 0.5, 0), tag="wrap")
    # fused ReLU == conv followed by the reference relu with identical scales / zero point
    x = rng.integers(0, 256, (1, 16, 8, 8), dtype=np.uint8)
    w = rng.integers(0, 256, (16, 16, 3, 3), dtype=np.uint8)
    q = (0.02, 100, 0.005, 128, 0.05, 90)
    y, _, _ = run_conv(x, w, None, 1, 1, 1, q, relu=True, want_acc=False)
    want = orc.relu_u8(orc.conv2d_u8(x, w, None, 1, 1, 1, *q), 0.05, 90, 0.05, 90)
    assert np.array_equal(y, want)
    # fewer output bits, with a zero point inside and beyond the saturation value (then only that value remains)
    for obits, ozp in ((4, 9), (4, 200), (7, 127), (7, 128)):
        q = (0.02, 100, 0.005, 128, 0.05, ozp)
        plan = hipq.Conv2d(x.shape, w, None, 1, 1, 1, *q, obits=obits, relu=True)
        got = hipq.from_device_nhwc(plan(hipq.to_device_nhwc(x)), 16)
        want = orc.relu_u8(orc.conv2d_u8(x, w, None, 1, 1, 1, *q, obits=obits), 0.05, ozp, 0.05, ozp, obits)
        assert np.array_equal(got, want), (obits, ozp)


def test_conv_with_fused_residual_add():
    """hipq_conv2d_run_add == conv followed by the reference add, byte for byte: both operand orders, the 32-bit
    fast form and the 64-bit form of the add (very unequal scales), every tile shape's epilogue, ragged tiles,
    a narrow output (plain store path) and asymmetric weights."""
    rng = np.random.default_rng(21)
    shapes = [  # N, C, H, W, K, R, pad, stride
        (2, 64, 14, 14, 256, 1, 0, 1), (1, 64, 9, 11, 64, 3, 1, 1), (3, 32, 10, 7, 48, 3, 1, 2), (1, 256, 5, 5, 512, 1, 0, 1),
        (1, 16, 6, 6, 3, 3, 1, 1), (2, 128, 28, 28, 128, 3, 1, 1),
    ]
    for i, (N, C, H, W, K, R, pad, st) in enumerate(shapes):
        x = rng.integers(0, 256, (N, C, H, W), dtype=np.uint8)
        w = rng.integers(0, 256, (K, C, R, R), dtype=np.uint8)
        b = rng.integers(-30000, 30000, K).astype(np.int32)
        for res_first, wzp, ratio in ((False, 128, 1.0), (True, 128, 1.7), (False, int(rng.integers(0, 256)), 3000.0),
                                      (True, 128, 1 / 2500.0)):
            q = (rand_q(rng), int(rng.integers(0, 256)), rand_q(rng), wzp, rand_q(rng, 1e-2, 1.0), int(rng.integers(0, 256)))
            plan = hipq.Conv2d(x.shape, w, b, pad, st, 1, *q)
            conv = orc.conv2d_u8(x, w, b, pad, st, 1, *q)
            res = rng.integers(0, 256, conv.shape, dtype=np.uint8)
            ra, rz = float(np.float32(q[4] * ratio)), int(rng.integers(0, 256))
            oa, oz = float(np.float32(max(q[4], ra) * 1.3)), int(rng.integers(0, 256))
            print("fused add case", i, x.shape, w.shape, res_first, ratio, plan.kernel, flush=True)
            want = orc.add_u8(res, conv, ra, rz, q[4], q[5], oa, oz) if res_first else orc.add_u8(conv, res, q[4], q[5], ra, rz, oa, oz)
            y = plan.empty_output()
            plan.run_add(hipq.to_device_nhwc(x), hipq.to_device_nhwc(res), res_first, ra, rz, oa, oz, y)
            torch.cuda.synchronize()
            got = hipq.from_device_nhwc(y, K)
            assert np.array_equal(got, want), (i, res_first, ratio, plan.kernel, int((got != want).sum()))
    # a plan that does not run an MFMA kernel refuses, loudly
    xdw = rng.integers(0, 256, (1, 32, 8, 8), dtype=np.uint8)
    plan = hipq.Conv2d(xdw.shape, rng.integers(0, 256, (32, 1, 3, 3), dtype=np.uint8), None, 1, 1, 32, 0.02, 3, 0.01, 128, 0.05, 9)
    with pytest.raises(hipq.HipqError, match="only the MFMA"):
        plan.run_add(hipq.to_device_nhwc(xdw), hipq.to_device_nhwc(xdw), False, 0.05, 0, 0.07, 0, plan.empty_output())


def test_channel_widening_1x1_layers():
    """conv_mfma_expand_kernel (1x1, 64 / 128 / 256 input channels, at least four times 64 output channels, 1024 pixels
    or more): alone against the oracle's convolution (accumulator dump through the tile kernels aside, outputs only), with
    ReLU, and with the residual add fused in, both operand orders; ragged pixel counts, an output width that is not a
    multiple of 64, strides, int8 tensors.  special(0) runs the same plans on the tile kernels: identical bytes."""
    rng = np.random.default_rng(77)
    shapes = [  # N, C, H, W, K, stride
        (2, 64, 28, 28, 256, 1), (1, 128, 40, 30, 512, 1), (8, 256, 28, 28, 1024, 2), (1, 64, 33, 37, 272, 1),
        (3, 128, 21, 19, 300, 1), (4, 256, 47, 30, 520, 2),
    ]
    seen = set()
    for i, (N, C, H, W, K, st) in enumerate(shapes):
        x = rng.integers(0, 256, (N, C, H, W), dtype=np.uint8)
        w = rng.integers(0, 256, (K, C, 1, 1), dtype=np.uint8)
        b = rng.integers(-30000, 30000, K).astype(np.int32)
        for relu in (False, True):
            q = (rand_q(rng), int(rng.integers(0, 256)), rand_q(rng), 128, rand_q(rng, 1e-2, 1.0), int(rng.integers(0, 256)))
            plan = hipq.Conv2d(x.shape, w, b, 0, st, 1, *q, relu=relu)
            # built-in rule: only on many pixels (below); special(2): wherever the kernel applies
            assert plan.kernel != "conv_mfma_i8_expand", plan.kernel
            plan.special(2)
            print("widening case", i, x.shape, w.shape, st, relu, plan.kernel, flush=True)
            assert plan.kernel == "conv_mfma_i8_expand", plan.kernel
            seen.add(plan.kernel)
            want = orc.conv2d_u8(x, w, b, 0, st, 1, *q)
            if relu:
                want = orc.relu_u8(want, q[4], q[5], q[4], q[5])
            xd = hipq.to_device_nhwc(x)
            got = hipq.from_device_nhwc(plan(xd), K)
            assert np.array_equal(got, want), (i, relu, int((got != want).sum()))
            plan.special(0)
            assert np.array_equal(hipq.from_device_nhwc(plan(xd), K), want), (i, relu, plan.kernel)
        for res_first, ratio, obits in ((False, 1.0, 8), (True, 1.7, 8), (False, 0.6, 7)):
            q = (rand_q(rng), int(rng.integers(0, 256)), rand_q(rng), 128, rand_q(rng, 1e-2, 1.0), int(rng.integers(0, 256)))
            plan = hipq.Conv2d(x.shape, w, b, 0, st, 1, *q)
            assert plan.kernel_add != "conv_mfma_i8_expand+add", plan.kernel_add  # built-in rule: many pixels only
            plan.special(2)
            assert plan.kernel_add == "conv_mfma_i8_expand+add", plan.kernel_add
            conv = orc.conv2d_u8(x, w, b, 0, st, 1, *q)
            res = rng.integers(0, 256, conv.shape, dtype=np.uint8)
            ra, rz = float(np.float32(q[4] * ratio)), int(rng.integers(0, 256))
            oa, oz = float(np.float32(max(q[4], ra) * 1.3)), int(rng.integers(0, 1 << obits))
            print("widening case with add", i, res_first, ratio, obits, plan.kernel_add, flush=True)
            want = (orc.add_u8(res, conv, ra, rz, q[4], q[5], oa, oz, obits) if res_first
                    else orc.add_u8(conv, res, q[4], q[5], ra, rz, oa, oz, obits))
            xd, rd = hipq.to_device_nhwc(x), hipq.to_device_nhwc(res)
            for mode in (2, 0):
                plan.special(mode)
                y = plan.empty_output()
                plan.run_add(xd, rd, res_first, ra, rz, oa, oz, y, obits=obits)
                torch.cuda.synchronize()
                got = hipq.from_device_nhwc(y, K)
                assert np.array_equal(got, want), (i, res_first, ratio, obits, mode, int((got != want).sum()))
    # the built-in rule: a launch of this kernel has a floor of 6.6 us, so it is chosen on many pixels only - without the
    # add at 256 input channels from 20 000 pixels, at 64 input channels (with or without the add) from 150 000, with the
    # add at 128 input channels from 50 000
    for (N, C, H, K, st), plain, added in (((64, 256, 56, 512, 2), True, False), ((16, 256, 56, 512, 2), False, False),
                                           ((64, 64, 56, 256, 1), True, True), ((32, 64, 56, 256, 1), False, False),
                                           ((64, 128, 28, 512, 1), False, True), ((32, 128, 28, 512, 1), False, False)):
        plan = hipq.Conv2d((N, C, H, H), rng.integers(0, 256, (K, C, 1, 1), dtype=np.uint8), None, 0, st, 1, 0.02, 3, 0.004, 128, 0.3, 5)
        assert (plan.kernel == "conv_mfma_i8_expand") == plain, (N, C, H, K, st, plan.kernel)
        assert (plan.kernel_add == "conv_mfma_i8_expand+add") == added, (N, C, H, K, st, plan.kernel_add)
    # int8 tensors through the same kernel
    x = rng.integers(-128, 128, (2, 64, 24, 24), dtype=np.int8)
    w = rng.integers(-127, 128, (256, 64, 1, 1), dtype=np.int8)
    b = rng.integers(-30000, 30000, 256).astype(np.int32)
    for obits in (8, 7):
        plan = hipq.Conv2d(x.shape, w, b, 0, 1, 1, 0.02, 0, 0.004, 0, 0.09, 0, obits=obits, dtype=hipq.DTYPE_I8).special(2)
        assert plan.kernel == "conv_mfma_i8_expand_signed", plan.kernel
        got = hipq.from_device_nhwc(plan(hipq.to_device_nhwc(x)), 256).view(np.int8)
        assert np.array_equal(got, orc.conv2d_i8(x, w, b, 0, 1, 1, 0.02, 0.004, 0.09, obits=obits)), obits


def test_fused_add_chained_with_the_next_1x1_convolution():
    """hipq_conv2d_run_add_conv: the widening 1x1 convolution of a bottleneck block, its residual add and the first 1x1
    convolution of the next block in one kernel, against the oracle's three operators: both operand orders of the add,
    64 and 128 channels out of the second convolution, with and without its ReLU, ragged pixel counts, five channel tiles.
    The sum itself is written as well.  Pairs the kernel does not serve are refused."""
    rng = np.random.default_rng(78)
    shapes = [  # N, C, H, W, K, mid, relu
        (2, 64, 28, 28, 256, 64, True), (1, 128, 40, 30, 512, 128, True), (1, 64, 33, 37, 256, 128, False),
        (3, 128, 21, 19, 320, 64, True),
    ]
    for i, (N, C, H, W, K, mid, relu) in enumerate(shapes):
        x = rng.integers(0, 256, (N, C, H, W), dtype=np.uint8)
        w = rng.integers(0, 256, (K, C, 1, 1), dtype=np.uint8)
        b = rng.integers(-30000, 30000, K).astype(np.int32)
        w2 = rng.integers(0, 256, (mid, K, 1, 1), dtype=np.uint8)
        b2 = rng.integers(-30000, 30000, mid).astype(np.int32)
        for res_first, ratio in ((False, 1.0), (True, 1.7)):
            # output scales of the order of the accumulators' spread: the requantisation shifts then lie inside the range of
            # the one-multiply form, which the kernel requires (as the scales of a calibrated network do)
            ia, wa = rand_q(rng), rand_q(rng)
            q = (ia, int(rng.integers(0, 256)), wa, 128, float(np.float32(ia * wa * np.sqrt(C) * 40.0)), int(rng.integers(0, 256)))
            plan = hipq.Conv2d(x.shape, w, b, 0, 1, 1, *q)
            conv = orc.conv2d_u8(x, w, b, 0, 1, 1, *q)
            res = rng.integers(0, 256, conv.shape, dtype=np.uint8)
            ra, rz = float(np.float32(q[4] * ratio)), int(rng.integers(0, 256))
            oa, oz = float(np.float32(max(q[4], ra) * 1.3)), int(rng.integers(0, 256))
            want = orc.add_u8(res, conv, ra, rz, q[4], q[5], oa, oz) if res_first else orc.add_u8(conv, res, q[4], q[5], ra, rz, oa, oz)
            wa2 = rand_q(rng)
            q2 = (oa, oz, wa2, 128, float(np.float32(oa * wa2 * np.sqrt(K) * 40.0)), int(rng.integers(0, 256)))
            nxt = hipq.Conv2d(want.shape, w2, b2, 0, 1, 1, *q2, relu=relu)
            want2 = orc.conv2d_u8(want, w2, b2, 0, 1, 1, *q2)
            if relu:
                want2 = orc.relu_u8(want2, q2[4], q2[5], q2[4], q2[5])
            print("chained case", i, x.shape, K, mid, relu, res_first, flush=True)
            assert plan.add_conv_fusable(res_first, ra, rz, oa, oz, nxt)
            y, y2 = plan.empty_output(), nxt.empty_output()
            y.fill_(3), y2.fill_(5)
            plan.run_add_conv(hipq.to_device_nhwc(x), hipq.to_device_nhwc(res), res_first, ra, rz, oa, oz, y, nxt, y2)
            torch.cuda.synchronize()
            got, got2 = hipq.from_device_nhwc(y, K), hipq.from_device_nhwc(y2, mid)
            assert np.array_equal(got, want), (i, res_first, "sum", int((got != want).sum()))
            assert np.array_equal(got2, want2), (i, res_first, "next layer", int((got2 != want2).sum()))
            # refusals: another input scale of the second convolution, a 3x3 second convolution, an explicit tile
            other = hipq.Conv2d(want.shape, w2, b2, 0, 1, 1, float(np.float32(oa * 1.01)), oz, *q2[2:])
            assert not plan.add_conv_fusable(res_first, ra, rz, oa, oz, other)
            if i == 0:
                k3 = hipq.Conv2d(want.shape, rng.integers(0, 256, (mid, K, 3, 3), dtype=np.uint8), b2, 1, 1, 1, *q2)
                assert not plan.add_conv_fusable(res_first, ra, rz, oa, oz, k3)
                with pytest.raises(hipq.HipqError, match="do not run as one kernel"):
                    plan.run_add_conv(hipq.to_device_nhwc(x), hipq.to_device_nhwc(res), res_first, ra, rz, oa, oz, y, k3, k3.empty_output())
                plan.select(4, 0)
                assert not plan.add_conv_fusable(res_first, ra, rz, oa, oz, nxt)


def test_conv_grouped_and_depthwise():
    rng = np.random.default_rng(13)
    kerns = set()
    for (N, C, H, W, K, R, S, pad, st, grp) in [(2, 32, 14, 14, 32, 3, 3, 1, 1, 32), (1, 96, 9, 9, 96, 3, 3, 1, 2, 96),
                                                 (1, 24, 7, 7, 24, 5, 5, 2, 1, 24), (1, 16, 8, 8, 32, 3, 3, 1, 1, 4),
                                                 (2, 12, 6, 6, 6, 1, 1, 0, 1, 3)]:
        x = rng.integers(0, 256, (N, C, H, W), dtype=np.uint8)
        w = rng.integers(0, 256, (K, C // grp, R, S), dtype=np.uint8)
        b = rng.integers(-3000, 3000, K).astype(np.int32)
        q = (rand_q(rng), int(rng.integers(0, 256)), rand_q(rng), int(rng.integers(0, 256)), rand_q(rng, 1e-2, 1.0),
             int(rng.integers(0, 256)))
        kerns.add(check_conv(x, w, b, pad, st, grp, q, tag="grouped"))
    assert "conv_depthwise_u8" in kerns and "conv_direct_u8" in kerns


def test_depthwise3x3_walk_shapes():
    """The depthwise 3x3 kernel whose threads walk down the image (weight zero point 128): widths that are not multiples
    of the 4-column strip, one to three rows, no padding, both strides on even and odd sizes, channel counts that fill a
    wave unevenly; with and without the accumulator dump, a ReLU clamp (one-multiply requantisation with clamps), the
    plain [0, 255] range (saturating packs) and a scale outside the one-multiply range (64-bit form).  A weight zero
    point other than 128 takes the older kernel and is checked beside it."""
    rng = np.random.default_rng(77)
    shapes = [  # N, C, H, W, pad, stride
        (2, 32, 14, 14, 1, 1), (1, 96, 9, 9, 1, 2), (3, 8, 5, 7, 1, 1), (1, 4, 1, 1, 1, 1), (1, 12, 2, 13, 1, 1),
        (2, 20, 3, 5, 1, 2), (1, 16, 8, 8, 1, 2), (1, 144, 6, 10, 0, 1), (1, 24, 7, 9, 0, 2), (1, 260, 4, 6, 1, 1),
        (1, 8, 33, 4, 1, 1), (2, 8, 12, 21, 1, 2),
    ]
    kerns = set()
    for i, (N, C, H, W, pad, st) in enumerate(shapes):
        x = rng.integers(0, 256, (N, C, H, W), dtype=np.uint8)
        w = rng.integers(0, 256, (C, 1, 3, 3), dtype=np.uint8)
        b = rng.integers(-3000, 3000, C).astype(np.int32)
        izp, ozp = int(rng.integers(0, 256)), int(rng.integers(0, 200))
        ia, wa = rand_q(rng), rand_q(rng)
        oa = float(np.float32(ia * wa * 3000.0 / 200.0))     # sums of +-3000 land on the byte range: one-multiply form
        for wzp in (128, 131):
            q = (ia, izp, wa, wzp, oa, ozp)
            kerns.add(check_conv(x, w, b, pad, st, C, q, tag="dw%d" % i))
            want = orc.conv2d_u8(x, w, b, pad, st, C, *q)
            plan = hipq.Conv2d(x.shape, w, b, pad, st, C, *q)
            xd = hipq.to_device_nhwc(x)
            assert np.array_equal(hipq.from_device_nhwc(plan(xd), C), want), (i, wzp, plan.kernel)          # no dump
            assert np.array_equal(hipq.from_device_nhwc(plan.run_relu(xd), C), np.maximum(want, ozp)), (i, wzp, plan.kernel)
            assert len(np.unique(want)) > 8 or want.size < 64, (i, "degenerate case")
        q = (ia, izp, wa, 128, float(np.float32(oa * 2.0 ** 22)), ozp)   # shift beyond the one-multiply range
        kerns.add(check_conv(x, w, b, pad, st, C, q, tag="dw%d_wide_shift" % i))
    assert kerns == {"conv_depthwise3x3_u8_s1", "conv_depthwise3x3_u8_s2", "conv_depthwise3x3_u8_s1_wzp",
                     "conv_depthwise3x3_u8_s2_wzp"}, kerns


def test_ip_as_1x1():
    rng = np.random.default_rng(14)
    for M, Kd, No in ((128, 512, 256), (5, 300, 37), (1, 2048, 1000)):
        x = rng.integers(0, 256, (M, Kd), dtype=np.uint8)
        w = rng.integers(0, 256, (No, Kd), dtype=np.uint8)
        b = rng.integers(-50000, 50000, No).astype(np.int32)
        q = (rand_q(rng), 128, rand_q(rng), int(rng.choice([128, 90])), rand_q(rng, 1e-1, 2.0), int(rng.integers(0, 256)))
        want_y, want_acc = orc.ip_u8(x, w, b, *q, return_acc=True)
        y, acc, _ = run_conv(x.reshape(M, Kd, 1, 1), w.reshape(No, Kd, 1, 1), b, 0, 1, 1, q)
        assert np.array_equal(acc.reshape(M, No), want_acc) and np.array_equal(y.reshape(M, No), want_y)
    # FC fed by a [M, C, H, W] tensor: weights re-ordered from (c,h,w) to the device's (h,w,c)
    M, Cc, H, W, No = 3, 20, 2, 3, 11
    x = rng.integers(0, 256, (M, Cc, H, W), dtype=np.uint8)
    w = rng.integers(0, 256, (No, Cc * H * W), dtype=np.uint8)
    q = (0.02, 128, 0.004, 131, 0.3, 5)
    want = orc.ip_u8(x.reshape(M, -1), w, None, *q)
    cs = hipq.channel_stride(Cc)
    w2 = np.empty((No, H * W * cs), np.uint8)
    hipq.check(hipq.lib().hipq_ip_reorder_weights(w.ctypes.data, w2.ctypes.data, No, Cc, H, W, cs, 131))
    plan = hipq.Conv2d((M, H * W * cs, 1, 1), w2.reshape(No, -1, 1, 1), None, 0, 1, 1, *q, in_cs=H * W * cs)
    yd = plan(hipq.to_device_nhwc(x))  # [M,H,W,cs] bytes == [M,1,1,H*W*cs]
    torch.cuda.synchronize()
    assert np.array_equal(yd.cpu().numpy().reshape(M, -1)[:, :No], want)


def test_fc_streaming_kernel():
    """Fully-connected layers (op_quant_ip_u8xu8_run, ip.cpp:133-209) on the streaming kernel: BASELINE configs[1] at
    its stated shape (M=128, K=4096, N=4096, full-range values, log-uniform scales) and the shapes around it, accumulators
    and bytes against the oracle; every work-group shape the kernel is instantiated for gives the same bytes."""
    rng = np.random.default_rng(141)
    shapes = [(128, 4096, 4096, False), (1, 512, 1000, False), (64, 2048, 1000, True), (5, 128, 37, False),
              (17, 256, 16, True), (130, 384, 100, False), (256, 1024, 48, False), (33, 1280, 1000, False)]
    for M, Kd, No, relu in shapes:
        print("fc case", M, Kd, No, relu, flush=True)
        x = rng.integers(0, 256, (M, Kd), dtype=np.uint8)
        w = rng.integers(0, 256, (No, Kd), dtype=np.uint8)
        b = rng.integers(-50000, 50000, No).astype(np.int32)
        ia, wa = rand_q(rng), rand_q(rng)
        # the output scale follows the spread of the sums (about 74 * 74 * sqrt(K) in input units), so that the bytes
        # are not all saturated; the accumulators are compared whatever the scales
        oa = float(np.float32(ia * wa * np.sqrt(Kd) * 60.0))
        q = (ia, 128 if M == 128 else int(rng.integers(0, 256)), wa, 128, oa, int(rng.integers(0, 256)))
        want_y, want_acc = orc.ip_u8(x, w, b, *q, return_acc=True)
        if relu:
            want_y = np.maximum(want_y, q[5]).astype(np.uint8)
        plan = hipq.Conv2d((M, Kd, 1, 1), w.reshape(No, Kd, 1, 1), b, 0, 1, 1, *q, relu=relu)
        assert "_stream_" in plan.kernel, plan.kernel
        xd = hipq.to_device_nhwc(x.reshape(M, Kd, 1, 1))
        acc = torch.zeros((M, 1, 1, plan.desc.out_cs), dtype=torch.int32, device="cuda")
        yd = plan(xd, acc=acc)
        torch.cuda.synchronize()
        got_acc = acc.cpu().numpy().reshape(M, -1)[:, :No]
        assert np.array_equal(got_acc, want_acc), (M, Kd, No, plan.kernel, int((got_acc != want_acc).sum()))
        first = yd.cpu().numpy().reshape(M, -1)
        assert np.array_equal(first[:, :No], want_y), (M, Kd, No, plan.kernel)
        assert len(np.unique(want_y)) > 8 or M < 8, "degenerate case: the scales saturate the outputs"
        for rows, cols, waves in ((128, 16, 4), (64, 32, 4), (64, 16, 4), (32, 16, 4), (32, 32, 4), (16, 16, 4), (16, 32, 4)):
            plan.stream(rows, cols, waves)
            assert plan.kernel.endswith("_stream_%dx%d" % (rows, cols)), plan.kernel
            y2 = plan(xd).cpu().numpy().reshape(M, -1)
            assert np.array_equal(y2[:, :No], want_y), (M, Kd, No, rows, cols, waves)
        plan.stream()
        # the dequantize that reads the layer, in the layer's epilogue (hipq_conv2d_run_dequant): the float bit patterns of
        # op_dequantize_run_u8 on the layer's bytes; refused for another scale or zero point than the bytes are written with
        assert plan.dequant_fusable(q[4], q[5]) and not plan.dequant_fusable(float(np.float32(q[4] * 1.5)), q[5])
        assert not plan.dequant_fusable(q[4], (q[5] + 1) % 256)
        yf = torch.full((M, No), 7.0, dtype=torch.float32, device="cuda")
        plan.run_dequant(xd, yf)
        want_f = orc.dequantize_u8(want_y, q[4], q[5])
        assert np.array_equal(yf.cpu().numpy().view(np.uint32), np.ascontiguousarray(want_f).reshape(M, No).view(np.uint32)), (M, Kd, No)
        # the tile kernels serve the same plan when the streaming kernel is switched off, with the same bytes
        plan.special(0)
        assert "_stream_" not in plan.kernel and not plan.dequant_fusable(q[4], q[5])
        y3 = plan(xd).cpu().numpy().reshape(M, -1)
        assert np.array_equal(y3[:, :No], want_y), (M, Kd, No, plan.kernel)
        plan.close()
    with pytest.raises(hipq.HipqError):  # not a streaming plan
        hipq.Conv2d((1, 64, 8, 8), np.zeros((64, 64, 3, 3), np.uint8), None, 1, 1, 1, 0.1, 0, 0.1, 128, 0.1, 0).stream(64, 16, 4)
    with pytest.raises(hipq.HipqError):  # no such instantiation
        hipq.Conv2d((4, 128, 1, 1), np.zeros((16, 128, 1, 1), np.uint8), None, 0, 1, 1, 0.1, 0, 0.1, 128, 0.1, 0).stream(128, 32, 4)


def test_streaming_kernel_on_convolutions_over_few_pixels():
    """conv_mfma_stream_kernel with the general pixel gather: any kernel size, stride and padding over at most 256 output
    pixels (1024 for long reductions) whose channels are whole 128-byte lines (the late stages of a network at batch 1), accumulators and
    bytes against the oracle; with the residual add fused, both operand orders; special(0) gives the same bytes."""
    rng = np.random.default_rng(91)
    cases = [  # N, C, H, W, K, R, pad, stride
        (1, 512, 7, 7, 512, 3, 1, 1), (1, 256, 14, 14, 512, 3, 1, 2), (1, 256, 14, 14, 256, 3, 1, 1), (2, 128, 9, 9, 64, 3, 1, 1),
        (1, 128, 5, 7, 40, 5, 2, 1), (1, 256, 14, 14, 512, 1, 0, 2), (3, 128, 6, 5, 136, 3, 0, 1), (1, 384, 16, 16, 96, 3, 1, 1),
        (1, 128, 28, 28, 128, 3, 1, 1), (3, 512, 17, 19, 72, 1, 0, 1),  # 257 to 1024 pixels: reductions of 512 bytes or more
    ]
    for i, (N, C, H, W, K, R, pad, st) in enumerate(cases):
        x = rng.integers(0, 256, (N, C, H, W), dtype=np.uint8)
        w = rng.integers(0, 256, (K, C, R, R), dtype=np.uint8)
        b = rng.integers(-30000, 30000, K).astype(np.int32)
        ia, wa = rand_q(rng), rand_q(rng)
        q = (ia, int(rng.integers(0, 256)), wa, 128, float(np.float32(ia * wa * np.sqrt(C * R * R) * 40.0)), int(rng.integers(0, 256)))
        kern = check_conv(x, w, b, pad, st, 1, q, tag="stream conv %d" % i)
        assert "_stream_" in kern, kern
        plan = hipq.Conv2d(x.shape, w, b, pad, st, 1, *q)
        conv = orc.conv2d_u8(x, w, b, pad, st, 1, *q)
        xd = hipq.to_device_nhwc(x)
        res = rng.integers(0, 256, conv.shape, dtype=np.uint8)
        rd = hipq.to_device_nhwc(res)
        ra, rz = float(np.float32(q[4] * (1.0, 1.7, 300.0)[i % 3])), int(rng.integers(0, 256))
        sa, sz = float(np.float32(max(q[4], ra) * 1.3)), int(rng.integers(0, 256))
        assert "_stream_" in plan.kernel_add and plan.kernel_add.endswith("+add"), plan.kernel_add
        for res_first in (False, True):
            want = orc.add_u8(res, conv, ra, rz, q[4], q[5], sa, sz) if res_first else orc.add_u8(conv, res, q[4], q[5], ra, rz, sa, sz)
            y = plan.empty_output()
            plan.run_add(xd, rd, res_first, ra, rz, sa, sz, y)
            assert np.array_equal(hipq.from_device_nhwc(y, K), want), (i, res_first, plan.kernel_add)
        plan.special(0)
        assert "_stream_" not in plan.kernel
        assert np.array_equal(hipq.from_device_nhwc(plan(xd), K), conv), (i, plan.kernel)


def test_output_stride_wider_than_the_channels():
    """A caller may write a convolution's output into a buffer with a wider channel stride than the layout rule gives
    (hipq_conv2d_desc.out_cs): the packed weights and folded constants cover every output-channel tile of that stride."""
    rng = np.random.default_rng(142)
    N, C, H, W, K = 2, 64, 9, 9, 64
    x = rng.integers(0, 256, (N, C, H, W), dtype=np.uint8)
    w = rng.integers(0, 256, (K, C, 3, 3), dtype=np.uint8)
    b = rng.integers(-1000, 1000, K).astype(np.int32)
    q = (0.02, 120, 0.005, 128, 0.05, 3)
    want = orc.conv2d_u8(x, w, b, 1, 1, 1, *q)
    for out_cs in (256, 384):
        plan = hipq.Conv2d(x.shape, w, b, 1, 1, 1, *q, out_cs=out_cs)
        for tile in (-1, 0, 2, 3, 4):
            if tile >= 0:
                plan.special(0).select(tile)
            yd = plan(hipq.to_device_nhwc(x))
            torch.cuda.synchronize()
            got = yd.cpu().numpy()[..., :K].transpose(0, 3, 1, 2)
            assert np.array_equal(got, want), (out_cs, plan.kernel)


def test_per_channel_weight_scales():
    """One weight scale per output channel (hipq_conv2d_plan_create_per_channel): every kernel family against the
    oracle's per-channel requantisation; K equal scales give the per-tensor plan's bytes; the fused add, the run-time
    ReLU, accumulator dumps, int8 tensors and the fully-connected kernel work on such plans."""
    rng = np.random.default_rng(143)
    #        N   C    H   W   K   R  pad st group
    cases = [(2, 64, 14, 14, 64, 3, 1, 1, 1), (1, 3, 33, 33, 24, 7, 3, 2, 1), (3, 32, 9, 9, 96, 1, 0, 1, 1),
             (2, 256, 7, 7, 128, 1, 0, 1, 1), (2, 32, 12, 12, 32, 3, 1, 1, 32), (1, 48, 11, 11, 48, 3, 1, 2, 48),
             (1, 24, 7, 7, 24, 5, 2, 1, 24), (1, 16, 8, 8, 32, 3, 1, 1, 4), (40, 256, 1, 1, 100, 1, 0, 1, 1)]
    kerns = set()
    for N, C, H, W, K, R, pad, st, grp in cases:
        print("per-channel case", N, C, H, W, K, R, pad, st, grp, flush=True)
        x = rng.integers(0, 256, (N, C, H, W), dtype=np.uint8)
        w = rng.integers(0, 256, (K, C // grp, R, R), dtype=np.uint8)
        b = rng.integers(-3000, 3000, K).astype(np.int32)
        ia, izp, wzp, ozp = rand_q(rng), int(rng.integers(0, 256)), 128, int(rng.integers(0, 256))
        wa = np.exp(rng.uniform(np.log(1e-3), np.log(3e-2), K)).astype(np.float32)
        oa = float(np.float32(ia * 5e-3 * np.sqrt(C // grp * R * R) * 60.0))
        want = orc.conv2d_u8_per_channel(x, w, b, pad, st, grp, ia, izp, wa, wzp, oa, ozp)
        _, want_acc = orc.conv2d_u8(x, w, b, pad, st, grp, ia, izp, float(wa[0]), wzp, oa, ozp, return_acc=True)
        plan = hipq.Conv2d(x.shape, w, b, pad, st, grp, ia, izp, wa, wzp, oa, ozp)
        assert plan.kernel.endswith("_perchannel"), plan.kernel
        kerns.add(plan.kernel)
        xd = hipq.to_device_nhwc(x)
        acc = torch.zeros((N, plan.OH, plan.OW, plan.desc.out_cs), dtype=torch.int32, device="cuda")
        got = hipq.from_device_nhwc(plan(xd, acc=acc), K)
        assert np.array_equal(acc.cpu().numpy()[..., :K].transpose(0, 3, 1, 2), want_acc), plan.kernel
        assert np.array_equal(got, want), (plan.kernel, int((got != want).sum()))
        assert np.array_equal(hipq.from_device_nhwc(plan(xd), K), want), plan.kernel  # without the dump
        assert len(np.unique(want)) > 8
        # run-time ReLU
        assert np.array_equal(hipq.from_device_nhwc(plan.run_relu(xd), K), np.maximum(want, ozp)), plan.kernel
        # K equal scales == the per-tensor plan
        same = np.full(K, wa[0], np.float32)
        p_same = hipq.Conv2d(x.shape, w, b, pad, st, grp, ia, izp, same, wzp, oa, ozp)
        p_tensor = hipq.Conv2d(x.shape, w, b, pad, st, grp, ia, izp, float(wa[0]), wzp, oa, ozp)
        assert torch.equal(p_same(xd)[..., :K], p_tensor(xd)[..., :K]), plan.kernel
        if grp == 1:  # fused residual add on a per-channel plan
            res = rng.integers(0, 256, want.shape, dtype=np.uint8)
            ra, rz, sa, sz = rand_q(rng, 1e-2, 1e-1), int(rng.integers(0, 256)), rand_q(rng, 3e-2, 3e-1), int(rng.integers(0, 256))
            yd = plan.run_add(xd, hipq.to_device_nhwc(res), False, ra, rz, sa, sz, plan.empty_output())
            assert np.array_equal(hipq.from_device_nhwc(yd, K), orc.add_u8(want, res, oa, ozp, ra, rz, sa, sz)), plan.kernel
    assert any("stream" in k for k in kerns) and any("depthwise3x3" in k for k in kerns) and any("_c4" in k for k in kerns), kerns
    assert "conv_depthwise_u8_perchannel" in kerns and "conv_direct_u8_perchannel" in kerns, kerns
    # int8 symmetric tensors
    x = rng.integers(-128, 128, (2, 64, 9, 9), dtype=np.int8)
    w = rng.integers(-128, 128, (80, 64, 3, 3), dtype=np.int8)
    b = rng.integers(-3000, 3000, 80).astype(np.int32)
    wa = np.exp(rng.uniform(np.log(1e-3), np.log(3e-2), 80)).astype(np.float32)
    _, acc8 = orc.conv2d_i8(x, w, b, 1, 1, 1, 0.02, float(wa[0]), 9.0, 7, return_acc=True)
    want8 = orc.requant_per_channel_i8(acc8, 0.02, wa, 9.0, 7)
    p8 = hipq.Conv2d(x.shape, w, b, 1, 1, 1, 0.02, 0, wa, 0, 9.0, 0, obits=7, dtype=hipq.DTYPE_I8)
    assert np.array_equal(hipq.from_device_nhwc(p8(hipq.to_device_nhwc(x)), 80).view(np.int8), want8), p8.kernel
    assert len(np.unique(want8)) > 8


def test_stem_convolution_with_fused_max_pooling():
    """hipq_conv2d_run_maxpool: the stem convolution (at most 4 input channels, stride 2) and the 3x3 / stride 2 / pad 1
    max pooling behind it in one kernel, against the oracle's convolution followed by the oracle's pooling: odd and even
    image sizes (ragged last row block, rows of fewer than 128 pixels), 7x7 / 6x6 / 5x5 kernels (a kernel row of 5 to 8 taps is one 32-byte k-step), 1 to 4 input channels,
    fewer than 64 output channels, ReLU folded into the convolution, shifts inside and outside the one-multiply form."""
    rng = np.random.default_rng(151)
    #        N  C   H    W   K  R pad relu
    cases = [(2, 3, 224, 224, 64, 7, 3, True), (3, 3, 64, 64, 64, 7, 3, False), (1, 4, 50, 36, 52, 5, 2, True),
             (2, 1, 37, 52, 64, 5, 1, False), (1, 3, 18, 20, 49, 7, 3, True), (1, 2, 9, 12, 64, 6, 0, False)]
    for N, C, H, W, K, R, pad, relu in cases:
        print("stem case", N, C, H, W, K, R, pad, relu, flush=True)
        x = rng.integers(0, 256, (N, C, H, W), dtype=np.uint8)
        w = rng.integers(0, 256, (K, C, R, R), dtype=np.uint8)
        b = rng.integers(-20000, 20000, K).astype(np.int32)
        ia, izp, wa = rand_q(rng), int(rng.integers(0, 256)), rand_q(rng)
        ozp = 0 if relu else int(rng.integers(0, 256))
        for oa in (float(np.float32(ia * wa * np.sqrt(C * R * R) * 60.0)), float(np.float32(ia * wa * 40.0))):
            q = (ia, izp, wa, 128, oa, ozp)
            conv = orc.conv2d_u8(x, w, b, pad, 2, 1, *q)
            if relu:
                conv = np.maximum(conv, ozp).astype(np.uint8)
            want = orc.pool_u8(conv, 3, 1, 2, 0, False, oa, ozp, oa, ozp)
            plan = hipq.Conv2d(x.shape, w, b, pad, 2, 1, *q, relu=relu)
            POH, POW = want.shape[2], want.shape[3]
            assert plan.maxpool_fusable(POH, POW, 3, 2, 1, oa, ozp, oa, ozp), plan.kernel
            assert not plan.maxpool_fusable(POH, POW, 3, 2, 1, oa, ozp, float(np.float32(oa * 1.5)), ozp)  # a real rescale
            assert not plan.maxpool_fusable(POH, POW, 2, 2, 0, oa, ozp, oa, ozp)                            # another window
            assert not plan.maxpool_fusable(POH + 1, POW, 3, 2, 1, oa, ozp, oa, ozp)                        # ceil_mode sizes
            yd = torch.full((N, POH, POW, 64), 7, dtype=torch.uint8, device="cuda")
            plan.run_maxpool(hipq.to_device_nhwc(x), yd)
            torch.cuda.synchronize()
            got = yd.cpu().numpy()[..., :K].transpose(0, 3, 1, 2)
            assert np.array_equal(got, want), (N, C, H, W, K, R, pad, relu, oa, int((got != want).sum()))
            # and the two operators run separately give the same bytes
            yc = plan(hipq.to_device_nhwc(x))
            yp = torch.empty((N, POH, POW, 64), dtype=torch.uint8, device="cuda")
            hipq.pool_u8(yc, yp, K, 3, 1, 2, 0, oa, ozp, oa, ozp)
            assert torch.equal(yp[..., :K], yd[..., :K])
            if not relu:  # the ReLU clamp asked for at run time (conv, relu, pool as three operators with equal scales)
                want_r = orc.pool_u8(orc.relu_u8(conv, oa, ozp, oa, ozp), 3, 1, 2, 0, False, oa, ozp, oa, ozp)
                plan.run_maxpool(hipq.to_device_nhwc(x), yd, relu=True)
                torch.cuda.synchronize()
                assert np.array_equal(yd.cpu().numpy()[..., :K].transpose(0, 3, 1, 2), want_r), (N, C, H, W, K, R, "relu at run time")
    # plans the kernel does not serve refuse
    p64 = hipq.Conv2d((1, 64, 8, 8), np.zeros((64, 64, 3, 3), np.uint8), None, 1, 2, 1, 0.1, 0, 0.1, 128, 0.1, 0)
    assert not p64.maxpool_fusable(2, 2, 3, 2, 1, 0.1, 0, 0.1, 0)
    with pytest.raises(hipq.HipqError):
        p64.run_maxpool(torch.zeros((1, 8, 8, 64), dtype=torch.uint8, device="cuda"), torch.zeros((1, 2, 2, 64), dtype=torch.uint8, device="cuda"))
    s1 = hipq.Conv2d((1, 3, 16, 16), np.zeros((64, 3, 3, 3), np.uint8), None, 1, 1, 1, 0.1, 0, 0.1, 128, 0.1, 0)  # stride 1
    assert not s1.maxpool_fusable(8, 8, 3, 2, 1, 0.1, 0, 0.1, 0)


def test_stem_with_pooling_and_the_next_convolution():
    """hipq_conv2d_run_maxpool_conv: stem convolution, max pooling and the 1x1 convolution (64 -> 64) that reads the pooled
    tensor in one kernel, against the oracle's three operators: pooled rows of 56, 16 and 9 pixels (two, one and a
    ragged pixel tile), a ragged last row block, with and without ReLU on either convolution; the pooled tensor is
    written as well; a second chained layer (64 -> 256); plans that do not chain refuse."""
    rng = np.random.default_rng(152)
    #        N  C   H    W   R pad relu relu_next
    cases = [(2, 3, 224, 224, 7, 3, True, True), (3, 3, 64, 64, 7, 3, False, False), (1, 4, 50, 36, 5, 2, True, False),
             (2, 3, 130, 100, 7, 3, False, True)]
    for N, C, H, W, R, pad, relu, relu_next in cases:
        print("stem chain case", N, C, H, W, R, pad, relu, relu_next, flush=True)
        x = rng.integers(0, 256, (N, C, H, W), dtype=np.uint8)
        w = rng.integers(0, 256, (64, C, R, R), dtype=np.uint8)
        b = rng.integers(-20000, 20000, 64).astype(np.int32)
        ia, izp, wa = rand_q(rng), int(rng.integers(0, 256)), rand_q(rng)
        ozp = 0 if relu else int(rng.integers(0, 256))
        oa = float(np.float32(ia * wa * np.sqrt(C * R * R) * 60.0))
        q = (ia, izp, wa, 128, oa, ozp)
        conv = orc.conv2d_u8(x, w, b, pad, 2, 1, *q)
        if relu:
            conv = np.maximum(conv, ozp).astype(np.uint8)
        pooled = orc.pool_u8(conv, 3, 1, 2, 0, False, oa, ozp, oa, ozp)
        w2 = rng.integers(0, 256, (64, 64, 1, 1), dtype=np.uint8)
        b2 = rng.integers(-20000, 20000, 64).astype(np.int32)
        wa2, oz2 = rand_q(rng), (0 if relu_next else int(rng.integers(0, 256)))
        oa2 = float(np.float32(oa * wa2 * 8.0 * 60.0))
        q2 = (oa, ozp, wa2, 128, oa2, oz2)
        want2 = orc.conv2d_u8(pooled, w2, b2, 0, 1, 1, *q2)
        if relu_next:
            want2 = np.maximum(want2, oz2).astype(np.uint8)
        assert len(np.unique(want2)) > 8
        plan = hipq.Conv2d(x.shape, w, b, pad, 2, 1, *q, relu=relu)
        nxt = hipq.Conv2d(pooled.shape, w2, b2, 0, 1, 1, *q2, relu=relu_next)
        POH, POW = pooled.shape[2], pooled.shape[3]
        assert plan.maxpool_conv_fusable(POH, POW, nxt), (plan.kernel, nxt.kernel)
        yd = torch.full((N, POH, POW, 64), 7, dtype=torch.uint8, device="cuda")
        y2 = torch.full((N, POH, POW, 64), 9, dtype=torch.uint8, device="cuda")
        plan.run_maxpool_conv(hipq.to_device_nhwc(x), yd, nxt, y2)
        torch.cuda.synchronize()
        assert np.array_equal(yd.cpu().numpy().transpose(0, 3, 1, 2), pooled), (N, C, H, W, "pooled tensor")
        got2 = y2.cpu().numpy().transpose(0, 3, 1, 2)
        assert np.array_equal(got2, want2), (N, C, H, W, R, int((got2 != want2).sum()), np.argwhere(got2 != want2)[:6].tolist())
        # a next layer that reads another scale, or is no 64 -> 64 1x1 layer, does not chain
        other = hipq.Conv2d(pooled.shape, w2, b2, 0, 1, 1, float(np.float32(oa * 1.25)), ozp, wa2, 128, oa2, oz2)
        assert not plan.maxpool_conv_fusable(POH, POW, other)
        with pytest.raises(hipq.HipqError, match="do not run as one kernel"):
            plan.run_maxpool_conv(hipq.to_device_nhwc(x), yd, other, y2)
        odd = hipq.Conv2d(pooled.shape, rng.integers(0, 256, (96, 64, 1, 1), dtype=np.uint8), None, 0, 1, 1, *q2)
        assert not plan.maxpool_conv_fusable(POH, POW, odd)
        # two chained layers: 64 -> 64 and 64 -> 256 (a block's first layer and its projection shortcut)
        w3 = rng.integers(0, 256, (256, 64, 1, 1), dtype=np.uint8)
        b3 = rng.integers(-20000, 20000, 256).astype(np.int32)
        wa3, oz3 = rand_q(rng), int(rng.integers(0, 256))
        q3 = (oa, ozp, wa3, 128, float(np.float32(oa * wa3 * 8.0 * 60.0)), oz3)
        want3 = orc.conv2d_u8(pooled, w3, b3, 0, 1, 1, *q3)
        sc = hipq.Conv2d(pooled.shape, w3, b3, 0, 1, 1, *q3)
        assert plan.maxpool_conv_fusable(POH, POW, nxt, sc), (plan.kernel, nxt.kernel, sc.kernel)
        yd.fill_(7), y2.fill_(9)
        y3 = torch.full((N, POH, POW, 256), 11, dtype=torch.uint8, device="cuda")
        plan.run_maxpool_conv(hipq.to_device_nhwc(x), yd, nxt, y2, nxt2=sc, y_next2=y3)
        torch.cuda.synchronize()
        assert np.array_equal(yd.cpu().numpy().transpose(0, 3, 1, 2), pooled), (N, C, H, W, "pooled tensor, two layers")
        assert np.array_equal(y2.cpu().numpy().transpose(0, 3, 1, 2), want2), (N, C, H, W, "first chained layer of two")
        got3 = y3.cpu().numpy().transpose(0, 3, 1, 2)
        assert np.array_equal(got3, want3), (N, C, H, W, int((got3 != want3).sum()), np.argwhere(got3 != want3)[:6].tolist())
        big = hipq.Conv2d(pooled.shape, rng.integers(0, 256, (320, 64, 1, 1), dtype=np.uint8), None, 0, 1, 1, *q3)
        assert plan.maxpool_conv_fusable(POH, POW, big) and not plan.maxpool_conv_fusable(POH, POW, nxt, big)  # 384 channels


def test_elementwise():
    rng = np.random.default_rng(15)
    for n in (1, 15, 16, 4099, 64 * 56 * 56 * 16 + 3):
        a = rng.integers(0, 256, n, dtype=np.uint8)
        b = rng.integers(0, 256, n, dtype=np.uint8)
        c = rng.integers(0, 256, n, dtype=np.uint8)
        ia = [rand_q(rng) for _ in range(3)]
        iz = [int(rng.integers(0, 256)) for _ in range(3)]
        oa, oz = rand_q(rng, 3e-3, 0.3), int(rng.integers(0, 256))
        ta, tb, tc = (torch.from_numpy(v).cuda() for v in (a, b, c))
        ty = torch.empty_like(ta)
        got = hipq.add_u8(ta, tb, ty, ia[0], iz[0], ia[1], iz[1], oa, oz).cpu().numpy()
        assert np.array_equal(got, orc.add_u8(a, b, ia[0], iz[0], ia[1], iz[1], oa, oz)), ("add", n)
        for operation in (1, 2):
            got = hipq.eltwise_u8([ta, tb, tc], ty, ia, iz, oa, oz, operation).cpu().numpy()
            assert np.array_equal(got, orc.eltwise_u8([a, b, c], ia, iz, oa, oz, operation)), ("eltwise", n, operation)
        got = hipq.eltwise_u8([ta, tb], ty, ia[:2], iz[:2], oa, oz, 1, coeff=[0.5, 1.75]).cpu().numpy()
        assert np.array_equal(got, orc.eltwise_u8([a, b], ia[:2], iz[:2], oa, oz, 1, coeff=[0.5, 1.75]))
        got = hipq.relu_u8(ta, ty, ia[0], iz[0], oa, oz).cpu().numpy()
        assert np.array_equal(got, orc.relu_u8(a, ia[0], iz[0], oa, oz)), ("relu", n)
        # very unequal scales: shifts beyond the 32-bit forms of add / eltwise (64-bit path), and 4 / 6 inputs
        wide = [ia[0], float(np.float32(ia[0] * 3.0e-4)), float(np.float32(ia[0] * 40.0))]
        got = hipq.add_u8(ta, tb, ty, wide[0], iz[0], wide[1], iz[1], wide[0], oz).cpu().numpy()
        assert np.array_equal(got, orc.add_u8(a, b, wide[0], iz[0], wide[1], iz[1], wide[0], oz)), ("add wide", n)
        got = hipq.eltwise_u8([ta, tb, tc], ty, wide, iz, wide[0], oz, 1).cpu().numpy()
        assert np.array_equal(got, orc.eltwise_u8([a, b, c], wide, iz, wide[0], oz, 1)), ("eltwise wide", n)
        for k in (4, 6):
            ins = [a, b, c, a[::-1].copy(), b[::-1].copy(), c[::-1].copy()][:k]
            tins = [torch.from_numpy(v).cuda() for v in ins]
            iak, izk = (ia * 2)[:k], (iz * 2)[:k]
            for operation in (1, 2):
                got = hipq.eltwise_u8(tins, ty, iak, izk, oa, oz, operation).cpu().numpy()
                assert np.array_equal(got, orc.eltwise_u8(ins, iak, izk, oa, oz, operation)), ("eltwise", k, n, operation)


def test_pool():
    rng = np.random.default_rng(16)
    cases = [(2, 64, 112, 112, 3, 1, 2, 0, False), (2, 64, 13, 13, 3, 1, 2, 0, True), (3, 40, 7, 7, 7, 0, 1, 1, True),
             (1, 20, 9, 11, 3, 1, 2, 1, True), (1, 3, 8, 8, 2, 0, 2, 1, False), (2, 17, 10, 10, (3, 2), (1, 0), (2, 1), 1, True),
             # global average windows: the one-work-group-per-image kernel, its 1024-pixel limit and the generic fallback
             (5, 2048, 7, 7, 7, 0, 1, 1, False), (2, 1280, 7, 7, 7, 0, 7, 1, True), (2, 200, 32, 32, 32, 0, 1, 1, False),
             (1, 16, 33, 33, 33, 0, 1, 1, False), (2, 1040, 5, 3, (5, 3), 0, 1, 1, False)]
    for N, C, H, W, k, pad, st, method, ceil_mode in cases:
        x = rng.integers(0, 256, (N, C, H, W), dtype=np.uint8)
        q = (rand_q(rng), int(rng.integers(0, 256)), rand_q(rng), int(rng.integers(0, 256)))
        want = orc.pool_u8(x, k, pad, st, method, ceil_mode, *q)
        xd = hipq.to_device_nhwc(x)
        yd = torch.empty((N, want.shape[2], want.shape[3], xd.shape[3]), dtype=torch.uint8, device="cuda")
        hipq.pool_u8(xd, yd, C, k, pad, st, method, *q)
        assert np.array_equal(hipq.from_device_nhwc(yd, C), want), (N, C, H, W, k, pad, st, method)


def test_quantize_dequantize():
    rng = np.random.default_rng(17)
    for shape in ((2, 3, 224, 224), (1, 16, 9, 9), (4, 1000, 1, 1)):
        oa, oz = rand_q(rng, 5e-3, 0.1), int(rng.integers(0, 256))
        x = (rng.standard_normal(shape) * 60 * oa).astype(np.float32)
        x.flat[:512] = (np.arange(512, dtype=np.float32) * 0.5 - oz) * np.float32(oa)  # exact ties, both clamps
        xd = torch.from_numpy(x).cuda()
        cs = hipq.channel_stride(shape[1])
        yd = torch.empty((shape[0], shape[2], shape[3], cs), dtype=torch.uint8, device="cuda")
        hipq.quantize_u8(xd, yd, oa, oz)
        want = orc.quantize_u8(x, oa, oz)
        got = hipq.from_device_nhwc(yd, shape[1])
        assert np.array_equal(got, want), (shape, int((got != want).sum()))
        fd = torch.empty(shape, dtype=torch.float32, device="cuda")
        hipq.dequantize_u8(yd, fd, oa, oz)
        assert np.array_equal(fd.cpu().numpy().view(np.uint32), orc.dequantize_u8(want, oa, oz).view(np.uint32))


def test_dequantize_of_int32_accumulators():
    """hipq_dequantize_i32 (no counterpart in the reference, which dequantizes bytes only): a convolution's accumulator
    dump times ialpha * walpha, against the oracle's closed form, plus values where int32 -> fp32 rounds."""
    rng = np.random.default_rng(18)
    x = rng.integers(0, 256, (2, 48, 9, 7), dtype=np.uint8)
    w = rng.integers(0, 256, (40, 48, 3, 3), dtype=np.uint8)
    b = rng.integers(-30000, 30000, 40).astype(np.int32)
    q = (0.02, 128, 0.005, 128, 0.05, 0)
    plan = hipq.Conv2d(x.shape, w, b, 1, 1, 1, *q)
    acc = torch.zeros((2, 9, 7, plan.desc.out_cs), dtype=torch.int32, device="cuda")
    plan(hipq.to_device_nhwc(x), acc=acc)
    _, want_acc = orc.conv2d_u8(x, w, b, 1, 1, 1, *q, return_acc=True)
    alpha = float(np.float32(q[0]) * np.float32(q[2]))
    fd = torch.empty((2, 40, 9, 7), dtype=torch.float32, device="cuda")
    hipq.dequantize_i32(acc, fd, alpha)
    assert np.array_equal(fd.cpu().numpy().view(np.uint32), orc.dequantize_i32(want_acc, alpha).view(np.uint32))
    big = np.concatenate([rng.integers(-2**31, 2**31, 4086), [2**24 + 1, 2**24 + 3, -(2**24) - 1, 2**31 - 1, -2**31, 0, 1, -1, 2**25 + 2,
                                                                2**25 + 6]]).astype(np.int32).reshape(1, 4096, 1, 1)
    bd = torch.from_numpy(big.reshape(1, 1, 1, 4096)).cuda()
    fd = torch.empty((1, 4096, 1, 1), dtype=torch.float32, device="cuda")
    hipq.dequantize_i32(bd, fd, 3.1e-5)
    assert np.array_equal(fd.cpu().numpy().view(np.uint32), orc.dequantize_i32(big, 3.1e-5).view(np.uint32))


def test_quantize_division_free_form_is_exact():
    """quantize_u8 divides by multiplying with the correctly rounded reciprocal and two FMA corrections, clamps before
    the division and rounds without the reference's double: checked against the reference arithmetic on the values where
    such shortcuts would show - the fp32 neighbours (five ulps either side) of every rounding boundary (k + 0.5) * alpha
    and of both clamps, zeros, subnormals, huge values, infinities and NaN, random bit patterns - for scales that are and
    are not powers of two, including ones whose reciprocal rounds awkwardly, and for fewer output bits."""
    rng = np.random.default_rng(171)
    scales = [0.0078125, 0.1, 1.0 / 3.0, 0.05, 0.007843137718737125, 1.9999998807907104, 1.0000001192092896, 3.0e-5,
              float(np.float32(1.0) / np.float32(255.0)), 123.456] + [rand_q(rng, 1e-4, 10.0) for _ in range(6)]
    for i, oa in enumerate(scales):
        oa = float(np.float32(oa))
        for oz, obits in ((0, 8), (128, 8), (255, 8), (int(rng.integers(0, 128)), 7), (3, 4)):
            hi = (1 << obits) - 1
            k = np.arange(-3, hi + 4, dtype=np.float64)
            centres = np.concatenate([(k + 0.5 - oz) * oa, (k - oz) * oa]).astype(np.float32)
            near = centres.view(np.int32)[:, None] + np.arange(-5, 6, dtype=np.int32)[None, :]
            special = np.array([0.0, -0.0, 1e-45, -1e-45, 1e-38, -1e-38, 3e38, -3e38, np.inf, -np.inf, np.nan, 65504.0, -65504.0],
                               np.float32)
            rnd = rng.integers(0, 1 << 32, 200000, dtype=np.uint64).astype(np.uint32).view(np.float32)
            norm = (rng.standard_normal(200000) * 80 * oa).astype(np.float32)
            x = np.concatenate([near.reshape(-1).view(np.float32), special, rnd, norm]).astype(np.float32)
            x = np.concatenate([x, np.zeros((-x.size) % 4, np.float32)]).reshape(1, 1, -1, 4)
            with np.errstate(all="ignore"):
                want = orc.quantize_u8(x, oa, oz, obits)
            xd = torch.from_numpy(x).cuda()
            yd = torch.empty((1, x.shape[2], 4, 4), dtype=torch.uint8, device="cuda")
            hipq.quantize_u8(xd, yd, oa, oz, obits)
            got = hipq.from_device_nhwc(yd, 1)
            bad = np.flatnonzero(got.reshape(-1) != want.reshape(-1))
            assert bad.size == 0, (oa, oz, obits, bad.size, x.reshape(-1)[bad[:5]], got.reshape(-1)[bad[:5]], want.reshape(-1)[bad[:5]])
    with pytest.raises(hipq.HipqError, match="scale"):
        hipq.quantize_u8(xd, yd, -0.5, 0)


def test_layout_round_trip_and_errors():
    rng = np.random.default_rng(18)
    x = rng.integers(0, 256, (2, 19, 5, 7), dtype=np.uint8)
    assert np.array_equal(hipq.from_device_nhwc(hipq.to_device_nhwc(x), 19), x)
    # error behaviour: a bad descriptor is refused with a message, nothing is launched
    with pytest.raises(hipq.HipqError, match="group"):
        hipq.Conv2d((1, 6, 4, 4), np.zeros((4, 2, 1, 1), np.uint8), None, 0, 1, 4, 0.1, 0, 0.1, 0, 0.1, 0)
    with pytest.raises(hipq.HipqError, match="shift"):
        hipq.Conv2d((1, 16, 4, 4), np.zeros((16, 16, 1, 1), np.uint8), None, 0, 1, 1, 1e4, 0, 1e4, 0, 1e-4, 0)


def test_full_size_properties():
    """BASELINE-size checks that do not need the slow CPU oracle on the full tensor: linearity in the
    bias (a per-channel constant shift of the accumulators) and batch independence at N = 64."""
    rng = np.random.default_rng(19)
    N, C, H, K = 64, 64, 56, 64
    x = rng.integers(0, 256, (N, C, H, H), dtype=np.uint8)
    w = rng.integers(1, 256, (K, C, 3, 3), dtype=np.uint8)
    b = rng.integers(-1000, 1000, K).astype(np.int32)
    q = (0.02, 128, 0.005, 128, 0.05, 0)
    y, acc, _ = run_conv(x, w, b, 1, 1, 1, q)
    y0, acc0, _ = run_conv(x, w, None, 1, 1, 1, q)
    assert np.array_equal(acc - acc0, np.broadcast_to(b[None, :, None, None], acc.shape))
    # images 0 and 63 alone give the same bytes as inside the batch, and match the oracle
    for i in (0, 63):
        want = orc.conv2d_u8(x[i:i + 1], w, b, 1, 1, 1, *q)
        assert np.array_equal(y[i:i + 1], want)


def test_conv_plan_variants_are_bit_identical():
    """hipq_conv2d_plan_select: every work-group tile and stage count of the MFMA kernel gives the bytes of the
    built-in choice, with and without the fused residual add; plans without variants refuse."""
    rng = np.random.default_rng(45)
    shapes = [(2, 64, 14, 14, 64, 3, 1, 1), (1, 128, 9, 11, 256, 1, 0, 1), (3, 64, 10, 7, 48, 3, 1, 2), (1, 256, 12, 12, 128, 3, 1, 1),
              (2, 1024, 7, 7, 256, 1, 0, 1), (1, 192, 20, 20, 320, 1, 0, 1),
              # 1x1 kernels whose channel stride is not a multiple of 64: partial last slab
              (2, 96, 9, 9, 24, 1, 0, 1), (1, 16, 12, 12, 96, 1, 0, 1), (1, 144, 7, 7, 32, 1, 0, 1), (3, 160, 5, 5, 320, 1, 0, 1),
              (1, 32, 10, 10, 192, 1, 0, 2), (1, 20, 6, 6, 16, 1, 0, 1),
              # the pointwise kernel: ragged strips, 1 and 2 k-steps, partial channel blocks, the widest output
              (3, 64, 7, 9, 256, 1, 0, 1), (1, 48, 5, 5, 40, 1, 0, 1), (2, 8, 3, 11, 16, 1, 0, 1), (1, 64, 33, 31, 64, 1, 0, 1),
              # four output channels or fewer: a 4-byte channel stride, which the pointwise kernel's 16-byte stores must not get
              (2, 32, 9, 9, 3, 1, 0, 1), (1, 17, 6, 5, 1, 1, 0, 1)]
    for N, C, H, W, K, R, pad, st in shapes:
        x = rng.integers(0, 256, (N, C, H, W), dtype=np.uint8)
        w = rng.integers(0, 256, (K, C, R, R), dtype=np.uint8)
        b = rng.integers(-30000, 30000, K).astype(np.int32)
        q = (rand_q(rng), int(rng.integers(0, 256)), rand_q(rng), 128, rand_q(rng, 1e-2, 1.0), int(rng.integers(0, 256)))
        want = orc.conv2d_u8(x, w, b, pad, st, 1, *q)
        plan = hipq.Conv2d(x.shape, w, b, pad, st, 1, *q)
        xd = hipq.to_device_nhwc(x)
        res = rng.integers(0, 256, want.shape, dtype=np.uint8)
        rd = hipq.to_device_nhwc(res)
        want_add = orc.add_u8(want, res, q[4], q[5], 0.07, 33, 0.1, 5)
        assert not (K <= 4 and "pointwise" in plan.kernel), plan.kernel
        if plan.kernel.endswith("pointwise"):  # small 1x1 layers: the pointwise kernel first, then the tile kernels
            assert R == 1 and C <= 64 and K <= 256, plan.kernel
            assert np.array_equal(hipq.from_device_nhwc(plan(xd), K), want), (x.shape, w.shape, plan.kernel)
            if K % 16 == 0:
                zd = plan.empty_output()
                plan.run_add(xd, rd, False, 0.07, 33, 0.1, 5, zd)
                assert np.array_equal(hipq.from_device_nhwc(zd, K), want_add), ("add", x.shape, plan.kernel)
                plan.run_add(xd, rd, True, 0.07, 33, 0.1, 5, zd)
                assert np.array_equal(hipq.from_device_nhwc(zd, K), orc.add_u8(res, want, 0.07, 33, q[4], q[5], 0.1, 5)), ("add first", x.shape)
            plan.special(0)
            assert not plan.kernel.endswith("pointwise")
        for tile in (0, 1, 2, 3, 4):
            for stages in (0, 2, 3, 4, 8):
                plan.select(tile, stages)
                yd = plan(xd)
                assert np.array_equal(hipq.from_device_nhwc(yd, K), want), (x.shape, w.shape, tile, stages, plan.kernel)
                if K % 16 == 0:
                    zd = torch.empty_like(yd)
                    plan.run_add(xd, rd, False, 0.07, 33, 0.1, 5, zd)
                    assert np.array_equal(hipq.from_device_nhwc(zd, K), want_add), ("add", x.shape, tile, stages, plan.kernel)
    dw = hipq.Conv2d((1, 32, 8, 8), rng.integers(0, 256, (32, 1, 3, 3), dtype=np.uint8), None, 1, 1, 32, 0.1, 3, 0.1, 128, 0.1, 0)
    with pytest.raises(hipq.HipqError):
        dw.select(0, 2)
    with pytest.raises(hipq.HipqError):
        plan.select(7, 2)
    with pytest.raises(hipq.HipqError):
        plan.select(0, 5)


def test_relu_decided_at_run_time():
    """hipq_conv2d_run_relu on a plan created without relu == a plan created with relu == convolution, then the relu
    operator with the convolution's output scale on both sides; every kernel family, obits below 8 included."""
    rng = np.random.default_rng(47)
    kerns = set()
    #         N, C,  H,  W,  K,  R, pad, stride, group
    shapes = [(2, 64, 12, 12, 64, 3, 1, 1, 1), (1, 64, 9, 9, 48, 3, 1, 1, 1), (1, 32, 9, 9, 96, 1, 0, 1, 1), (2, 256, 7, 7, 128, 1, 0, 1, 1), (1, 3, 20, 20, 32, 3, 1, 2, 1),
              (1, 3, 20, 20, 32, 3, 1, 1, 1),
              (2, 48, 10, 10, 48, 3, 1, 1, 48), (1, 32, 9, 9, 32, 3, 1, 2, 32), (1, 24, 7, 7, 24, 5, 2, 1, 24), (1, 16, 8, 8, 32, 3, 1, 1, 4)]
    for N, C, H, W, K, R, pad, st, g in shapes:
        x = rng.integers(0, 256, (N, C, H, W), dtype=np.uint8)
        w = rng.integers(0, 256, (K, C // g, R, R), dtype=np.uint8)
        b = rng.integers(-20000, 20000, K).astype(np.int32)
        for obits, ozp in ((8, 40), (8, 0), (7, 100), (4, 200)):
            q = (rand_q(rng), int(rng.integers(0, 256)), rand_q(rng), 128, rand_q(rng, 1e-2, 0.5), ozp)
            plain = hipq.Conv2d(x.shape, w, b, pad, st, g, *q, obits=obits)
            fused = hipq.Conv2d(x.shape, w, b, pad, st, g, *q, obits=obits, relu=True)
            kerns.add(plain.kernel)
            xd = hipq.to_device_nhwc(x)
            want = orc.relu_u8(orc.conv2d_u8(x, w, b, pad, st, g, *q, obits=obits), q[4], ozp, q[4], ozp, obits)
            assert np.array_equal(hipq.from_device_nhwc(plain.run_relu(xd), K), want), (plain.kernel, obits, ozp)
            assert np.array_equal(hipq.from_device_nhwc(fused(xd), K), want), (fused.kernel, obits, ozp)
    assert any("halo" in k for k in kerns) and any("pointwise" in k for k in kerns) and any("_c4" in k for k in kerns)
    assert any("stem3x3" in k for k in kerns)
    assert any("depthwise3x3" in k for k in kerns) and "conv_depthwise_u8" in kerns and "conv_direct_u8" in kerns
    p8 = hipq.Conv2d((1, 16, 4, 4), rng.integers(-128, 128, (16, 16, 1, 1), dtype=np.int8), None, 0, 1, 1, 0.1, 0, 0.1, 0, 0.1, 0,
                     dtype=hipq.DTYPE_I8)
    with pytest.raises(hipq.HipqError, match="uint8 plans only"):
        p8.run_relu(hipq.to_device_nhwc(np.zeros((1, 16, 4, 4), np.int8)))


def test_conv3x3_rows_kernel():
    """conv3x3_c64_rows_kernel (3x3 / stride 1 / pad 1, 64 channels in, 49 to 64 out, images up to 64 pixels wide; input
    rows resident in LDS, weights in registers) against the oracle and against the tile kernels: widths that are and
    are not multiples of 16 and 32 (the pad pixel right of a row comes with the row's loads), one-pixel and one-row
    images, row blocks that do not divide the height, several images, ReLU, fewer output bits, int8 tensors."""
    rng = np.random.default_rng(47)
    shapes = [(2, 56, 56, 64), (1, 9, 64, 64), (3, 17, 63, 52), (1, 1, 1, 64), (2, 5, 32, 49), (1, 30, 16, 64), (4, 3, 33, 60),
              (1, 64, 48, 64), (64, 8, 8, 64),
              # batches large enough for the host to give a work-group 3, 4 and 6 output rows (5, 6 and 8 input rows: the
              # rows behind the first four arrive after the weights have passed through their space)
              (40, 28, 20, 64), (64, 28, 8, 64), (96, 27, 12, 56)]
    for i, (N, H, W, K) in enumerate(shapes):
        print("rows case", N, H, W, K, flush=True)
        x = rng.integers(0, 256, (N, 64, H, W), dtype=np.uint8)
        w = rng.integers(0, 256, (K, 64, 3, 3), dtype=np.uint8)
        b = rng.integers(-30000, 30000, K).astype(np.int32)
        ia, wa = rand_q(rng), rand_q(rng)
        relu, obits = bool(i & 1), (8, 8, 7)[i % 3]
        q = (ia, int(rng.integers(0, 256)), wa, 128, float(np.float32(ia * wa * 24.0 * 40.0)), int(rng.integers(0, 1 << obits)))
        want = orc.conv2d_u8(x, w, b, 1, 1, 1, *q, obits=obits)
        if relu:
            want = orc.relu_u8(want, q[4], q[5], q[4], q[5], obits)
        plan = hipq.Conv2d(x.shape, w, b, 1, 1, 1, *q, relu=relu, obits=obits)
        assert plan.kernel == "conv_mfma_i8_rows3x3", plan.kernel
        xd = hipq.to_device_nhwc(x)
        got = hipq.from_device_nhwc(plan(xd), K)
        assert np.array_equal(got, want), (N, H, W, K, relu, obits, int((got != want).sum()))
        # the residual add fused into the same kernel, both operand orders, scale ratios that do and do not fit the
        # add's 32-bit form
        res = rng.integers(0, 1 << obits, want.shape, dtype=np.uint8)
        rd = hipq.to_device_nhwc(res)
        ra, rz = float(np.float32(q[4] * (1.0, 1.7, 300.0)[i % 3])), int(rng.integers(0, 256))
        sa, sz = float(np.float32(max(q[4], ra) * 1.3)), int(rng.integers(0, 1 << obits))
        assert plan.kernel_add == "conv_mfma_i8_rows3x3+add", plan.kernel_add
        for res_first in (False, True):
            want_sum = (orc.add_u8(res, want, ra, rz, q[4], q[5], sa, sz, obits) if res_first
                        else orc.add_u8(want, res, q[4], q[5], ra, rz, sa, sz, obits))
            y = plan.empty_output()
            plan.run_add(xd, rd, res_first, ra, rz, sa, sz, y, obits=obits)
            got = hipq.from_device_nhwc(y, K)
            assert np.array_equal(got, want_sum), (N, H, W, K, relu, obits, res_first, int((got != want_sum).sum()))
        plan.special(0)
        assert "rows3x3" not in plan.kernel and "rows3x3" not in plan.kernel_add
        assert np.array_equal(hipq.from_device_nhwc(plan(xd), K), want)
        y = plan.empty_output()
        plan.run_add(xd, rd, True, ra, rz, sa, sz, y, obits=obits)
        assert np.array_equal(hipq.from_device_nhwc(y, K), want_sum), (N, H, W, K, "tile kernel with the add")
    x = rng.integers(-128, 128, (2, 64, 20, 24), dtype=np.int8)
    w = rng.integers(-127, 128, (64, 64, 3, 3), dtype=np.int8)
    b = rng.integers(-30000, 30000, 64).astype(np.int32)
    for obits in (8, 7):
        plan = hipq.Conv2d(x.shape, w, b, 1, 1, 1, 0.02, 0, 0.004, 0, 2.0, 0, obits=obits, dtype=hipq.DTYPE_I8)
        assert plan.kernel == "conv_mfma_i8_rows3x3_signed", plan.kernel
        got = hipq.from_device_nhwc(plan(hipq.to_device_nhwc(x)), 64).view(np.int8)
        assert np.array_equal(got, orc.conv2d_i8(x, w, b, 1, 1, 1, 0.02, 0.004, 2.0, obits=obits)), obits


def test_stem3x3_stride2_kernel():
    """conv_stem3x3_kernel (3x3 / stride 2 from an image with at most 4 channels to at most 32; input rows resident in
    LDS, two multiplies per 32 pixels x 32 channels) against the oracle and against the tile kernel: with and without
    padding, odd and even heights, rows shorter than / equal to / a ragged multiple of a wave's 32 pixels, 1 to 3 input
    channels, 17 to 32 output channels, row blocks that do not divide the height, ReLU, fewer output bits, a
    scale that takes the 64-bit requantisation; the accumulator dump falls back to the tile kernel."""
    rng = np.random.default_rng(53)
    shapes = [(2, 3, 224, 224, 32, 1), (1, 3, 32, 32, 32, 1), (3, 3, 31, 44, 24, 1), (1, 1, 9, 12, 32, 0), (2, 2, 65, 248, 17, 1),
              (1, 3, 3, 4, 32, 1), (5, 3, 30, 132, 32, 0), (64, 3, 48, 40, 32, 1), (1, 4, 20, 200, 20, 1)]
    for i, (N, C, H, W, K, pad) in enumerate(shapes):
        print("stem3x3 case", N, C, H, W, K, pad, flush=True)
        x = rng.integers(0, 256, (N, C, H, W), dtype=np.uint8)
        w = rng.integers(0, 256, (K, C, 3, 3), dtype=np.uint8)
        b = rng.integers(-3000, 3000, K).astype(np.int32)
        ia, wa = rand_q(rng), rand_q(rng)
        relu, obits = bool(i & 1), (8, 8, 7)[i % 3]
        # requantisation shifts below 33 (the 64-bit form), in the one-multiply range, and far up in it
        oa = float(np.float32(ia * wa * (200.0, 2000.0, 3e6)[i % 3]))
        q = (ia, int(rng.integers(0, 256)), wa, 128, oa, int(rng.integers(0, 1 << obits)))
        want = orc.conv2d_u8(x, w, b, pad, 2, 1, *q, obits=obits)
        if relu:
            want = orc.relu_u8(want, q[4], q[5], q[4], q[5], obits)
        plan = hipq.Conv2d(x.shape, w, b, pad, 2, 1, *q, relu=relu, obits=obits)
        assert plan.kernel == "conv_mfma_i8_stem3x3", plan.kernel
        xd = hipq.to_device_nhwc(x)
        got = hipq.from_device_nhwc(plan(xd), K)
        assert np.array_equal(got, want), (N, C, H, W, K, pad, relu, obits, int((got != want).sum()))
        plan.special(0)
        assert "stem3x3" not in plan.kernel
        assert np.array_equal(hipq.from_device_nhwc(plan(xd), K), want)
    # the accumulators come from the tile kernel (this kernel never writes them); bytes and sums both match
    x = rng.integers(0, 256, (2, 3, 40, 40), dtype=np.uint8)
    w = rng.integers(0, 256, (32, 3, 3, 3), dtype=np.uint8)
    b = rng.integers(-3000, 3000, 32).astype(np.int32)
    check_conv(x, w, b, 1, 2, 1, (0.02, 7, 0.004, 128, 0.5, 3), "stem3x3 shape with accumulators")
    # a weight zero point other than 128 stays with the tile kernel
    plan = hipq.Conv2d(x.shape, w, b, 1, 2, 1, 0.02, 7, 0.004, 120, 0.5, 3)
    assert "stem3x3" not in plan.kernel


def test_conv3x3_halo_kernel_matches_the_streaming_kernel_and_the_oracle():
    """3x3 / stride 1 / pad 1 layers load a pixel tile with its halo once and read the nine taps from LDS: every tile
    shape, one and several channel slabs, images narrower and wider than a tile, several images per tile (taps must
    not leak across image or row borders), ragged last tiles, int8 tensors."""
    rng = np.random.default_rng(46)
    shapes = [(2, 64, 56, 56, 64), (3, 64, 5, 7, 48), (1, 128, 28, 28, 128), (5, 192, 3, 3, 80), (2, 256, 14, 14, 256), (7, 64, 1, 1, 16),
              (1, 64, 2, 63, 64), (4, 512, 7, 7, 512), (3, 128, 9, 31, 200), (1, 64, 40, 62, 32), (1, 128, 6, 32, 64)]
    for N, C, H, W, K in shapes:
        print("halo case", N, C, H, W, K, flush=True)
        x = rng.integers(0, 256, (N, C, H, W), dtype=np.uint8)
        w = rng.integers(0, 256, (K, C, 3, 3), dtype=np.uint8)
        b = rng.integers(-30000, 30000, K).astype(np.int32)
        q = (rand_q(rng), int(rng.integers(0, 256)), rand_q(rng), 128, rand_q(rng, 1e-2, 1.0), int(rng.integers(0, 256)))
        want, want_acc = orc.conv2d_u8(x, w, b, 1, 1, 1, *q, return_acc=True)
        plan = hipq.Conv2d(x.shape, w, b, 1, 1, 1, *q)
        # the built-in rule: single channel slab only (64 output channels with a one-multiply requantisation: the rows kernel)
        assert (plan.kernel.endswith("_halo") or "rows3x3" in plan.kernel) == (C == 64), plan.kernel
        plan.special(2)
        xd = hipq.to_device_nhwc(x)
        for tile in (0, 2, 3, 4):
            plan.select(tile, 0)
            # one channel slab: every tile; 2, 4 or 8 slabs: the 128-channel tiles, images up to 31 pixels wide
            applies = C == 64 or (C in (128, 256, 512) and tile in (0, 3) and W <= 31)
            assert plan.kernel.endswith("_halo") == applies, (plan.kernel, x.shape, tile)
            assert np.array_equal(hipq.from_device_nhwc(plan(xd), K), want), (x.shape, K, tile, plan.kernel)
        plan.select(3, 0)
        acc = torch.empty((N, H, W, plan.desc.out_cs), dtype=torch.int32, device="cuda")
        plan(xd, acc=acc)
        assert np.array_equal(acc.cpu().numpy()[..., :K].transpose(0, 3, 1, 2), want_acc)
        plan.special(0)
        assert not plan.kernel.endswith("_halo")
        assert np.array_equal(hipq.from_device_nhwc(plan(xd), K), want)
        plan.select(1, 0).special(2)  # the 256-pixel tile has no halo variant
        assert not plan.kernel.endswith("_halo")
        assert np.array_equal(hipq.from_device_nhwc(plan(xd), K), want)
        # int8 tensors: zero padding
        xs, ws = x.view(np.int8), w.view(np.int8)
        want8 = orc.conv2d_i8(xs, ws, b, 1, 1, 1, q[0], q[2], q[4], 7)
        p8 = hipq.Conv2d(x.shape, ws, b, 1, 1, 1, q[0], 0, q[2], 0, q[4], 0, obits=7, dtype=hipq.DTYPE_I8)
        p8.select(0, 0).special(2)
        assert p8.kernel.endswith("_halo") == (C == 64 or (C in (128, 256, 512) and W <= 31)), p8.kernel
        assert np.array_equal(hipq.from_device_nhwc(p8(hipq.to_device_nhwc(xs)), K).view(np.int8), want8), (x.shape, K)
    # not eligible: stride 2, pad 0, wide images, asymmetric weights
    for kw in (dict(stride=2), dict(pad=0), dict(W=64), dict(wzp=100)):
        W_ = kw.get("W", 16)
        x = rng.integers(0, 256, (1, 64, 16, W_), dtype=np.uint8)
        w = rng.integers(0, 256, (64, 64, 3, 3), dtype=np.uint8)
        plan = hipq.Conv2d(x.shape, w, None, kw.get("pad", 1), kw.get("stride", 1), 1, 0.02, 7, 0.005, kw.get("wzp", 128), 0.05, 3)
        assert not plan.kernel.endswith("_halo"), (kw, plan.kernel)
        want = orc.conv2d_u8(x, w, None, kw.get("pad", 1), kw.get("stride", 1), 1, 0.02, 7, 0.005, kw.get("wzp", 128), 0.05, 3)
        assert np.array_equal(hipq.from_device_nhwc(plan(hipq.to_device_nhwc(x)), 64), want), kw


def test_concat_softmax():
    rng = np.random.default_rng(44)
    for it in range(12):
        n_in = int(rng.integers(2, 9))
        N, H, W = int(rng.integers(1, 4)), int(rng.integers(1, 9)), int(rng.integers(1, 9))
        chans = [int(rng.choice([1, 3, 4, 7, 16, 20, 64, 100])) for _ in range(n_in)]
        if it == 0:
            N, H, W, chans = 4, 28, 28, [64, 128, 32, 32]  # an inception-style block: every piece dword-aligned
        ins = [rng.integers(0, 256, (N, c, H, W), dtype=np.uint8) for c in chans]
        ia, iz = [rand_q(rng) for _ in ins], [int(rng.integers(0, 256)) for _ in ins]
        oa, oz = rand_q(rng), int(rng.integers(0, 256))
        want = orc.concat_u8(ins, ia, iz, oa, oz)
        yd = torch.full((N, H, W, hipq.channel_stride(sum(chans))), 0xAB, dtype=torch.uint8, device="cuda")
        hipq.concat_u8([hipq.to_device_nhwc(a) for a in ins], chans, yd, ia, iz, oa, oz)
        assert np.array_equal(hipq.from_device_nhwc(yd, sum(chans)), want), (it, chans)
        assert int(yd[..., sum(chans):].max().item() if yd.shape[-1] > sum(chans) else 0) == 0  # pad channels cleared
    for it, shape in enumerate([(64, 1000, 1, 1), (2, 21, 33, 17), (1, 2, 5, 5), (3, 7, 1, 9), (5, 300, 2, 2)]):
        x = rng.integers(0, 256, shape, dtype=np.uint8)
        q = (rand_q(rng, 1e-2, 0.2), int(rng.integers(0, 256)), float(np.float32(1.0 / 255)), int(rng.integers(0, 3)))
        want = orc.softmax_u8(x, 1, *q)
        xd = hipq.to_device_nhwc(x)
        yd = torch.empty_like(xd)
        hipq.softmax_u8(xd, yd, shape[1], *q)
        assert np.array_equal(hipq.from_device_nhwc(yd, shape[1]), want), (it, shape, q)


# ---- int8 symmetric variants (op_conv_2d_i8xi8_run, op_quant_ip_i8xi8_run, op_quantize_run_i8, op_dequantize_run_i8) ----
def run_conv_i8(x, w, b, pad, stride, group, q, obits=8, in_cs=None):
    ia, wa, oa = q
    plan = hipq.Conv2d(x.shape, w, b, pad, stride, group, ia, 0, wa, 0, oa, 0, obits=obits, dtype=hipq.DTYPE_I8, in_cs=in_cs)
    xd = hipq.to_device_nhwc(x)
    acc = torch.zeros((x.shape[0], plan.OH, plan.OW, plan.desc.out_cs), dtype=torch.int32, device="cuda")
    yd = plan(xd, acc=acc)
    torch.cuda.synchronize()
    y = hipq.from_device_nhwc(yd, w.shape[0]).view(np.int8)
    return y, acc.cpu().numpy()[..., :w.shape[0]].transpose(0, 3, 1, 2), plan.kernel


def test_conv_int8():
    """Every kernel variant with int8 tensors: MFMA tiles (DMA-fed and the small-C stem form), depthwise, grouped;
    obits 8 (clip to +-255, then two's complement wrap), 7 and 4; with and without bias; ragged tiles and paddings."""
    rng = np.random.default_rng(41)
    kerns = set()
    cases = [  # N, C, H, W, K, R, S, pad, stride, group
        (2, 64, 14, 14, 64, 3, 3, 1, 1, 1), (1, 64, 9, 11, 128, 1, 1, 0, 1, 1), (3, 32, 10, 7, 48, 3, 3, 1, 2, 1),
        (1, 16, 12, 12, 24, 5, 3, (1, 2), 1, 1), (2, 128, 7, 7, 256, 1, 1, 0, 2, 1), (1, 3, 33, 29, 64, 7, 7, 3, 2, 1),
        (2, 3, 16, 16, 16, 3, 3, 1, 1, 1), (1, 256, 6, 6, 64, 3, 3, 1, 1, 1), (2, 32, 9, 9, 32, 3, 3, 1, 1, 32),
        (1, 48, 10, 10, 48, 3, 3, 1, 2, 48), (1, 24, 8, 8, 24, 5, 5, 2, 1, 24), (1, 8, 9, 9, 12, 3, 3, (2, 0), (1, 2), 2),
        (2, 512, 7, 7, 512, 3, 3, 1, 1, 1), (4, 256, 14, 14, 1024, 1, 1, 0, 1, 1),
    ]
    for i, (N, C, H, W, K, R, S, pad, st, grp) in enumerate(cases):
        x = rng.integers(-128, 128, (N, C, H, W), dtype=np.int8)
        w = rng.integers(-128, 128, (K, C // grp, R, S), dtype=np.int8)
        b = rng.integers(-30000, 30000, K).astype(np.int32) if i % 3 else None
        for obits in (8, 7, 4):
            q = (rand_q(rng), rand_q(rng), rand_q(rng, 1e-2, 1.0))
            print("int8 conv case", i, x.shape, w.shape, pad, st, grp, q, obits, flush=True)
            want_y, want_acc = orc.conv2d_i8(x, w, b, pad, st, grp, *q, obits=obits, return_acc=True)
            y, acc, kern = run_conv_i8(x, w, b, pad, st, grp, q, obits)
            kerns.add(kern)
            assert np.array_equal(acc, want_acc), (i, kern, "accumulators differ", int((acc != want_acc).sum()))
            assert np.array_equal(y, want_y), (i, kern, obits, "outputs differ", int((y != want_y).sum()))
    assert any("mfma" in k and "_c4" in k for k in kerns) and any("depthwise_i8" in k for k in kerns) \
        and any("direct_i8" in k for k in kerns), kerns
    # extremes: -128 * -128 over a long reduction, and outputs that wrap with obits = 8
    x = np.full((1, 512, 3, 3), -128, np.int8)
    w = np.full((16, 512, 3, 3), -128, np.int8)
    for oa in (0.5, 40.0):
        want = orc.conv2d_i8(x, w, None, 1, 1, 1, 0.01, 0.01, oa, 8)
        y, _, _ = run_conv_i8(x, w, None, 1, 1, 1, (0.01, 0.01, oa), 8)
        assert np.array_equal(y, want)
    assert want.min() < -100 or want.max() > 100
    with pytest.raises(hipq.HipqError):  # the fused residual add is a uint8 operator
        plan = hipq.Conv2d((1, 64, 4, 4), np.zeros((64, 64, 1, 1), np.int8), None, 0, 1, 1, 0.1, 0, 0.1, 0, 0.1, 0,
                           dtype=hipq.DTYPE_I8)
        t = torch.zeros((1, 4, 4, 64), dtype=torch.uint8, device="cuda")
        plan.run_add(t, t, False, 0.1, 0, 0.1, 0, t.clone())


def test_ip_int8():
    rng = np.random.default_rng(42)
    for M, Kd, No, obits in ((1, 64, 10, 8), (7, 300, 33, 7), (128, 4096, 256, 8), (5, 2048, 1000, 7)):
        x = rng.integers(-128, 128, (M, Kd), dtype=np.int8)
        w = rng.integers(-128, 128, (No, Kd), dtype=np.int8)
        b = rng.integers(-50000, 50000, No).astype(np.int32)
        q = (rand_q(rng), rand_q(rng), rand_q(rng, 1e-1, 10.0))
        want_y, want_acc = orc.ip_i8(x, w, b, *q, obits=obits, return_acc=True)
        y, acc, kern = run_conv_i8(x.reshape(M, Kd, 1, 1), w.reshape(No, Kd, 1, 1), b, 0, 1, 1, q, obits)
        assert np.array_equal(acc.reshape(M, No), want_acc), (M, Kd, No, kern)
        assert np.array_equal(y.reshape(M, No), want_y), (M, Kd, No, kern)


def test_quantize_dequantize_int8():
    rng = np.random.default_rng(43)
    for shape in ((2, 3, 224, 224), (1, 16, 9, 9), (4, 1000, 1, 1), (2, 3, 7, 5)):
        for obits in (8, 7, 4, 2):
            oa = rand_q(rng, 5e-3, 0.1)
            x = (rng.standard_normal(shape) * 60 * oa).astype(np.float32)
            n = min(600, x.size - 8)
            x.flat[:n] = (np.arange(n, dtype=np.float32) * 0.5 - 150) * np.float32(oa)  # ties of both signs, both clips
            x.flat[n:n + 6] = [3e9, -3e9, 1e30, -1e30, np.inf, -np.inf]                 # beyond int32: the conversion's sentinel
            xd = torch.from_numpy(x).cuda()
            cs = hipq.channel_stride(shape[1])
            yd = torch.empty((shape[0], shape[2], shape[3], cs), dtype=torch.uint8, device="cuda")
            hipq.quantize_i8(xd, yd, oa, obits)
            want = orc.quantize_i8(x, oa, obits)
            got = hipq.from_device_nhwc(yd, shape[1]).view(np.int8)
            assert np.array_equal(got, want), (shape, obits, int((got != want).sum()))
            fd = torch.empty(shape, dtype=torch.float32, device="cuda")
            hipq.dequantize_i8(yd, fd, oa)
            assert np.array_equal(fd.cpu().numpy().view(np.uint32), orc.dequantize_i8(want, oa).view(np.uint32))


def test_golden_int8_outputs_on_gpu():
    """The compiled reference's recorded int8 outputs, reproduced by the HIP kernels."""
    g = np.load(os.path.join(HERE, "golden", "quant_ops_int8.npz"))
    meta = json.loads(bytes(g["meta"]).decode())
    for name, m in meta.items():
        kind, a = m["kind"], m["args"]
        ins = [g["%s.in%d" % (name, i)] for i in range(m["n_in"])]
        want = g[name + ".out"]
        if kind == "conv":
            got, _, _ = run_conv_i8(ins[0], ins[1], ins[2], a["pad"], a["stride"], a["group"], a["q"], a["obits"])
        elif kind == "ip":
            M, Kd = ins[0].shape
            got, _, _ = run_conv_i8(ins[0].reshape(M, Kd, 1, 1), ins[1].reshape(-1, Kd, 1, 1), ins[2], 0, 1, 1, a["q"], a["obits"])
            got = got.reshape(want.shape)
        elif kind == "quantize":
            N, Cc, H, W = ins[0].shape
            yd = torch.empty((N, H, W, hipq.channel_stride(Cc)), dtype=torch.uint8, device="cuda")
            hipq.quantize_i8(torch.from_numpy(ins[0]).cuda(), yd, a["q"][0], a["obits"])
            got = hipq.from_device_nhwc(yd, Cc).view(np.int8)
        else:
            fd = torch.empty(ins[0].shape, dtype=torch.float32, device="cuda")
            hipq.dequantize_i8(hipq.to_device_nhwc(ins[0]), fd, a["q"][0])
            got = fd.cpu().numpy()
        assert np.array_equal(got.view(np.uint8), want.view(np.uint8)), name


def test_two_group_kernel_matches_the_oracle():
    """Layers with a long reduction and few tiles run the tile kernel with two groups of waves that reduce every other
    slab each and add their partial sums through LDS: 3x3 and 1x1 kernels, stride 2, a partial last slab (1x1 with a
    channel stride that is no multiple of 64), ragged pixel and channel tiles, accumulator dumps, int8 tensors, every tile
    shape; an odd number of slabs, an explicit stage count or mode 0 keep the four-wave kernel."""
    rng = np.random.default_rng(47)
    #         N   C    H   W   K   R  pad stride
    shapes = [(2, 256, 14, 14, 256, 3, 1, 1), (3, 512, 7, 7, 200, 3, 1, 1), (5, 512, 9, 9, 96, 1, 0, 1), (2, 1000, 3, 5, 130, 1, 0, 1),
              (1, 128, 17, 17, 64, 3, 1, 2), (64, 2048, 1, 1, 1000, 1, 0, 1), (1, 64, 12, 12, 32, 3, 0, 1),
              (16, 512, 14, 14, 512, 1, 0, 1)]  # the last one: more tiles than CUs with the small tiles (on request only)
    for N, C, H, W, K, R, pad, stride in shapes:
        print("two-group case", N, C, H, W, K, R, pad, stride, flush=True)
        x = rng.integers(0, 256, (N, C, H, W), dtype=np.uint8)
        w = rng.integers(0, 256, (K, C, R, R), dtype=np.uint8)
        b = rng.integers(-30000, 30000, K).astype(np.int32)
        q = (rand_q(rng), int(rng.integers(0, 256)), rand_q(rng), 128, rand_q(rng, 1e-2, 1.0), int(rng.integers(0, 256)))
        want, want_acc = orc.conv2d_u8(x, w, b, pad, stride, 1, *q, return_acc=True)
        plan = hipq.Conv2d(x.shape, w, b, pad, stride, 1, *q)
        nslab = (R * R * plan.desc.in_cs + 63) // 64
        eligible = nslab % 2 == 0 and nslab >= 8
        # few pixels of whole 128-byte lines go to the streaming kernel unless a tile is named
        npix = N * plan.OH * plan.OW
        stream = plan.desc.in_cs % 128 == 0 and (npix <= 256 or (npix <= 1024 and R * R * plan.desc.in_cs >= 512))
        assert ("_stream_" in plan.kernel) == stream
        assert plan.kernel.endswith("_k2") == (eligible and not stream), (plan.kernel, nslab)  # every case has at most 256 tiles of the rule's own tile
        xd = hipq.to_device_nhwc(x)
        assert np.array_equal(hipq.from_device_nhwc(plan(xd), K), want), (x.shape, K, plan.kernel)
        if not stream:  # the fused residual add takes the same kernel where it applies, in both operand orders
            assert plan.kernel_add.endswith("_k2+add") == eligible, plan.kernel_add
            res = rng.integers(0, 256, want.shape, dtype=np.uint8)
            ra, rz, sa, sz = rand_q(rng, 1e-2, 1e-1), int(rng.integers(0, 256)), rand_q(rng, 3e-2, 3e-1), int(rng.integers(0, 256))
            for first in (False, True):
                yd = plan.run_add(xd, hipq.to_device_nhwc(res), first, ra, rz, sa, sz, plan.empty_output())
                want_add = orc.add_u8(res, want, ra, rz, q[4], q[5], sa, sz) if first else orc.add_u8(want, res, q[4], q[5], ra, rz, sa, sz)
                assert np.array_equal(hipq.from_device_nhwc(yd, K), want_add), (x.shape, K, first, plan.kernel_add)
        plan.special(2)
        for tile in (0, 2, 3, 4):
            plan.select(tile, 0)
            # on request the halo kernel takes the 3x3 / stride 1 / pad 1 layers it can (128-channel tiles, narrow images)
            halo = R == 3 and pad == 1 and stride == 1 and C in (128, 256, 512) and tile in (0, 3) and W <= 31
            assert plan.kernel.endswith("_halo") == halo and plan.kernel.endswith("_k2") == (eligible and not halo), (plan.kernel, tile)
            assert np.array_equal(hipq.from_device_nhwc(plan(xd), K), want), (x.shape, K, tile, plan.kernel)
            acc = torch.empty((N, plan.OH, plan.OW, plan.desc.out_cs), dtype=torch.int32, device="cuda")
            plan(xd, acc=acc)
            assert np.array_equal(acc.cpu().numpy()[..., :K].transpose(0, 3, 1, 2), want_acc), (x.shape, tile)
        plan.select(1, 0)  # the 256-pixel tile has no two-group variant
        assert not plan.kernel.endswith("_k2")
        plan.select(3, 3)  # an explicit stage count means the four-wave kernel
        assert not plan.kernel.endswith("_k2")
        assert np.array_equal(hipq.from_device_nhwc(plan(xd), K), want)
        plan.select(3, 0).special(0)
        assert not plan.kernel.endswith("_k2")
        assert np.array_equal(hipq.from_device_nhwc(plan(xd), K), want)
        xs, ws = x.view(np.int8), w.view(np.int8)
        want8 = orc.conv2d_i8(xs, ws, b, pad, stride, 1, q[0], q[2], q[4], 7)
        p8 = hipq.Conv2d(x.shape, ws, b, pad, stride, 1, q[0], 0, q[2], 0, q[4], 0, obits=7, dtype=hipq.DTYPE_I8)
        assert p8.kernel.endswith("_k2") == (eligible and not stream), p8.kernel
        assert np.array_equal(hipq.from_device_nhwc(p8(hipq.to_device_nhwc(xs)), K).view(np.int8), want8), (x.shape, K)
    # asymmetric weights keep the generic kernel
    x = rng.integers(0, 256, (1, 256, 8, 8), dtype=np.uint8)
    w = rng.integers(0, 256, (64, 256, 3, 3), dtype=np.uint8)
    plan = hipq.Conv2d(x.shape, w, None, 1, 1, 1, 0.02, 7, 0.005, 100, 0.05, 3)
    assert not plan.kernel.endswith("_k2"), plan.kernel
