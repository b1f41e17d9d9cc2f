"""Pins the CPU oracle (oracle/quant_oracle.c):
  1. against the conv known answers recorded from the reference CPU quant module (FNV-1a-64 of the
     uint8 output for ten seeded cases; tests/golden/conv_kat.json),
  2. against the reference module itself where oracle/_ref is built (differential, random cases),
  3. against committed golden outputs of the compiled reference (tests/golden/quant_ops.npz),
  4. against independent numpy formulations (exact rational rounding, int64 tensordot) so that a
     dropped term, a wrong sign or a transposed operand fails without any reference at hand.
"""
import json
import os
from fractions import Fraction

import numpy as np
import pytest

from oracle import orc

import refrun

HERE = os.path.dirname(os.path.abspath(__file__))
GOLD = os.path.join(HERE, "golden")


# ----------------------------------------------------------------------------------------------
# 1. recorded known answers
def kat_case(c):
    """Inputs of a recorded case: one xorshift stream, x then w then bias."""
    g = orc.XorShift()
    N, C, H, K, R, pad, st, grp = c["N"], c["C"], c["H"], c["K"], c["R"], c["pad"], c["stride"], c["group"]
    x = (g.u32(N * C * H * H) & 255).astype(np.uint8).reshape(N, C, H, H)
    w = ((g.u32(K * (C // grp) * R * R) % 255).astype(np.int64) - 127 + 128).astype(np.uint8)
    w = w.reshape(K, C // grp, R, R)
    b = ((g.u32(K) % 2001).astype(np.int64) - 1000).astype(np.int32)
    return x, w, b


with open(os.path.join(GOLD, "conv_kat.json")) as f:
    KATS = json.load(f)


@pytest.mark.parametrize("c", KATS["cases"], ids=lambda c: c["id"])
def test_conv_known_answers(c):
    x, w, b = kat_case(c)
    y = orc.conv2d_u8(x, w, b, c["pad"], c["stride"], c["group"], 0.02, c["izp"], 0.005, 128, 0.05,
                      c["ozp"])
    assert orc.quant_scale(np.float32(0.02) * np.float32(0.005) / np.float32(0.05), 32) == (1099511552, 39)
    assert "%016x" % orc.fnv1a64(y) == c["fnv"]
    if y.size < 50000:  # the reference-shaped variant must agree as well
        y2 = orc.conv2d_u8(x, w, b, c["pad"], c["stride"], c["group"], 0.02, c["izp"], 0.005, 128,
                           0.05, c["ozp"], refshape=True)
        assert np.array_equal(y, y2)


# ----------------------------------------------------------------------------------------------
# 2. differential against the compiled reference
def rand_q(rng, lo=1e-3, hi=1e-1):
    return float(np.float32(np.exp(rng.uniform(np.log(lo), np.log(hi)))))


def test_conv_vs_reference(ref_ws):
    rng = np.random.default_rng(1)
    for it in range(60):
        grp = int(rng.choice([1, 1, 1, 2, 4]))
        C = grp * int(rng.integers(1, 9))
        K = grp * int(rng.integers(1, 9))
        if it % 10 == 0:  # depthwise
            grp = C = K = int(rng.integers(2, 12))
        R, S = int(rng.integers(1, 6)), int(rng.integers(1, 6))
        H, W = int(rng.integers(R, R + 12)), int(rng.integers(S, S + 12))
        # the reference's im2col bounds its bottom-border rows with pad_w instead of pad_h
        # (im2col.cpp:757, `j < height + pad_w`), so it is only meaningful for pad_h == pad_w
        p = int(rng.integers(0, min(R, S)))
        pad = (p, p)
        st = (int(rng.integers(1, 4)), int(rng.integers(1, 4)))
        N = int(rng.integers(1, 3))
        x = rng.integers(0, 256, (N, C, H, W), dtype=np.uint8)
        w = rng.integers(0, 256, (K, C // grp, R, S), dtype=np.uint8)
        b = rng.integers(-20000, 20000, K).astype(np.int32)
        q = (rand_q(rng), int(rng.integers(0, 256)), rand_q(rng), int(rng.integers(0, 256)),
             rand_q(rng, 1e-2, 1.0), int(rng.integers(0, 256)))
        want = refrun.conv2d_u8(ref_ws, x, w, b, pad, st, grp, *q)
        got = orc.conv2d_u8(x, w, b, pad, st, grp, *q)
        assert np.array_equal(got, want), (it, x.shape, w.shape, pad, st, grp, q)
        got2 = orc.conv2d_u8(x, w, b, pad, st, grp, *q, refshape=True)
        assert np.array_equal(got2, want)


def test_ip_vs_reference(ref_ws):
    rng = np.random.default_rng(2)
    for it in range(25):
        M, Kd, No = int(rng.integers(1, 6)), int(rng.integers(1, 400)), int(rng.integers(1, 50))
        x = rng.integers(0, 256, (M, Kd), dtype=np.uint8)
        w = rng.integers(0, 256, (No, Kd), dtype=np.uint8)
        b = rng.integers(-50000, 50000, No).astype(np.int32)
        q = (rand_q(rng), int(rng.integers(0, 256)), rand_q(rng), int(rng.integers(0, 256)),
             rand_q(rng, 1e-2, 1.0), int(rng.integers(0, 256)))
        assert np.array_equal(orc.ip_u8(x, w, b, *q), refrun.ip_u8(ref_ws, x, w, b, *q)), (it, q)


def test_elementwise_vs_reference(ref_ws):
    rng = np.random.default_rng(3)
    for it in range(40):
        shape = (1, int(rng.integers(1, 5)), int(rng.integers(1, 9)), int(rng.integers(1, 9)))
        a = rng.integers(0, 256, shape, dtype=np.uint8)
        b = rng.integers(0, 256, shape, dtype=np.uint8)
        c = rng.integers(0, 256, shape, dtype=np.uint8)
        ia = [rand_q(rng) for _ in range(3)]
        iz = [int(rng.integers(0, 256)) for _ in range(3)]
        oa, oz = rand_q(rng, 3e-3, 0.3), int(rng.integers(0, 256))
        assert np.array_equal(orc.add_u8(a, b, ia[0], iz[0], ia[1], iz[1], oa, oz),
                              refrun.add_u8(ref_ws, a, b, ia[0], iz[0], ia[1], iz[1], oa, oz)), it
        for n_in in (2, 3):
            for operation in (1, 2):
                got = orc.eltwise_u8([a, b, c][:n_in], ia[:n_in], iz[:n_in], oa, oz, operation)
                want = refrun.eltwise_u8(ref_ws, [a, b, c][:n_in], ia[:n_in], iz[:n_in], oa, oz, operation)
                assert np.array_equal(got, want), (it, n_in, operation)
        coeff = [float(np.float32(rng.uniform(0.25, 2.0))) for _ in range(2)]
        assert np.array_equal(orc.eltwise_u8([a, b], ia[:2], iz[:2], oa, oz, 1, coeff),
                              refrun.eltwise_u8(ref_ws, [a, b], ia[:2], iz[:2], oa, oz, 1, coeff))
        assert np.array_equal(orc.relu_u8(a, ia[0], iz[0], oa, oz),
                              refrun.relu_u8(ref_ws, a, ia[0], iz[0], oa, oz)), it
    # a fused-ReLU conv equals conv followed by this op when scales and zero points coincide
    x = np.arange(256, dtype=np.uint8).reshape(1, 1, 16, 16)
    assert np.array_equal(orc.relu_u8(x, 0.05, 77, 0.05, 77), np.maximum(x, 77))


def test_pool_vs_reference(ref_ws):
    rng = np.random.default_rng(4)
    done = 0
    while done < 60:
        k = (int(rng.integers(1, 5)), int(rng.integers(1, 5)))
        pad = (int(rng.integers(0, k[0])), int(rng.integers(0, k[1])))
        # stride <= kernel: with a larger stride and ceil_mode the reference sweeps a window that lies
        # wholly outside the image, divides by a pool size of 0 and never returns (pool.c:211-214)
        st = (int(rng.integers(1, k[0] + 1)), int(rng.integers(1, k[1] + 1)))
        H, W = int(rng.integers(k[0], 15)), int(rng.integers(k[1], 15))
        method, ceil_mode = int(rng.integers(0, 2)), bool(rng.integers(0, 2))
        N, C = int(rng.integers(1, 3)), int(rng.integers(1, 5))
        x = rng.integers(0, 256, (N, C, H, W), dtype=np.uint8)
        q = (rand_q(rng), int(rng.integers(0, 256)), rand_q(rng), int(rng.integers(0, 256)))
        want = refrun.pool_u8(ref_ws, x, k, pad, st, method, ceil_mode, *q)
        got = orc.pool_u8(x, k, pad, st, method, ceil_mode, *q)
        assert got.shape == want.shape, (k, pad, st, H, W, ceil_mode)
        assert np.array_equal(got, want), (k, pad, st, H, W, method, ceil_mode, q)
        done += 1
    # the two shapes ResNet needs: 3x3/s2/p1 max (112 -> 56 with ceil_mode off) and global average
    assert orc.pool_out_dim(112, 1, 3, 2, False) == 56 and orc.pool_out_dim(112, 1, 3, 2, True) == 57
    assert orc.pool_out_dim(7, 0, 7, 1, True) == 1


def test_quantize_dequantize_vs_reference(ref_ws):
    rng = np.random.default_rng(5)
    for it in range(10):
        oa, oz = rand_q(rng, 5e-3, 0.1), int(rng.integers(0, 256))
        x = (rng.standard_normal((1, 3, 40, 40)) * 6 * oa * 40).astype(np.float32)
        # exact ties and saturation edges
        x.flat[:512] = (np.arange(512, dtype=np.float32) * 0.5 - oz) * np.float32(oa)
        want = refrun.quantize_u8(ref_ws, x, oa, oz)
        assert np.array_equal(orc.quantize_u8(x, oa, oz), want), it
        d = refrun.dequantize_u8(ref_ws, want, oa, oz)
        assert np.array_equal(orc.dequantize_u8(want, oa, oz).view(np.uint32), d.view(np.uint32))


def test_concat_softmax_vs_reference(ref_ws):
    rng = np.random.default_rng(24)
    for it in range(20):
        n_in = int(rng.integers(2, 5))
        N, H, W = int(rng.integers(1, 4)), int(rng.integers(1, 7)), int(rng.integers(1, 7))
        ins = [rng.integers(0, 256, (N, int(rng.integers(1, 20)), H, W), dtype=np.uint8) for _ in range(n_in)]
        ia, iz = [rand_q(rng) for _ in ins], [int(rng.integers(0, 256)) for _ in ins]
        oa, oz = rand_q(rng), int(rng.integers(0, 256))
        want = refrun.concat_u8(ref_ws, ins, ia, iz, oa, oz)
        assert np.array_equal(orc.concat_u8(ins, ia, iz, oa, oz), want), (it, ia, iz, oa, oz)
    for it in range(20):
        shape = [(int(rng.integers(1, 4)), int(rng.integers(2, 40)), int(rng.integers(1, 6)), int(rng.integers(1, 6))),
                 (int(rng.integers(1, 5)), int(rng.integers(2, 1200)), 1, 1)][it % 2]
        axis = 1 if it % 4 else int(rng.integers(1, 4))
        x = rng.integers(0, 256, shape, dtype=np.uint8)
        q = (rand_q(rng, 1e-2, 0.2), int(rng.integers(0, 256)), float(np.float32(1.0 / 255)), int(rng.integers(0, 3)))
        want = refrun.softmax_u8(ref_ws, x, axis, *q)
        assert np.array_equal(orc.softmax_u8(x, axis, *q), want), (it, shape, axis, q)


def test_int8_conv_vs_reference(ref_ws):
    """op_conv_2d_i8xi8_run with the portable gemm_i8xi8 (ibits == wbits == 8; the lower-bit GEMMs are not
    implemented outside aarch64).  7x7 kernels take the reference's region-split im2col and are left out."""
    rng = np.random.default_rng(21)
    for it in range(50):
        grp = int(rng.choice([1, 1, 1, 2, 4]))
        C = grp * int(rng.integers(1, 9))
        K = grp * int(rng.integers(1, 9))
        if it % 10 == 0:
            grp = C = K = int(rng.integers(2, 12))
        R, S = int(rng.integers(1, 6)), int(rng.integers(1, 6))
        H, W = int(rng.integers(R, R + 12)), int(rng.integers(S, S + 12))
        pad = (int(rng.integers(0, R)), int(rng.integers(0, S)))
        st = (int(rng.integers(1, 4)), int(rng.integers(1, 4)))
        N = int(rng.integers(1, 4))
        x = rng.integers(-128, 128, (N, C, H, W), dtype=np.int8)
        w = rng.integers(-128, 128, (K, C // grp, R, S), dtype=np.int8)
        b = rng.integers(-20000, 20000, K).astype(np.int32) if it % 4 else None
        q = (rand_q(rng), rand_q(rng), rand_q(rng, 1e-2, 1.0))
        obits = int(rng.choice([8, 8, 7, 4]))
        want = refrun.conv2d_i8(ref_ws, x, w, b, pad, st, grp, *q, obits=obits)
        got = orc.conv2d_i8(x, w, b, pad, st, grp, *q, obits=obits)
        assert want.dtype == np.int8 and np.array_equal(got, want), (it, x.shape, w.shape, pad, st, grp, q, obits)


def test_int8_ip_vs_reference(ref_ws):
    rng = np.random.default_rng(22)
    for it in range(25):
        M, Kd, No = int(rng.integers(1, 6)), int(rng.integers(1, 400)), int(rng.integers(1, 50))
        x = rng.integers(-128, 128, (M, Kd), dtype=np.int8)
        w = rng.integers(-128, 128, (No, Kd), dtype=np.int8)
        b = rng.integers(-50000, 50000, No).astype(np.int32) if it % 3 else None
        q = (rand_q(rng), rand_q(rng), rand_q(rng, 1e-2, 1.0))
        obits = int(rng.choice([8, 7]))
        assert np.array_equal(orc.ip_i8(x, w, b, *q, obits=obits), refrun.ip_i8(ref_ws, x, w, b, *q, obits=obits)), (it, q)


def test_int8_quantize_dequantize_vs_reference(ref_ws):
    rng = np.random.default_rng(23)
    for it in range(12):
        oa = rand_q(rng, 5e-3, 0.1)
        obits = int(rng.choice([8, 8, 7, 6, 4, 3, 2]))
        x = (rng.standard_normal((2, 3, 20, 20)) * 60 * oa).astype(np.float32)
        x.flat[:600] = (np.arange(600, dtype=np.float32) * 0.5 - 150) * np.float32(oa)  # ties of both signs, both clips
        x.flat[600:606] = [3e9, -3e9, 1e30, -1e30, np.inf, -np.inf]  # beyond int32: the conversion's sentinel
        want = refrun.quantize_i8(ref_ws, x, oa, obits)
        assert want.dtype == np.int8 and np.array_equal(orc.quantize_i8(x, oa, obits), want), (it, oa, obits)
        d = refrun.dequantize_i8(ref_ws, want, oa, obits)
        assert np.array_equal(orc.dequantize_i8(want, oa).view(np.uint32), d.view(np.uint32))


# ----------------------------------------------------------------------------------------------
# 3. committed golden outputs of the compiled reference
def test_golden_outputs():
    g = np.load(os.path.join(GOLD, "quant_ops.npz"))
    meta = json.loads(bytes(g["meta"]).decode())
    for name, m in meta.items():
        kind, a = m["kind"], m["args"]
        ins = [g["%s.in%d" % (name, i)] for i in range(m["n_in"])]
        want = g[name + ".out"]
        if kind == "conv":
            got = orc.conv2d_u8(ins[0], ins[1], ins[2], a["pad"], a["stride"], a["group"], *a["q"])
        elif kind == "ip":
            got = orc.ip_u8(ins[0], ins[1], ins[2], *a["q"])
        elif kind == "add":
            got = orc.add_u8(ins[0], ins[1], *a["q"])
        elif kind == "eltwise":
            got = orc.eltwise_u8(ins, a["ialpha"], a["izp"], a["oalpha"], a["ozp"], a["operation"])
        elif kind == "relu":
            got = orc.relu_u8(ins[0], *a["q"])
        elif kind == "pool":
            got = orc.pool_u8(ins[0], a["kernel"], a["pad"], a["stride"], a["method"], a["ceil_mode"], *a["q"])
        elif kind == "quantize":
            got = orc.quantize_u8(ins[0], *a["q"])
        elif kind == "dequantize":
            got = orc.dequantize_u8(ins[0], *a["q"])
        else:
            raise AssertionError(kind)
        assert got.shape == want.shape, name
        assert np.array_equal(got.view(np.uint8), want.view(np.uint8)), name


def test_golden_outputs_int8():
    g = np.load(os.path.join(GOLD, "quant_ops_int8.npz"))
    meta = json.loads(bytes(g["meta"]).decode())
    assert len(meta) == 10
    for name, m in meta.items():
        kind, a = m["kind"], m["args"]
        ins = [g["%s.in%d" % (name, i)] for i in range(m["n_in"])]
        want = g[name + ".out"]
        if kind == "conv":
            got = orc.conv2d_i8(ins[0], ins[1], ins[2], a["pad"], a["stride"], a["group"], *a["q"], obits=a["obits"])
        elif kind == "ip":
            got = orc.ip_i8(ins[0], ins[1], ins[2], *a["q"], obits=a["obits"])
        elif kind == "quantize":
            got = orc.quantize_i8(ins[0], *a["q"], obits=a["obits"])
        elif kind == "dequantize":
            got = orc.dequantize_i8(ins[0], *a["q"])
        else:
            raise AssertionError(kind)
        assert got.shape == want.shape and got.dtype == want.dtype, name
        assert np.array_equal(got.view(np.uint8), want.view(np.uint8)), name


# ----------------------------------------------------------------------------------------------
# 4. what the mathematics fixes, formulated independently of the C code
def test_rshift_rn_is_round_half_up():
    rng = np.random.default_rng(6)
    for _ in range(2000):
        x = int(rng.integers(-2**62, 2**62))
        s = int(rng.integers(1, 62))
        want = (Fraction(x, 2**s) + Fraction(1, 2)).__floor__()
        assert orc.rshift_rn(x, s) == want
    assert orc.rshift_rn(-3, 1) == -1 and orc.rshift_rn(3, 1) == 2 and orc.rshift_rn(-1, 1) == 0


def test_quant_scale_is_exact():
    rng = np.random.default_rng(7)
    for bits in (16, 23, 24, 32):
        for _ in range(300):
            f = np.float32(np.exp(rng.uniform(np.log(1e-6), np.log(30.0))))
            m, s = orc.quant_scale(f, bits)
            assert 2 ** (bits - 2) <= m < 2 ** (bits - 1)
            # mult is the scale's mantissa truncated to bits-1 bits; with 32 bits nothing is lost
            assert m == (Fraction(float(f)) * 2 ** s).__floor__()
            if bits == 32:
                assert Fraction(m, 2 ** s) == Fraction(float(f))
    assert orc.quant_scale(0.0, 32) == (0, 0)


def _requant(acc, scale_f32, ozp):
    """floor(acc * scale + 1/2) + ozp, clamped — exact rational arithmetic."""
    f = Fraction(float(scale_f32))
    return np.array([min(255, max(0, (Fraction(int(a)) * f + Fraction(1, 2)).__floor__() + ozp))
                     for a in acc.ravel()], np.uint8).reshape(acc.shape)


def test_conv_against_int64_tensordot():
    rng = np.random.default_rng(8)
    for grp, C, K, R, S, pad, st in ((1, 5, 7, 3, 3, (1, 1), (1, 1)), (1, 4, 6, 1, 1, (0, 0), (2, 2)),
                                     (2, 6, 4, 3, 2, (2, 0), (1, 2)), (6, 6, 6, 3, 3, (1, 1), (2, 1)),
                                     (1, 3, 8, 7, 7, (3, 3), (2, 2))):
        N, H, W = 2, 11, 9
        x = rng.integers(0, 256, (N, C, H, W), dtype=np.uint8)
        w = rng.integers(0, 256, (K, C // grp, R, S), dtype=np.uint8)
        b = rng.integers(-5000, 5000, K).astype(np.int32)
        ia, izp, wa, wzp, oa, ozp = 0.017, 113, 0.0031, 140, 0.041, 9
        y, acc = orc.conv2d_u8(x, w, b, pad, st, grp, ia, izp, wa, wzp, oa, ozp, return_acc=True)
        OH, OW = y.shape[2:]
        xp = np.zeros((N, C, H + 2 * pad[0], W + 2 * pad[1]), np.int64)  # zero == "x - izp" of padding
        xp[:, :, pad[0]:pad[0] + H, pad[1]:pad[1] + W] = x.astype(np.int64) - izp
        ws = w.astype(np.int64) - wzp
        want = np.zeros((N, K, OH, OW), np.int64)
        cg, kg = C // grp, K // grp
        for oh in range(OH):
            for ow in range(OW):
                patch = xp[:, :, oh * st[0]:oh * st[0] + R, ow * st[1]:ow * st[1] + S]
                for g in range(grp):
                    want[:, g * kg:(g + 1) * kg, oh, ow] = np.tensordot(
                        patch[:, g * cg:(g + 1) * cg], ws[g * kg:(g + 1) * kg], axes=([1, 2, 3], [1, 2, 3]))
        want += b[None, :, None, None]
        assert np.array_equal(acc, want.astype(np.int32))
        scale = np.float32(ia) * np.float32(wa) / np.float32(oa)
        assert np.array_equal(y, _requant(want, scale, ozp))


def test_ip_against_matmul():
    rng = np.random.default_rng(9)
    x = rng.integers(0, 256, (4, 333), dtype=np.uint8)
    w = rng.integers(0, 256, (21, 333), dtype=np.uint8)
    b = rng.integers(-9000, 9000, 21).astype(np.int32)
    ia, izp, wa, wzp, oa, ozp = 0.02, 128, 0.004, 128, 0.09, 3
    y, acc = orc.ip_u8(x, w, b, ia, izp, wa, wzp, oa, ozp, return_acc=True)
    want = (x.astype(np.int64) - izp) @ (w.astype(np.int64) - wzp).T + b
    assert np.array_equal(acc, want.astype(np.int32))
    assert np.array_equal(y, _requant(want, np.float32(ia) * np.float32(wa) / np.float32(oa), ozp))


def test_int32_accumulator_wraps():
    # 70000 taps of 255 * 255 exceed 2^31: the accumulator must wrap like the reference's int32
    Kd = 70000
    x = np.full((1, Kd), 255, np.uint8)
    w = np.full((1, Kd), 255, np.uint8)
    _, acc = orc.ip_u8(x, w, None, 0.01, 0, 0.01, 0, 1.0, 0, return_acc=True)
    assert int(acc[0, 0]) == ((Kd * 255 * 255 + 2**31) % 2**32) - 2**31


def test_add_is_close_to_real_arithmetic():
    # the fixed-point add approximates (a0*(x0-z0) + a1*(x1-z1))/oa + oz to well within one LSB
    rng = np.random.default_rng(10)
    a = rng.integers(0, 256, 4000, dtype=np.uint8)
    b = rng.integers(0, 256, 4000, dtype=np.uint8)
    ia0, z0, ia1, z1, oa, oz = 0.031, 17, 0.0123, 201, 0.027, 99
    y = orc.add_u8(a, b, ia0, z0, ia1, z1, oa, oz).astype(np.float64)
    real = (ia0 * (a.astype(np.float64) - z0) + ia1 * (b.astype(np.float64) - z1)) / oa + oz
    assert np.max(np.abs(y - np.clip(real, 0, 255))) <= 1.0
    # operands are ordered by scale inside the op: swapping them changes nothing
    assert np.array_equal(orc.add_u8(a, b, ia0, z0, ia1, z1, oa, oz), orc.add_u8(b, a, ia1, z1, ia0, z0, oa, oz))
    # and a SUM eltwise over the same two inputs gives the same bytes
    assert np.array_equal(orc.add_u8(a, b, ia0, z0, ia1, z1, oa, oz),
                          orc.eltwise_u8([a, b], [ia0, ia1], [z0, z1], oa, oz, 1))


def test_quantize_formula():
    oa, oz = np.float32(0.02), 128
    x = np.array([0.0, 0.5 * 0.02 - 128 * 0.02, 1e9, -1e9, 0.02 * 0.49, 0.02 * 126.6], np.float32)
    beta = np.float32(-(oa * np.float32(oz)))
    q = (x - beta) / oa  # numpy fp32: IEEE subtract and divide
    want = np.where(q > 255, 255, np.where(q < 0, 0, np.floor(q.astype(np.float64) + 0.5))).astype(np.uint8)
    assert np.array_equal(orc.quantize_u8(x, oa, oz), want)
    d = orc.dequantize_u8(want, oa, oz)
    assert np.array_equal(d, (want.astype(np.int32) - oz).astype(np.float32) * oa)


def test_pool_closed_forms():
    x = np.arange(2 * 3 * 6 * 6, dtype=np.uint8).reshape(2, 3, 6, 6) * 3 % 251
    # identical scales and zero points: max pooling is a plain maximum
    y = orc.pool_u8(x, 2, 0, 2, 0, False, 0.05, 0, 0.05, 0)
    assert np.array_equal(y, x.reshape(2, 3, 3, 2, 3, 2).max(axis=(3, 5)))
    # global average, same scales: round-half-up mean to within the 15-bit multiplier's precision
    y = orc.pool_u8(x, 6, 0, 1, 1, True, 0.05, 0, 0.05, 0).astype(np.float64).ravel()
    assert np.max(np.abs(y - x.reshape(6, 36).mean(axis=1))) <= 0.51


def test_int8_conv_against_int64_tensordot():
    """Signed conv: zero padding, no zero points, clip to +-(2^obits - 1) then two's complement truncation."""
    rng = np.random.default_rng(31)
    for it in range(12):
        grp = int(rng.choice([1, 2]))
        C, K = grp * int(rng.integers(1, 6)), grp * int(rng.integers(1, 6))
        R, S = int(rng.integers(1, 4)), int(rng.integers(1, 4))
        H, W = int(rng.integers(R, 9)), int(rng.integers(S, 9))
        ph, pw, sh, sw = int(rng.integers(0, R)), int(rng.integers(0, S)), int(rng.integers(1, 3)), int(rng.integers(1, 3))
        x = rng.integers(-128, 128, (2, C, H, W), dtype=np.int8)
        w = rng.integers(-128, 128, (K, C // grp, R, S), dtype=np.int8)
        b = rng.integers(-5000, 5000, K).astype(np.int32)
        ia, wa, oa = rand_q(rng), rand_q(rng), rand_q(rng, 1e-2, 1.0)
        obits = int(rng.choice([8, 7, 5]))
        y, acc = orc.conv2d_i8(x, w, b, (ph, pw), (sh, sw), grp, ia, wa, oa, obits, return_acc=True)
        OH, OW = (H + 2 * ph - R) // sh + 1, (W + 2 * pw - S) // sw + 1
        xp = np.pad(x.astype(np.int64), ((0, 0), (0, 0), (ph, ph), (pw, pw)))
        ref = np.zeros((2, K, OH, OW), np.int64) + b[None, :, None, None]
        cg, kg = C // grp, K // grp
        for g in range(grp):
            for r in range(R):
                for s in range(S):
                    win = xp[:, g * cg:(g + 1) * cg, r:r + sh * (OH - 1) + 1:sh, s:s + sw * (OW - 1) + 1:sw]
                    ref[:, g * kg:(g + 1) * kg] += np.einsum("nchw,kc->nkhw", win, w[g * kg:(g + 1) * kg, :, r, s].astype(np.int64))
        assert np.array_equal(acc, ref)
        mult, shift = orc.quant_scale(np.float32(ia) * np.float32(wa) / np.float32(oa), 32)
        m = (1 << obits) - 1
        q = np.array([int(Fraction(int(v) * mult, 1 << shift) + Fraction(1, 2)) if (int(v) * mult) % (1 << shift) == 0
                      else (int(v) * mult + (1 << (shift - 1))) >> shift for v in ref.ravel()], dtype=np.int64)
        want = (np.clip(q, -m, m) & 255).astype(np.uint8).view(np.int8).reshape(ref.shape)
        assert np.array_equal(y, want), (it, obits)


def test_int8_quantize_formula():
    """clip(round_half_away(fp32(x * fp32(1/alpha))), +-(2^(bits-1) - 1)); dequantize is one fp32 product."""
    rng = np.random.default_rng(32)
    for bits in (8, 7, 4, 2):
        oa = np.float32(rand_q(rng, 5e-3, 0.1))
        x = (rng.standard_normal(4000) * 80 * oa).astype(np.float32)
        inv = np.float32(1.0 / np.float64(oa))
        p = (x * inv).astype(np.float64)
        r = np.sign(p) * np.floor(np.abs(p) + 0.5)
        lim = (1 << (bits - 1)) - 1
        want = np.clip(r, -lim, lim).astype(np.int8)
        got = orc.quantize_i8(x, oa, bits)
        assert np.array_equal(got, want), bits
        assert np.array_equal(orc.dequantize_i8(got, oa), got.astype(np.float32) * oa)


def test_concat_and_softmax_closed_forms():
    rng = np.random.default_rng(33)
    a, b = rng.integers(0, 256, (2, 3, 4, 5), dtype=np.uint8), rng.integers(0, 256, (2, 6, 4, 5), dtype=np.uint8)
    # equal scales and zero points: a plain concatenation along the channels
    assert np.array_equal(orc.concat_u8([a, b], [0.05, 0.05], [9, 9], 0.05, 9), np.concatenate([a, b], 1))
    # otherwise each piece is the affine map round_half_up((x - z) * m / 2^s) + oz of its input, saturated
    ia, iz, oa, oz = [0.02, 0.07], [100, 3], 0.04, 50
    y = orc.concat_u8([a, b], ia, iz, oa, oz)
    for piece, src, al, z in ((y[:, :3], a, ia[0], iz[0]), (y[:, 3:], b, ia[1], iz[1])):
        m, s = orc.quant_scale(np.float32(al) / np.float32(oa), 16)
        want = np.clip(((src.astype(np.int64) - z) * m + (1 << (s - 1)) >> s) + oz, 0, 255)
        assert np.array_equal(piece, want.astype(np.uint8))
    # softmax: within one step of the real-valued softmax of the dequantized input, and each pixel sums to ~1/oalpha
    x = rng.integers(0, 256, (3, 10, 2, 2), dtype=np.uint8)
    y = orc.softmax_u8(x, 1, 0.05, 128, 1.0 / 255, 0)
    z = 0.05 * (x.astype(np.float64) - 128)
    p = np.exp(z) / np.exp(z).sum(1, keepdims=True)
    assert np.abs(y.astype(np.float64) - p * 255).max() <= 0.5 + 1e-3
    # along another axis the same numbers appear with the axes swapped
    xt = np.ascontiguousarray(x.transpose(0, 2, 1, 3))
    assert np.array_equal(orc.softmax_u8(xt, 2, 0.05, 128, 1.0 / 255, 0).transpose(0, 2, 1, 3), y)


def test_per_channel_requantisation_is_pinned():
    """Per-channel weight scales (no counterpart in the reference CPU module, which reads walpha[0]): (a) with K equal
    scales the bytes are those of the per-tensor functions, which the compiled reference pins; (b) every channel equals
    exact rational rounding with ITS scale ialpha * walpha[k] / oalpha (fp32 operations in that order)."""
    rng = np.random.default_rng(77)
    N, C, H, W, K = 2, 6, 7, 5, 9
    x = rng.integers(0, 256, (N, C, H, W), dtype=np.uint8)
    w = rng.integers(0, 256, (K, C, 3, 3), dtype=np.uint8)
    b = rng.integers(-3000, 3000, K).astype(np.int32)
    ia, izp, wzp, oa, ozp = 0.021, 117, 131, 0.37, 11
    same = np.full(K, 0.0043, np.float32)
    y_t, acc = orc.conv2d_u8(x, w, b, 1, 1, 1, ia, izp, float(same[0]), wzp, oa, ozp, return_acc=True)
    assert np.array_equal(orc.conv2d_u8_per_channel(x, w, b, 1, 1, 1, ia, izp, same, wzp, oa, ozp), y_t)
    wa = np.exp(rng.uniform(np.log(5e-4), np.log(5e-2), K)).astype(np.float32)
    y = orc.conv2d_u8_per_channel(x, w, b, 1, 1, 1, ia, izp, wa, wzp, oa, ozp)
    assert len(np.unique(y)) > 20
    for k in range(K):
        scale = np.float32(np.float32(ia) * wa[k]) / np.float32(oa)
        assert np.array_equal(y[:, k], _requant(acc[:, k], scale, ozp)), k
        # and each channel alone is the per-tensor function with that channel's scale
        y_k = orc.conv2d_u8(x, w, b, 1, 1, 1, ia, izp, float(wa[k]), wzp, oa, ozp)
        assert np.array_equal(y[:, k], y_k[:, k]), k
    # int8 symmetric
    xs, ws = x.view(np.int8), w.view(np.int8)
    y8_t, acc8 = orc.conv2d_i8(xs, ws, b, 1, 1, 1, ia, float(same[0]), oa, 7, return_acc=True)
    assert np.array_equal(orc.requant_per_channel_i8(acc8, ia, same, oa, 7), y8_t)
    y8 = orc.requant_per_channel_i8(acc8, ia, wa, oa, 7)
    for k in range(K):
        assert np.array_equal(y8[:, k], orc.conv2d_i8(xs, ws, b, 1, 1, 1, ia, float(wa[k]), oa, 7)[:, k]), k


def test_dequantize_of_int32_accumulators_is_its_closed_form():
    """orc.dequantize_i32 has no reference counterpart (op_dequantize_run_u8 / _i8 read bytes only): it is pinned by
    what the arithmetic fixes - one int32 -> fp32 conversion, round to nearest even, and one fp32 multiply - computed
    independently by numpy, on values on both sides of 2^24 (where the conversion starts to round), the int32 extremes
    and ties."""
    rng = np.random.default_rng(5)
    acc = np.concatenate([rng.integers(-2**31, 2**31, 4000), rng.integers(-2**24 - 64, 2**24 + 64, 4000),
                          np.array([0, 1, -1, 2**24 + 1, 2**24 + 3, -(2**24) - 1, 2**25 + 2, 2**25 + 6, 2**31 - 1, -2**31])]).astype(np.int32)
    for alpha in (np.float32(0.02) * np.float32(0.005), np.float32(1.0), np.float32(3.1e-5)):
        want = acc.astype(np.float32) * np.float32(alpha)
        got = orc.dequantize_i32(acc, float(alpha))
        assert np.array_equal(got.view(np.uint32), want.view(np.uint32))
    # the conversion is to NEAREST EVEN: 2^24 + 1 -> 2^24, 2^24 + 3 -> 2^24 + 4
    assert orc.dequantize_i32(np.array([2**24 + 1, 2**24 + 3], np.int32), 1.0).tolist() == [2.0**24, 2.0**24 + 4]
