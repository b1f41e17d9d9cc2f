"""Writes tests/golden/quant_ops.npz (uint8 operators) and tests/golden/quant_ops_int8.npz (the int8 symmetric
variants): seeded inputs and the outputs the REFERENCE CPU quant module (compiled from its own sources into
oracle/_ref by `make -C oracle ref`) gives for them.

Only runs where the reference tree is mounted; the .npz files it writes are committed so that the oracle
stays pinned to the reference on machines that never see it.
Usage: python tests/golden/make_golden.py [u8|int8|all]      (default: all)
"""
import json
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
sys.path[:0] = [ROOT, os.path.dirname(HERE)]

from nart_amd import art  # noqa: E402
import refrun  # noqa: E402


def main_int8(ws):
    rng = np.random.default_rng(20240602)
    out, meta = {}, {}

    def put(name, kind, ins, res, **args):
        for i, a in enumerate(ins):
            out["%s.in%d" % (name, i)] = a
        out[name + ".out"] = res
        meta[name] = {"kind": kind, "n_in": len(ins), "args": args}

    def i8(*shape):
        return rng.integers(-128, 128, shape, dtype=np.int8)

    convs = [("conv3x3", 2, 16, 16, 12, 3, 1, 1, 1, (0.02, 0.005, 0.05), 8),
             ("conv1x1_s2", 1, 24, 8, 9, 1, 0, 2, 1, (0.011, 0.007, 0.03), 7),
             ("conv5x5", 1, 3, 8, 20, 5, 2, 2, 1, (0.0157, 0.004, 0.06), 8),
             ("conv_dw", 1, 12, 12, 10, 3, 1, 1, 12, (0.03, 0.02, 0.008), 8),
             ("conv_grp", 1, 8, 6, 7, 3, 2, 1, 2, (0.02, 0.006, 0.07), 4)]
    for name, N, C, K, H, R, pad, st, grp, q, obits in convs:
        x, w = i8(N, C, H, H), i8(K, C // grp, R, R)
        b = rng.integers(-3000, 3000, K).astype(np.int32)
        put(name, "conv", [x, w, b], refrun.conv2d_i8(ws, x, w, b, pad, st, grp, *q, obits=obits),
            pad=pad, stride=st, group=grp, q=list(q), obits=obits)
    x, w = i8(3, 200), i8(17, 200)
    b = rng.integers(-9000, 9000, 17).astype(np.int32)
    q = (0.013, 0.0071, 0.093)
    put("ip", "ip", [x, w, b], refrun.ip_i8(ws, x, w, b, *q, obits=7), q=list(q), obits=7)
    xf = (rng.standard_normal((1, 3, 16, 16)) * 3).astype(np.float32)
    xf.flat[:300] = (np.arange(300, dtype=np.float32) * 0.5 - 75) * np.float32(0.02)
    for bits in (8, 4):
        yq = refrun.quantize_i8(ws, xf, 0.02, bits)
        put("quantize%d" % bits, "quantize", [xf], yq, q=[0.02], obits=bits)
        put("dequantize%d" % bits, "dequantize", [yq], refrun.dequantize_i8(ws, yq, 0.02, bits), q=[0.02])
    out["meta"] = np.frombuffer(json.dumps(meta).encode(), dtype=np.uint8)
    np.savez_compressed(os.path.join(HERE, "quant_ops_int8.npz"), **out)
    print("int8: wrote", len(meta), "cases")


def main():
    which = sys.argv[1] if len(sys.argv) > 1 else "all"
    ws = art.Runtime(os.path.join(ROOT, "oracle", "_ref", "libnart_ref.so")).workspace("quant")
    if which in ("int8", "all"):
        main_int8(ws)
    if which == "int8":
        return
    rng = np.random.default_rng(20240601)
    out, meta = {}, {}

    def put(name, kind, ins, res, **args):
        for i, a in enumerate(ins):
            out["%s.in%d" % (name, i)] = a
        out[name + ".out"] = res
        meta[name] = {"kind": kind, "n_in": len(ins), "args": args}

    def u8(*shape):
        return rng.integers(0, 256, shape, dtype=np.uint8)

    convs = [("conv3x3", 1, 16, 16, 12, 3, 1, 1, 1, (0.02, 128, 0.005, 128, 0.05, 0)),
             ("conv1x1_s2", 1, 24, 8, 9, 1, 0, 2, 1, (0.011, 90, 0.007, 128, 0.03, 17)),
             ("conv7x7_stem", 1, 3, 8, 20, 7, 3, 2, 1, (0.0157, 114, 0.004, 128, 0.06, 0)),
             ("conv_dw", 1, 12, 12, 10, 3, 1, 1, 12, (0.03, 5, 0.02, 131, 0.08, 250)),
             ("conv_wzp", 1, 8, 6, 7, 3, 2, 1, 2, (0.02, 33, 0.006, 77, 0.07, 128))]
    for name, N, C, K, H, R, pad, st, grp, q in convs:
        x, w = u8(N, C, H, H), u8(K, C // grp, R, R)
        b = rng.integers(-3000, 3000, K).astype(np.int32)
        put(name, "conv", [x, w, b], refrun.conv2d_u8(ws, x, w, b, pad, st, grp, *q),
            pad=pad, stride=st, group=grp, q=list(q))
    x, w = u8(3, 200), u8(17, 200)
    b = rng.integers(-9000, 9000, 17).astype(np.int32)
    q = (0.013, 131, 0.0071, 128, 0.093, 3)
    put("ip", "ip", [x, w, b], refrun.ip_u8(ws, x, w, b, *q), q=list(q))
    a, b2, c = u8(1, 5, 7, 6), u8(1, 5, 7, 6), u8(1, 5, 7, 6)
    q = (0.031, 17, 0.0123, 201, 0.027, 99)
    put("add", "add", [a, b2], refrun.add_u8(ws, a, b2, *q), q=list(q))
    for operation, nm in ((1, "eltwise_sum3"), (2, "eltwise_max3")):
        ia, iz = [0.031, 0.0123, 0.02], [17, 201, 128]
        put(nm, "eltwise", [a, b2, c], refrun.eltwise_u8(ws, [a, b2, c], ia, iz, 0.04, 60, operation),
            ialpha=ia, izp=iz, oalpha=0.04, ozp=60, operation=operation)
    q = (0.031, 117, 0.02, 40)
    put("relu", "relu", [a], refrun.relu_u8(ws, a, *q), q=list(q))
    xp = u8(2, 3, 13, 13)
    for nm, k, pad, st, method, cm in (("pool_max_3x3s2p1", 3, 1, 2, 0, False), ("pool_max_ceil", 3, 1, 2, 0, True),
                                       ("pool_avg_global", 13, 0, 1, 1, True), ("pool_avg_pad", 3, 1, 2, 1, True)):
        q = (0.02, 30, 0.025, 10)
        put(nm, "pool", [xp], refrun.pool_u8(ws, xp, k, pad, st, method, cm, *q),
            kernel=k, pad=pad, stride=st, method=method, ceil_mode=cm, q=list(q))
    xf = (rng.standard_normal((1, 3, 16, 16)) * 3).astype(np.float32)
    xf.flat[:256] = (np.arange(256, dtype=np.float32) + 0.5 - 128) * np.float32(0.02)
    yq = refrun.quantize_u8(ws, xf, 0.02, 128)
    put("quantize", "quantize", [xf], yq, q=[0.02, 128])
    put("dequantize", "dequantize", [yq], refrun.dequantize_u8(ws, yq, 0.02, 128), q=[0.02, 128])
    out["meta"] = np.frombuffer(json.dumps(meta).encode(), dtype=np.uint8)
    np.savez_compressed(os.path.join(HERE, "quant_ops.npz"), **out)
    print("wrote", len(meta), "cases")


if __name__ == "__main__":
    main()
