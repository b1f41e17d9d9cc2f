"""Loads the `hip` case module, compiled against the reference's own headers, into the REFERENCE art runtime
(oracle/_ref/libnart_ref.so: its libart + its CPU quant module, built from the reference's sources) and runs the
same engine.bin on both workspaces.  The hip workspace's output must equal the reference CPU module's and the
oracle's, bit for bit.  Batch 1 only: the reference's CPU conv aborts for larger batches
(art/modules/quant/src/op/conv_2d_uint8_impl.c:104), and images no smaller than the kernel: where one window
spans both the leading and the trailing padding (a 3x3 kernel on a 2x2 image) the reference's im2col_i16 region
split (art/modules/quant/src/utils/im2col.cpp:503-560) treats the window as touching the leading padding only and
its output departs from the convolution's definition, which the oracle and the kernels follow.  Run by tests/test_module_gpu.py in a process of its own."""
import os
import sys

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
sys.path.insert(0, ROOT)

from nart_amd import art, cases, engine  # noqa: E402

from oracle import casecpu  # noqa: E402


def same_bits(a, b):
    return np.array_equal(np.ascontiguousarray(a).view(np.uint8).ravel(), np.ascontiguousarray(b).view(np.uint8).ravel())


def main():
    rt = art.Runtime(os.path.join(ROOT, "oracle", "_ref", "libnart_ref.so"),
                     [os.path.join(ROOT, "nart_amd", "lib", "libart_module_hip_narttree.so")])
    hip, quant = rt.workspace("hip"), rt.workspace("quant")
    for case in (cases.single_conv(N=1), cases.single_fc(M=1, K=256, Nout=64), cases.resnet18(N=1, hw=96),
                 cases.mobilenet_v2(N=1, hw=96), cases.resnet50(N=1, hw=96)):
        print("case", case.name, flush=True)
        blob = engine.write_engine(case)
        p_hip = engine.Parade(rt, blob, [hip])
        p_cpu = engine.Parade(rt, blob, [quant])
        casecpu.zero_reference_conv_scratch(p_cpu)
        x = casecpu.random_input(case, 21)
        got, ref = p_hip.forward(x), p_cpu.forward(x)
        assert same_bits(got, ref), case.name + ": hip workspace differs from the reference CPU quant module"
        assert same_bits(got, casecpu.run_case(case, x)[case.output.name]), case.name + ": differs from the oracle"
        p_hip.delete()
        p_cpu.delete()
    hip.delete()
    quant.delete()
    print("refruntime_hip ok")


if __name__ == "__main__":
    main()
