"""The drop-in boundary on a real GPU: an engine.bin written by nart_amd.engine (the file the unchanged quant
converter would hand over) is loaded by an art runtime with the `hip` workspace selected, run, and its
output compared with the CPU oracle, bit for bit.

Two runtimes are driven through the same C ABI:
  * the repo's own host core (nart_amd/lib/libart.so) + libart_module_hip.so;
  * where it was built (oracle/_ref, from the reference's own sources): the REFERENCE libart with the module
    compiled against the reference's own headers — the module is then a true plug-in of the unmodified
    runtime, and the reference's CPU quant module runs the same file in the same process as a second checker.
"""
import os

import numpy as np
import pytest

pytestmark = pytest.mark.gpu

torch = pytest.importorskip("torch")

from nart_amd import art, cases, engine  # noqa: E402

from oracle import casecpu  # noqa: E402

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
LIB = os.path.join(ROOT, "nart_amd", "lib")
REF_SO = os.path.join(ROOT, "oracle", "_ref", "libnart_ref.so")
HIP_FOR_REF = os.path.join(LIB, "libart_module_hip_narttree.so")


def small_cases():
    return [cases.single_conv(N=1), cases.single_fc(M=5, K=256, Nout=64), cases.resnet18(N=2, hw=96),
            cases.mobilenet_v2(N=1, hw=96), cases.resnet50(N=2, hw=64)]


def same_bits(a, b):
    return a.shape == b.shape and np.array_equal(np.ascontiguousarray(a).view(np.uint8), np.ascontiguousarray(b).view(np.uint8))


@pytest.fixture(scope="module")
def own_rt():
    return art.Runtime(os.path.join(LIB, "libart.so"), [os.path.join(LIB, "libart_module_hip.so")])


def test_engine_file_runs_on_hip_workspace(own_rt):
    ws = own_rt.workspace("hip")
    assert ws.name.startswith("hip")
    for case in small_cases():
        print("case", case.name, flush=True)
        p = engine.Parade(own_rt, engine.write_engine(case), [ws])
        for seed in (7, 8):  # the second pass re-uses every prepared plan and buffer
            x = casecpu.random_input(case, seed)
            got = p.forward(x).reshape(case.output.shape)
            want = casecpu.run_case(case, x)[case.output.name]
            assert same_bits(got, want), (case.name, seed)
        p.delete()
    ws.delete()


def test_version2_engine_file(own_rt):
    """Version-2 engine files (an optional pre-processing block after every input declaration) load on the repo's core
    and run on the hip workspace; the block is handed back unchanged."""
    ws = own_rt.workspace("hip")
    case = cases.resnet18(N=2, hw=96)
    x = casecpu.random_input(case, 4)
    want = casecpu.run_case(case, x)[case.output.name]
    tf = (0x11, 2, (1.5, 2.5, 3.5), (0.25, 0.5, 0.75), (7.0, 8.0, 9.0))
    for transform in (None, tf):
        p = engine.Parade(own_rt, engine.write_engine(case, version=2, transform=transform), [ws])
        assert same_bits(p.forward(x).reshape(case.output.shape), want)
        if transform:
            assert p.transform_param() == (0x11, (1.5, 2.5, 3.5), (0.25, 0.5, 0.75), (7.0, 8.0, 9.0))
        p.delete()
    ws.delete()


def test_prepare_twice_and_batch_reshape(own_rt):
    """parade_apply_reshape re-infers every shape and calls prepare again (art/src/parade.c:199-215): plans and
    device buffers must follow the new batch size."""
    ws = own_rt.workspace("hip")
    case1, case3 = cases.resnet18(N=1, hw=64), cases.resnet18(N=3, hw=64)
    p = engine.Parade(own_rt, engine.write_engine(case1), [ws])
    x1 = casecpu.random_input(case1, 1)
    assert same_bits(p.forward(x1).reshape(case1.output.shape), casecpu.run_case(case1, x1)[case1.output.name])
    own_rt.core.parade_prepare(p.ptr)  # idempotent
    assert same_bits(p.forward(x1).reshape(case1.output.shape), casecpu.run_case(case1, x1)[case1.output.name])
    inp = p.inputs()[0]
    inp.set_shape(case3.input.shape)
    assert own_rt.core.parade_apply_reshape(p.ptr)
    x3 = casecpu.random_input(case3, 2)
    got = p.forward(x3).reshape(case3.output.shape)
    assert same_bits(got, casecpu.run_case(case3, x3)[case3.output.name])
    p.delete()
    ws.delete()


def test_single_ops_through_the_op_api(own_rt):
    """workspace_new_op / op_config / op_prepare / op_run on device tensors, the way the reference's tests drive a
    module without a file."""
    from oracle import orc
    ws = own_rt.workspace("hip")
    rng = np.random.default_rng(11)
    x = rng.integers(0, 256, (2, 24, 9, 11), dtype=np.uint8)
    w = rng.integers(0, 256, (40, 24, 3, 3), dtype=np.uint8)
    b = rng.integers(-5000, 5000, 40).astype(np.int32)
    q = dict(ialpha=0.031, izp=77, walpha=0.0042, wzp=131, oalpha=0.09, ozp=13)
    tx, tw, tb = ws.tensor(x), ws.tensor(w), ws.tensor(b)
    conv = ws.conv2d(tx, tw, tb, 1, 2, 1, q).prepare().run()
    want = orc.conv2d_u8(x, w, b, 1, 2, 1, 0.031, 77, 0.0042, 131, 0.09, 13)
    assert same_bits(conv.output(0).numpy(), want)
    relu = ws.relu(conv.output(0), dict(ialpha=0.09, izp=13, oalpha=0.05, ozp=3)).prepare().run()
    want_r = orc.relu_u8(want, 0.09, 13, 0.05, 3)
    assert same_bits(relu.output(0).numpy(), want_r)
    elt = ws.eltwise([conv.output(0), relu.output(0)], dict(ialpha=[0.09, 0.05], izp=[13, 3], oalpha=0.11, ozp=9),
                     coeff=[1.0, 0.5]).prepare().run()
    want_e = orc.eltwise_u8([want, want_r], [0.09, 0.05], [13, 3], 0.11, 9, operation=1, coeff=[1.0, 0.5])
    assert same_bits(elt.output(0).numpy(), want_e)
    # overwrite the input through the host mirror: the next run must see it
    x2 = rng.integers(0, 256, x.shape, dtype=np.uint8)
    tx.write(x2)
    conv.run()
    assert same_bits(conv.output(0).numpy(), orc.conv2d_u8(x2, w, b, 1, 2, 1, 0.031, 77, 0.0042, 131, 0.09, 13))
    for o in (elt, relu, conv):
        o.delete()
    ws.delete()


def test_per_channel_weight_scales_through_the_op_api(own_rt):
    """A walpha array with one entry per output channel selects per-channel requantisation (the convention of the
    reference's CUDA module, cuda_quant/src/op/conv_2d_quant.cu:751-764); one entry stays per tensor.  conv_2d and ip."""
    from oracle import orc
    ws = own_rt.workspace("hip")
    rng = np.random.default_rng(12)
    x = rng.integers(0, 256, (2, 24, 9, 11), dtype=np.uint8)
    w = rng.integers(0, 256, (40, 24, 3, 3), dtype=np.uint8)
    b = rng.integers(-5000, 5000, 40).astype(np.int32)
    wa = np.exp(rng.uniform(np.log(1e-3), np.log(2e-2), 40)).astype(np.float32)
    q = dict(ialpha=0.031, izp=77, walpha=wa, wzp=128, oalpha=0.9, ozp=13)
    tx, tw, tb = ws.tensor(x), ws.tensor(w), ws.tensor(b)
    conv = ws.conv2d(tx, tw, tb, 1, 2, 1, q).prepare().run()
    want = orc.conv2d_u8_per_channel(x, w, b, 1, 2, 1, 0.031, 77, wa, 128, 0.9, 13)
    assert same_bits(conv.output(0).numpy(), want) and len(np.unique(want)) > 8
    conv.prepare().run()  # prepared again with the same scales: the plan is kept
    assert same_bits(conv.output(0).numpy(), want)
    xf = rng.integers(0, 256, (6, 256), dtype=np.uint8)
    wf = rng.integers(0, 256, (37, 256), dtype=np.uint8)
    waf = np.exp(rng.uniform(np.log(1e-3), np.log(2e-2), 37)).astype(np.float32)
    ip = ws.ip(ws.tensor(xf), ws.tensor(wf), None, dict(ialpha=0.02, izp=128, walpha=waf, wzp=128, oalpha=2.5, ozp=100)).prepare().run()
    _, acc = orc.ip_u8(xf, wf, None, 0.02, 128, float(waf[0]), 128, 2.5, 100, return_acc=True)
    want_ip = orc.requant_per_channel_u8(acc, 0.02, waf, 2.5, 100)
    assert same_bits(ip.output(0).numpy().reshape(6, 37), want_ip) and len(np.unique(want_ip)) > 8
    for o in (ip, conv):
        o.delete()
    # The reference's converter writes one walpha entry per constant input - the weights' scale, then the bias's
    # (python/nart/modules/quant.py:178-208) - and the CPU module reads the first (conv_2d_uint8_impl.c:61, ip.cpp:148): a
    # two-channel layer with a bias carries two entries and is still per tensor.
    x2 = rng.integers(0, 256, (1, 16, 6, 6), dtype=np.uint8)
    w2 = rng.integers(0, 256, (2, 16, 3, 3), dtype=np.uint8)
    b2 = rng.integers(-3000, 3000, 2).astype(np.int32)
    wa2 = np.array([0.004, 0.004 * 0.031], np.float32)
    conv2 = ws.conv2d(ws.tensor(x2), ws.tensor(w2), ws.tensor(b2), 1, 1, 1,
                      dict(ialpha=0.031, izp=77, walpha=wa2, wzp=128, oalpha=0.4, ozp=13)).prepare().run()
    want2 = orc.conv2d_u8(x2, w2, b2, 1, 1, 1, 0.031, 77, float(wa2[0]), 128, 0.4, 13)
    assert same_bits(conv2.output(0).numpy(), want2) and len(np.unique(want2)) > 8
    xf2 = rng.integers(0, 256, (5, 64), dtype=np.uint8)
    wf2 = rng.integers(0, 256, (2, 64), dtype=np.uint8)
    ip2 = ws.ip(ws.tensor(xf2), ws.tensor(wf2), ws.tensor(b2),
                dict(ialpha=0.02, izp=128, walpha=wa2, wzp=128, oalpha=0.7, ozp=100)).prepare().run()
    want_ip2 = orc.ip_u8(xf2, wf2, b2, 0.02, 128, float(wa2[0]), 128, 0.7, 100)
    assert same_bits(ip2.output(0).numpy().reshape(5, 2), want_ip2.reshape(5, 2))
    # without a bias two entries for two channels ARE one per channel
    conv3 = ws.conv2d(ws.tensor(x2), ws.tensor(w2), None, 1, 1, 1,
                      dict(ialpha=0.031, izp=77, walpha=wa2 * np.float32([1, 40]), wzp=128, oalpha=0.4, ozp=13)).prepare().run()
    want3 = orc.conv2d_u8_per_channel(x2, w2, None, 1, 1, 1, 0.031, 77, wa2 * np.float32([1, 40]), 128, 0.4, 13)
    assert same_bits(conv3.output(0).numpy(), want3)
    for o in (conv2, ip2, conv3):
        o.delete()
    ws.delete()


def test_convolution_and_add_run_as_one_kernel(own_rt):
    """A convolution whose output only an add reads leaves its launch to that add (one fused kernel, the convolution's
    output is never written); whoever asks for the elided tensor afterwards gets it computed on demand.  Results are
    those of the two operators run one after the other; a convolution with a second reader is not deferred."""
    import ctypes as C
    from oracle import orc
    fused = own_rt.libs[1].hip_module_fused_adds
    fused.restype = C.c_long
    ws = own_rt.workspace("hip")
    rng = np.random.default_rng(21)
    x = rng.integers(0, 256, (2, 64, 9, 11), dtype=np.uint8)
    w = rng.integers(0, 256, (128, 64, 1, 1), dtype=np.uint8)
    b = rng.integers(-5000, 5000, 128).astype(np.int32)
    r = rng.integers(0, 256, (2, 128, 9, 11), dtype=np.uint8)
    q = dict(ialpha=0.031, izp=77, walpha=0.0042, wzp=128, oalpha=0.09, ozp=13)
    want_c = orc.conv2d_u8(x, w, b, 0, 1, 1, 0.031, 77, 0.0042, 128, 0.09, 13)
    for conv_first in (True, False):
        tx, tr = ws.tensor(x), ws.tensor(r)
        conv = ws.conv2d(tx, ws.tensor(w), ws.tensor(b), 0, 1, 1, q).prepare()
        ins = [conv.output(0), tr] if conv_first else [tr, conv.output(0)]
        qa = dict(ialpha=[0.09, 0.05] if conv_first else [0.05, 0.09], izp=[13, 200] if conv_first else [200, 13], oalpha=0.12, ozp=31)
        add = ws.add(ins[0], ins[1], qa).prepare()
        want_a = orc.add_u8(want_c, r, 0.09, 13, 0.05, 200, 0.12, 31) if conv_first else orc.add_u8(r, want_c, 0.05, 200, 0.09, 13, 0.12, 31)
        n0 = fused()
        for _ in range(2):  # the second pass defers and fuses again
            conv.run()
            add.run()
            assert same_bits(add.output(0).numpy(), want_a), conv_first
        assert fused() == n0 + 2
        assert same_bits(conv.output(0).numpy(), want_c)  # elided so far: computed now
        # new input through the host mirror, then only the convolution: the deferred launch happens when the output is read
        x2 = rng.integers(0, 256, x.shape, dtype=np.uint8)
        tx.write(x2)
        conv.run()
        assert same_bits(conv.output(0).numpy(), orc.conv2d_u8(x2, w, b, 0, 1, 1, 0.031, 77, 0.0042, 128, 0.09, 13))
        tx.write(x)
        # a second reader: no deferral from now on (decided at prepare + first run), results unchanged
        relu = ws.relu(conv.output(0), dict(ialpha=0.09, izp=13, oalpha=0.05, ozp=3)).prepare()
        conv.prepare()
        n1 = fused()
        conv.run()
        add.run()
        relu.run()
        assert fused() == n1
        assert same_bits(add.output(0).numpy(), want_a) and same_bits(relu.output(0).numpy(), orc.relu_u8(want_c, 0.09, 13, 0.05, 3))
        for o in (relu, add, conv):
            o.delete()
    ws.delete()


def test_plain_eltwise_sum_fuses_like_add(own_rt):
    """Caffe-style graphs carry the residual sum as Eltwise(SUM): two inputs with unit coefficients give add's bytes and
    take the same fused path; other coefficients, MAX and three inputs run as operators of their own."""
    import ctypes as C
    from oracle import orc
    fused = own_rt.libs[1].hip_module_fused_adds
    fused.restype = C.c_long
    ws = own_rt.workspace("hip")
    rng = np.random.default_rng(23)
    x = rng.integers(0, 256, (2, 128, 7, 7), dtype=np.uint8)
    w = rng.integers(0, 256, (256, 128, 1, 1), dtype=np.uint8)
    r = rng.integers(0, 256, (2, 256, 7, 7), dtype=np.uint8)
    q = dict(ialpha=0.031, izp=77, walpha=0.0042, wzp=128, oalpha=0.09, ozp=13)
    want_c = orc.conv2d_u8(x, w, None, 0, 1, 1, 0.031, 77, 0.0042, 128, 0.09, 13)
    qa = dict(ialpha=[0.05, 0.09], izp=[200, 13], oalpha=0.12, ozp=31)
    for coeff, op, expect in ((None, 1, 1), ([1.0, 1.0], 1, 1), ([1.0, 0.5], 1, 0), (None, 2, 0)):
        conv = ws.conv2d(ws.tensor(x), ws.tensor(w), None, 0, 1, 1, q).prepare()
        elt = ws.eltwise([ws.tensor(r), conv.output(0)], qa, operation=op, coeff=coeff).prepare()
        n0 = fused()
        conv.run()
        elt.run()
        want = orc.eltwise_u8([r, want_c], [0.05, 0.09], [200, 13], 0.12, 31, operation=op, coeff=coeff)
        assert same_bits(elt.output(0).numpy(), want), (coeff, op)
        assert fused() == n0 + expect, (coeff, op)
        if expect:
            assert same_bits(want, orc.add_u8(r, want_c, 0.05, 200, 0.09, 13, 0.12, 31))
        elt.delete()
        conv.delete()
    ws.delete()


def test_add_and_the_next_1x1_convolution_run_as_one_kernel(own_rt):
    """conv_2d (64 -> 256, 1x1) -> add -> conv_2d (256 -> 64, 1x1) [-> relu]: the first convolution defers to the add, the
    add defers to the convolution that reads the sum, and that convolution (or the relu behind it) launches all of it as
    one kernel; the sum is written as well, for its other readers.  A host that reads the sum before the second
    convolution runs gets convolution + add as one kernel and the second convolution on its own.  Same bytes as the
    operators run one by one, pass after pass."""
    import ctypes as C
    from oracle import orc
    chained = own_rt.libs[1].hip_module_chained_convs
    chained.restype = C.c_long
    ws = own_rt.workspace("hip")
    rng = np.random.default_rng(24)
    x = rng.integers(0, 256, (2, 64, 24, 24), dtype=np.uint8)
    w = rng.integers(0, 256, (256, 64, 1, 1), dtype=np.uint8)
    b = rng.integers(-5000, 5000, 256).astype(np.int32)
    r = rng.integers(0, 256, (2, 256, 24, 24), dtype=np.uint8)
    w2 = rng.integers(0, 256, (64, 256, 1, 1), dtype=np.uint8)
    b2 = rng.integers(-5000, 5000, 64).astype(np.int32)
    q = dict(ialpha=0.031, izp=77, walpha=0.0042, wzp=128, oalpha=0.09, ozp=13)
    q2 = dict(ialpha=0.12, izp=31, walpha=0.003, wzp=128, oalpha=0.4, ozp=40)
    want_c = orc.conv2d_u8(x, w, b, 0, 1, 1, 0.031, 77, 0.0042, 128, 0.09, 13)
    want_a = orc.add_u8(r, want_c, 0.05, 200, 0.09, 13, 0.12, 31)
    want_2 = orc.conv2d_u8(want_a, w2, b2, 0, 1, 1, 0.12, 31, 0.003, 128, 0.4, 40)
    want_r = orc.relu_u8(want_2, 0.4, 40, 0.4, 40)
    for with_relu, peek, expect in ((True, False, 1), (False, False, 1), (True, True, 0)):
        conv = ws.conv2d(ws.tensor(x), ws.tensor(w), ws.tensor(b), 0, 1, 1, q).prepare()
        add = ws.add(ws.tensor(r), conv.output(0), dict(ialpha=[0.05, 0.09], izp=[200, 13], oalpha=0.12, ozp=31)).prepare()
        conv2 = ws.conv2d(add.output(0), ws.tensor(w2), ws.tensor(b2), 0, 1, 1, q2).prepare()
        relu = ws.relu(conv2.output(0), dict(ialpha=0.4, izp=40, oalpha=0.4, ozp=40)).prepare() if with_relu else None
        for rep in range(2):
            n0 = chained()
            conv.run()
            add.run()
            if peek:
                assert same_bits(add.output(0).numpy(), want_a)
            conv2.run()
            if relu:
                relu.run()
            last = relu if relu else conv2
            assert same_bits(last.output(0).numpy(), want_r if relu else want_2), (with_relu, peek, rep)
            assert chained() == n0 + expect, (with_relu, peek, rep)
            assert same_bits(add.output(0).numpy(), want_a), (with_relu, peek, rep)
        assert same_bits(conv2.output(0).numpy(), want_2)  # elided behind the relu: computed on demand
        assert same_bits(conv.output(0).numpy(), want_c)
        for o in ([relu] if relu else []) + [conv2, add, conv]:
            o.delete()
    ws.delete()


def test_whole_bottleneck_block_runs_as_one_kernel(own_rt):
    """conv_2d (1024 -> 256, 1x1) -> conv_2d (3x3) -> conv_2d (256 -> 1024, 1x1) -> add with the block's input: the three
    convolutions leave their launches to the add, whose run() launches hipq_bottleneck_run.  A host that reads an
    intermediate tensor in between gets the operators one by one (the hooks settle in a chain); every tensor of the
    block can still be read afterwards.  Same bytes as the oracle's four operators, pass after pass."""
    import ctypes as C
    from oracle import orc
    blocks = own_rt.libs[1].hip_module_fused_blocks
    blocks.restype = C.c_long
    ws = own_rt.workspace("hip")
    rng = np.random.default_rng(31)
    x = rng.integers(0, 256, (2, 1024, 14, 14), dtype=np.uint8)
    shapes = ((256, 1024, 1), (256, 256, 3), (1024, 256, 1))
    ws_w = [rng.integers(1, 256, (K, Cc, k, k), dtype=np.uint8) for K, Cc, k in shapes]
    bs = [rng.integers(-20000, 20000, K).astype(np.int32) for K, _, _ in shapes]
    qs = [dict(ialpha=0.05, izp=9, walpha=0.0011, wzp=128, oalpha=0.06, ozp=0),
          dict(ialpha=0.06, izp=0, walpha=0.0016, wzp=128, oalpha=0.055, ozp=0),
          dict(ialpha=0.055, izp=0, walpha=0.0035, wzp=128, oalpha=0.07, ozp=121)]
    t = x
    wants = []
    for w, b, q, (K, Cc, k) in zip(ws_w, bs, qs, shapes):
        t = orc.conv2d_u8(t, w, b, k // 2, 1, 1, q["ialpha"], q["izp"], q["walpha"], 128, q["oalpha"], q["ozp"])
        wants.append(t)
    for res_first in (False, True):
        want = orc.add_u8(x, t, 0.05, 9, 0.07, 121, 0.09, 0) if res_first else orc.add_u8(t, x, 0.07, 121, 0.05, 9, 0.09, 0)
        assert len(np.unique(want)) > 32
        for peek, expect in ((None, 1), (0, 0), (1, 0)):
            tx = ws.tensor(x)
            convs, cur = [], tx
            for w, b, q, (K, Cc, k) in zip(ws_w, bs, qs, shapes):
                convs.append(ws.conv2d(cur, ws.tensor(w), ws.tensor(b), k // 2, 1, 1, q).prepare())
                cur = convs[-1].output(0)
            ins = [tx, cur] if res_first else [cur, tx]
            qa = dict(ialpha=[0.05, 0.07] if res_first else [0.07, 0.05], izp=[9, 121] if res_first else [121, 9], oalpha=0.09, ozp=0)
            add = ws.add(ins[0], ins[1], qa).prepare()
            for rep in range(2):
                n0 = blocks()
                for j, c in enumerate(convs):
                    c.run()
                    if peek == j:
                        assert same_bits(c.output(0).numpy(), wants[j]), (res_first, peek, rep)
                add.run()
                assert same_bits(add.output(0).numpy(), want), (res_first, peek, rep)
                assert blocks() == n0 + expect, (res_first, peek, rep)
            for j, c in enumerate(convs):  # never written by the fused launch: computed on demand
                assert same_bits(c.output(0).numpy(), wants[j]), (res_first, peek, j)
            for o in [add] + convs[::-1]:
                o.delete()
    ws.delete()


def test_whole_block_and_the_next_stage_first_layer_run_as_one_kernel(own_rt):
    """The same block followed by conv_2d (1024 -> 512, 1x1) that reads the sum: the add leaves its launch to that
    convolution, whose run() launches hipq_bottleneck_run_conv for all five operators; the sum is written as well.  A host
    that reads the sum before that convolution has run gets the block's four operators as one launch and the
    convolution as its own."""
    import ctypes as C
    from oracle import orc
    blocks = own_rt.libs[1].hip_module_fused_blocks
    blocks.restype = C.c_long
    chained = own_rt.libs[1].hip_module_chained_convs
    chained.restype = C.c_long
    ws = own_rt.workspace("hip")
    rng = np.random.default_rng(33)
    x = rng.integers(0, 256, (2, 1024, 14, 14), dtype=np.uint8)
    shapes = ((256, 1024, 1), (256, 256, 3), (1024, 256, 1))
    ws_w = [rng.integers(1, 256, (K, Cc, k, k), dtype=np.uint8) for K, Cc, k in shapes]
    bs = [rng.integers(-20000, 20000, K).astype(np.int32) for K, _, _ in shapes]
    qs = [dict(ialpha=0.05, izp=9, walpha=0.0011, wzp=128, oalpha=0.06, ozp=0),
          dict(ialpha=0.06, izp=0, walpha=0.0016, wzp=128, oalpha=0.055, ozp=0),
          dict(ialpha=0.055, izp=0, walpha=0.0035, wzp=128, oalpha=0.07, ozp=121)]
    wn, bn = rng.integers(1, 256, (512, 1024, 1, 1), dtype=np.uint8), rng.integers(-20000, 20000, 512).astype(np.int32)
    qn = dict(ialpha=0.09, izp=0, walpha=0.0011, wzp=128, oalpha=0.08, ozp=0)
    t = x
    for w, b, q, (K, Cc, k) in zip(ws_w, bs, qs, shapes):
        t = orc.conv2d_u8(t, w, b, k // 2, 1, 1, q["ialpha"], q["izp"], q["walpha"], 128, q["oalpha"], q["ozp"])
    want = orc.add_u8(t, x, 0.07, 121, 0.05, 9, 0.09, 0)
    wantn = orc.conv2d_u8(want, wn, bn, 0, 1, 1, 0.09, 0, 0.0011, 128, 0.08, 0)
    assert len(np.unique(wantn)) > 32
    for peek, expect_chain in ((False, 1), (True, 0)):
        tx = ws.tensor(x)
        convs, cur = [], tx
        for w, b, q, (K, Cc, k) in zip(ws_w, bs, qs, shapes):
            convs.append(ws.conv2d(cur, ws.tensor(w), ws.tensor(b), k // 2, 1, 1, q).prepare())
            cur = convs[-1].output(0)
        add = ws.add(cur, tx, dict(ialpha=[0.07, 0.05], izp=[121, 9], oalpha=0.09, ozp=0)).prepare()
        nxt = ws.conv2d(add.output(0), ws.tensor(wn), ws.tensor(bn), 0, 1, 1, qn).prepare()
        for rep in range(2):
            b0, c0 = blocks(), chained()
            for c in convs:
                c.run()
            add.run()
            if peek:
                assert same_bits(add.output(0).numpy(), want), (peek, rep)
            nxt.run()
            assert same_bits(nxt.output(0).numpy(), wantn), (peek, rep)
            assert same_bits(add.output(0).numpy(), want), (peek, rep)
            assert blocks() == b0 + 1 and chained() == c0 + expect_chain, (peek, rep, blocks() - b0, chained() - c0)
        for o in [nxt, add] + convs[::-1]:
            o.delete()
    ws.delete()


def test_block_tail_and_next_convolution_run_as_one_kernel(own_rt):
    """conv_2d (3x3, 128 -> 128) -> conv_2d (128 -> 512, 1x1) -> add with any residual -> conv_2d (512 -> 128, 1x1): the 3x3
    and the widening convolution leave their launches to the add, the add leaves its own to the convolution that reads
    the sum, and that convolution's run() launches hipq_bottleneck_tail_run for all four.  Without a chained reader the
    add launches the first three.  A host that peeks gets the operators one by one."""
    import ctypes as C
    from oracle import orc
    tails = own_rt.libs[1].hip_module_fused_tails
    tails.restype = C.c_long
    chained = own_rt.libs[1].hip_module_chained_convs
    chained.restype = C.c_long
    ws = own_rt.workspace("hip")
    rng = np.random.default_rng(32)
    t1 = rng.integers(0, 256, (2, 128, 28, 28), dtype=np.uint8)
    r = rng.integers(0, 256, (2, 512, 28, 28), dtype=np.uint8)
    w2, b2 = rng.integers(1, 256, (128, 128, 3, 3), dtype=np.uint8), rng.integers(-20000, 20000, 128).astype(np.int32)
    w3, b3 = rng.integers(1, 256, (512, 128, 1, 1), dtype=np.uint8), rng.integers(-9000, 9000, 512).astype(np.int32)
    wn, bn = rng.integers(1, 256, (128, 512, 1, 1), dtype=np.uint8), rng.integers(-9000, 9000, 128).astype(np.int32)
    q2 = dict(ialpha=0.05, izp=0, walpha=0.0022, wzp=128, oalpha=0.055, ozp=0)
    q3 = dict(ialpha=0.055, izp=0, walpha=0.005, wzp=128, oalpha=0.07, ozp=121)
    qn = dict(ialpha=0.09, izp=0, walpha=0.0024, wzp=128, oalpha=0.06, ozp=0)
    want2 = orc.conv2d_u8(t1, w2, b2, 1, 1, 1, 0.05, 0, 0.0022, 128, 0.055, 0)
    want3 = orc.conv2d_u8(want2, w3, b3, 0, 1, 1, 0.055, 0, 0.005, 128, 0.07, 121)
    want_a = orc.add_u8(want3, r, 0.07, 121, 0.04, 77, 0.09, 0)
    want_n = orc.conv2d_u8(want_a, wn, bn, 0, 1, 1, 0.09, 0, 0.0024, 128, 0.06, 0)
    assert len(np.unique(want_n)) > 32
    for with_next, peek, exp_tail, exp_chain in ((True, False, 1, 1), (False, False, 1, 0), (True, True, 0, 0)):
        c2 = ws.conv2d(ws.tensor(t1), ws.tensor(w2), ws.tensor(b2), 1, 1, 1, q2).prepare()
        c3 = ws.conv2d(c2.output(0), ws.tensor(w3), ws.tensor(b3), 0, 1, 1, q3).prepare()
        add = ws.add(c3.output(0), ws.tensor(r), dict(ialpha=[0.07, 0.04], izp=[121, 77], oalpha=0.09, ozp=0)).prepare()
        cn = ws.conv2d(add.output(0), ws.tensor(wn), ws.tensor(bn), 0, 1, 1, qn).prepare() if with_next else None
        for rep in range(2):
            t0, k0 = tails(), chained()
            c2.run()
            if peek:
                assert same_bits(c2.output(0).numpy(), want2)
            c3.run()
            add.run()
            if cn:
                cn.run()
                assert same_bits(cn.output(0).numpy(), want_n), (with_next, peek, rep)
            assert same_bits(add.output(0).numpy(), want_a), (with_next, peek, rep)
            assert tails() == t0 + exp_tail and chained() - k0 in (exp_chain, 1 if (peek and with_next) else exp_chain), (with_next, peek, rep)
        assert same_bits(c3.output(0).numpy(), want3) and same_bits(c2.output(0).numpy(), want2)
        for o in ([cn] if cn else []) + [add, c3, c2]:
            o.delete()
    ws.delete()


def test_convolution_and_relu_run_as_one_kernel(own_rt):
    """A convolution whose output only a relu with the same scale and zero point on both sides reads leaves its launch
    to that relu (the clamp moves into the convolution's epilogue); other relus run as operators of their own."""
    import ctypes as C
    from oracle import orc
    fused = own_rt.libs[1].hip_module_fused_relus
    fused.restype = C.c_long
    ws = own_rt.workspace("hip")
    rng = np.random.default_rng(22)
    for (Cc, K, R, pad, g) in ((32, 96, 1, 0, 1), (48, 48, 3, 1, 48), (64, 64, 3, 1, 1)):
        x = rng.integers(0, 256, (2, Cc, 10, 9), dtype=np.uint8)
        w = rng.integers(0, 256, (K, Cc // g, R, R), dtype=np.uint8)
        b = rng.integers(-5000, 5000, K).astype(np.int32)
        q = dict(ialpha=0.031, izp=77, walpha=0.0042, wzp=128, oalpha=0.09, ozp=60)
        want_c = orc.conv2d_u8(x, w, b, pad, 1, g, 0.031, 77, 0.0042, 128, 0.09, 60)
        for same in (True, False):
            conv = ws.conv2d(ws.tensor(x), ws.tensor(w), ws.tensor(b), pad, 1, g, q).prepare()
            qr = dict(ialpha=0.09, izp=60, oalpha=0.09 if same else 0.05, ozp=60 if same else 3)
            relu = ws.relu(conv.output(0), qr).prepare()
            n0 = fused()
            conv.run()
            relu.run()
            assert same_bits(relu.output(0).numpy(), orc.relu_u8(want_c, 0.09, 60, qr["oalpha"], qr["ozp"])), (Cc, K, same)
            assert fused() == n0 + (1 if same else 0)
            assert same_bits(conv.output(0).numpy(), want_c)
            relu.delete()
            conv.delete()
    ws.delete()


def test_fully_connected_layer_and_dequantize_run_as_one_kernel(own_rt):
    """A fully-connected layer whose output only a dequantize reads leaves its launch to that operator: one kernel computes
    the layer and writes the float values (op_dequantize_run_u8 on the layer's bytes, bit for bit); the layer's own bytes are
    computed when somebody asks for them.  A dequantize with another scale runs as an operator of its own."""
    import ctypes as C
    from oracle import orc
    fused = own_rt.libs[1].hip_module_fused_dequants
    fused.restype = C.c_long
    ws = own_rt.workspace("hip")
    rng = np.random.default_rng(29)
    x = rng.integers(0, 256, (6, 256), dtype=np.uint8)
    w = rng.integers(0, 256, (37, 256), dtype=np.uint8)
    b = rng.integers(-5000, 5000, 37).astype(np.int32)
    q = dict(ialpha=0.02, izp=121, walpha=0.004, wzp=128, oalpha=0.35, ozp=100)
    want_ip = orc.ip_u8(x, w, b, 0.02, 121, 0.004, 128, 0.35, 100)
    assert len(np.unique(want_ip)) > 8
    for alpha, expect in ((0.35, 1), (0.36, 0)):
        tx = ws.tensor(x)
        ip = ws.ip(tx, ws.tensor(w), ws.tensor(b), q).prepare()
        dq = ws.dequantize(ip.output(0), alpha, 100).prepare()
        want = orc.dequantize_u8(want_ip, alpha, 100)
        n0 = fused()
        for _ in range(2):
            ip.run()
            dq.run()
            assert same_bits(dq.output(0).numpy().reshape(6, 37), np.ascontiguousarray(want).reshape(6, 37)), alpha
        assert fused() == n0 + 2 * expect
        assert same_bits(ip.output(0).numpy().reshape(6, 37), want_ip)  # elided when fused: computed now
        for o in (dq, ip):
            o.delete()
    ws.delete()


def test_stem_convolution_relu_and_max_pooling_run_as_one_kernel(own_rt):
    """conv_2d (3 channels, 7x7, stride 2) -> relu -> max pooling 3x3 / 2 / 1 with equal scales: the relu passes the
    convolution's launch on to the pooling, which runs all three in the convolution's kernel (no relu in between: the
    pooling takes the launch directly).  A pooling the kernel does not implement (2x2), a relu that rescales, or a
    host that asks for an intermediate tensor get the operators one by one, with the same bytes."""
    import ctypes as C
    from oracle import orc
    from nart_amd import art
    pools = own_rt.libs[1].hip_module_fused_pools
    pools.restype = C.c_long
    ws = own_rt.workspace("hip")
    rng = np.random.default_rng(23)
    x = rng.integers(0, 256, (2, 3, 64, 48), dtype=np.uint8)
    w = rng.integers(0, 256, (64, 3, 7, 7), dtype=np.uint8)
    b = rng.integers(-5000, 5000, 64).astype(np.int32)
    q = dict(ialpha=0.031, izp=77, walpha=0.0042, wzp=128, oalpha=0.09, ozp=60)
    want_c = orc.conv2d_u8(x, w, b, 3, 2, 1, 0.031, 77, 0.0042, 128, 0.09, 60)
    want_r = orc.relu_u8(want_c, 0.09, 60, 0.09, 60)
    qs = dict(ialpha=0.09, izp=60, oalpha=0.09, ozp=60)
    for with_relu, kernel, pad, peek, expect in ((True, 3, 1, False, 1), (False, 3, 1, False, 1), (True, 2, 0, False, 0),
                                                 (True, 3, 1, True, 0)):
        conv = ws.conv2d(ws.tensor(x), ws.tensor(w), ws.tensor(b), 3, 2, 1, q).prepare()
        relu = ws.relu(conv.output(0), qs).prepare() if with_relu else None
        src = relu if with_relu else conv
        pool = ws.pool(src.output(0), kernel, pad, 2, 0, False, qs).prepare()  # method 0: max
        n0 = pools()
        conv.run()
        if relu:
            relu.run()
        if peek:  # the host reads the relu's output before the pooling runs: the deferred launch happens here
            assert same_bits(relu.output(0).numpy(), want_r)
        pool.run()
        want = orc.pool_u8(want_r if with_relu else want_c, kernel, pad, 2, 0, False, 0.09, 60, 0.09, 60)
        assert same_bits(pool.output(0).numpy(), want), (with_relu, kernel, peek)
        assert pools() == n0 + expect, (with_relu, kernel, peek)
        # the intermediate tensors are still there for whoever asks
        assert same_bits(src.output(0).numpy(), want_r if with_relu else want_c)
        pool.delete()
        if relu:
            relu.delete()
        conv.delete()
    ws.delete()


def test_stem_pooling_and_the_convolutions_that_read_it_run_as_one_kernel(own_rt):
    """conv_2d (7x7, stride 2) -> max pooling 3x3 / 2 / 1 -> two 1x1 conv_2d operators on the pooled tensor (64 -> 64 and
    64 -> 256, a residual network's first layer and its projection shortcut): the pooling's run() launches the stem's
    kernel for all four operators and the two convolutions' run() find their work done.  A third reader of the pooled
    tensor, or a reader the kernel does not take (3x3), gets the stem with its pooling and the readers one by one."""
    import ctypes as C
    from oracle import orc
    pools = own_rt.libs[1].hip_module_fused_pools
    pools.restype = C.c_long
    chained = own_rt.libs[1].hip_module_chained_convs
    chained.restype = C.c_long
    ws = own_rt.workspace("hip")
    rng = np.random.default_rng(29)
    x = rng.integers(0, 256, (2, 3, 64, 96), dtype=np.uint8)
    w = rng.integers(0, 256, (64, 3, 7, 7), dtype=np.uint8)
    b = rng.integers(-5000, 5000, 64).astype(np.int32)
    q = dict(ialpha=0.031, izp=77, walpha=0.0042, wzp=128, oalpha=0.09, ozp=0)
    qp = dict(ialpha=0.09, izp=0, oalpha=0.09, ozp=0)
    want_c = orc.conv2d_u8(x, w, b, 3, 2, 1, 0.031, 77, 0.0042, 128, 0.09, 0)
    want_p = orc.pool_u8(want_c, 3, 1, 2, 0, False, 0.09, 0, 0.09, 0)
    readers = []
    for K, k, oa, oz in ((64, 1, 0.07, 0), (256, 1, 0.11, 113), (64, 3, 0.2, 0)):
        wr = rng.integers(1, 256, (K, 64, k, k), dtype=np.uint8)
        br = rng.integers(-9000, 9000, K).astype(np.int32)
        qr = dict(ialpha=0.09, izp=0, walpha=0.004, wzp=128, oalpha=oa, ozp=oz)
        readers.append((wr, br, qr, k, orc.conv2d_u8(want_p, wr, br, k // 2, 1, 1, 0.09, 0, 0.004, 128, oa, oz)))
    assert all(len(np.unique(r[4])) > 32 for r in readers)
    for pick, expect_chain in (((0, 1), 2), ((0,), 1), ((0, 1, 2), 0), ((2,), 0)):
        conv = ws.conv2d(ws.tensor(x), ws.tensor(w), ws.tensor(b), 3, 2, 1, q).prepare()
        pool = ws.pool(conv.output(0), 3, 1, 2, 0, False, qp).prepare()
        ops = [ws.conv2d(pool.output(0), ws.tensor(readers[i][0]), ws.tensor(readers[i][1]), readers[i][3] // 2, 1, 1,
                         readers[i][2]).prepare() for i in pick]
        for rep in range(2):
            n0, c0 = pools(), chained()
            conv.run()
            pool.run()
            for o in ops:
                o.run()
            for i, o in zip(pick, ops):
                assert same_bits(o.output(0).numpy(), readers[i][4]), (pick, i, rep)
            assert same_bits(pool.output(0).numpy(), want_p), (pick, rep)
            assert pools() == n0 + 1 and chained() == c0 + expect_chain, (pick, rep, pools() - n0, chained() - c0)
        for o in ops[::-1] + [pool, conv]:
            o.delete()
    ws.delete()


def test_concat_softmax_through_the_op_api(own_rt):
    import refrun
    from oracle import orc
    ws = own_rt.workspace("hip")
    rng = np.random.default_rng(13)
    ins = [rng.integers(0, 256, (2, c, 6, 5), dtype=np.uint8) for c in (16, 5, 32)]
    ia, iz = [0.02, 0.05, 0.011], [3, 128, 250]
    assert same_bits(refrun.concat_u8(ws, ins, ia, iz, 0.03, 17), orc.concat_u8(ins, ia, iz, 0.03, 17))
    x = rng.integers(0, 256, (4, 1000), dtype=np.uint8)
    got = refrun.softmax_u8(ws, x.reshape(4, 1000, 1, 1), 1, 0.07, 140, 1.0 / 255, 0)
    assert same_bits(got.reshape(4, 1000), orc.softmax_u8(x, 1, 0.07, 140, 1.0 / 255, 0))
    ws.delete()


def test_int8_ops_through_the_op_api(own_rt):
    """quantize (symmetric) -> conv (int8) -> flatten -> ip (int8) -> dequantize on the hip workspace, every
    stage against the oracle; the operators are chosen from the tensor dtype / the qtype setting as in the reference
    (conv_2d.c:113-146, ip.cpp:297-336, quantize.c:233-262, dequantize.c:141-167)."""
    import refrun
    from oracle import orc
    ws = own_rt.workspace("hip")
    rng = np.random.default_rng(12)
    xf = (rng.standard_normal((3, 16, 10, 10)) * 2).astype(np.float32)
    w = rng.integers(-128, 128, (24, 16, 3, 3), dtype=np.int8)
    b = rng.integers(-5000, 5000, 24).astype(np.int32)
    wf = rng.integers(-128, 128, (10, 24 * 5 * 5), dtype=np.int8)
    bf = rng.integers(-5000, 5000, 10).astype(np.int32)
    qz = ws.quantize(ws.tensor(xf), 0.03, 0, bits=8, qtype=2).prepare().run()
    xq = orc.quantize_i8(xf, 0.03, 8)
    assert qz.output(0).dtype == np.int8 and same_bits(qz.output(0).numpy(), xq)
    q = dict(ialpha=0.03, izp=0, walpha=0.004, wzp=0, oalpha=0.2, ozp=0, obits=7)
    conv = ws.conv2d(qz.output(0), ws.tensor(w), ws.tensor(b), 1, 2, 1, q).prepare().run()
    yc = orc.conv2d_i8(xq, w, b, 1, 2, 1, 0.03, 0.004, 0.2, 7)
    assert conv.output(0).dtype == np.int8 and same_bits(conv.output(0).numpy(), yc)
    flat = ws.reshape_flatten(conv.output(0)).prepare().run()
    q2 = dict(ialpha=0.2, izp=0, walpha=0.002, wzp=0, oalpha=0.9, ozp=0, obits=7)
    ip = ws.ip(flat.output(0), ws.tensor(wf), ws.tensor(bf), q2).prepare().run()
    yi = orc.ip_i8(yc.reshape(3, -1), wf, bf, 0.2, 0.002, 0.9, 7)
    assert same_bits(ip.output(0).numpy().reshape(yi.shape), yi)
    dq = ws.dequantize(ip.output(0), 0.9, 0, bits=8, qtype=2).prepare().run()
    assert same_bits(dq.output(0).numpy().reshape(yi.shape), orc.dequantize_i8(yi, 0.9))
    # the same through refrun's helpers (the signatures the reference workspace is driven with)
    assert same_bits(refrun.conv2d_i8(ws, xq, w, None, (1, 0), (1, 2), 1, 0.03, 0.004, 0.2, 8),
                     orc.conv2d_i8(xq, w, None, (1, 0), (1, 2), 1, 0.03, 0.004, 0.2, 8))
    for o in (dq, ip, flat, conv, qz):
        o.delete()
    ws.delete()


def test_command_line_runner(tmp_path):
    """nart_promark loads an engine file with the `hip` workspace named in a JSON configuration, reshapes the batch
    (-b), times runs (-n, with and without copies), reads the input from a file (-i) and writes nart-out-<name>.bin
    (-s) — the reference runner's contract (tools/promark.cpp:192-522).  The saved output must be the oracle's."""
    import subprocess
    tool = os.path.join(LIB, "nart_promark")
    case = cases.resnet18(N=1, hw=64)
    (tmp_path / "engine.bin").write_bytes(engine.write_engine(case))
    (tmp_path / "cfg.json").write_text('{"workspaces": {"hip": {}}, "input_workspace": "hip"}')
    big = cases.resnet18(N=3, hw=64)  # what -b 3 turns the case into
    x = casecpu.random_input(big, 5)
    npdt = {"u8": np.uint8, "f32": np.float32}
    np.ascontiguousarray(x, npdt[big.input.dtype]).tofile(tmp_path / "in.bin")
    shown = {"u8": "UINT8", "f32": "FLOAT32"}[big.input.dtype] + " " + ", ".join(str(d) for d in big.input.shape)
    for extra in ([], ["-y"], ["-d"], ["-p", "2"]):
        r = subprocess.run([tool, "-m", "engine.bin", "-c", "cfg.json", "-n", "3", "-b", "3", "-i", "in.bin", "-s"] + extra,
                           cwd=tmp_path, stdout=subprocess.PIPE, stderr=subprocess.PIPE, text=True, timeout=300)
        assert r.returncode == 0, r.stderr[-2000:]
        assert "average cost" in r.stdout and "Process 2 : cost" in r.stdout and shown in r.stdout, r.stdout
        assert ("2 parades in flight, 3 passes: average cost per batch" in r.stdout) == (extra == ["-p", "2"]), r.stdout
        name = "nart-out-" + case.output.name.replace("/", "_") + ".bin"
        got = np.fromfile(tmp_path / name, dtype=npdt[big.output.dtype]).reshape(big.output.shape)
        want = casecpu.run_case(big, x)[big.output.name]
        assert same_bits(got, want), extra
        os.remove(tmp_path / name)


@pytest.mark.skipif(not (os.path.exists(REF_SO) and os.path.exists(HIP_FOR_REF)),
                    reason="reference runtime / module built against its headers not present")
def test_module_plugs_into_the_reference_runtime():
    """Runs in a process of its own: two art cores in one process would resolve each other's global symbols."""
    import subprocess
    import sys
    r = subprocess.run([sys.executable, "-u", os.path.join(ROOT, "tests", "refruntime_hip.py")], cwd=ROOT,
                       stdout=subprocess.PIPE, stderr=subprocess.STDOUT, timeout=170)
    out = r.stdout.decode()
    print(out, flush=True)
    assert r.returncode == 0 and "refruntime_hip ok" in out, out[-2000:]
