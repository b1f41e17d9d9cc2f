"""The engine.bin writer and the drop-in boundary, as far as they can be checked without a GPU:
  * a file written by nart_amd.engine loads in the REFERENCE runtime (its own deserializer + CPU quant module)
    and produces the oracle's outputs -> the writer speaks the reference's format;
  * the repo's host core reads the same file identically (same shapes, same op count) with the reference quant
    module plugged into it -> the core's ABI and reader match the reference's;
  * the `hip` module's table, op configuration and shape inference work against both cores;
  * struct layouts of include/art/art.h equal the reference headers' (sizeof / offsetof probe).
"""
import ctypes as C
import os
import subprocess

import numpy as np
import pytest

from nart_amd import art, cases, engine
from oracle import casecpu

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
LIB = os.path.join(ROOT, "nart_amd", "lib")
REF_SO = os.path.join(ROOT, "oracle", "_ref", "libnart_ref.so")
REF_TREE = "/root/reference"

needs_ref = pytest.mark.skipif(not os.path.exists(REF_SO), reason="oracle/_ref not built")


def small_cases():
    return [cases.resnet18(N=1, hw=96), cases.mobilenet_v2(N=1, hw=96), cases.resnet50(N=1, hw=224),
            cases.single_conv(N=1), cases.single_fc(M=3, K=256, Nout=64)]


@needs_ref
def test_engine_file_runs_on_reference_runtime():
    rt = art.Runtime(REF_SO)
    for case in small_cases():
        ws = rt.workspace("quant")
        p = engine.Parade(rt, engine.write_engine(case), [ws])
        casecpu.zero_reference_conv_scratch(p)
        x = casecpu.random_input(case, 7)
        got = p.forward(x).reshape(case.output.shape)
        want = casecpu.run_case(case, x)[case.output.name]
        assert np.array_equal(got.view(np.uint8), want.view(np.uint8)), case.name
        p.delete()


@needs_ref
def test_version2_engine_file_on_reference_runtime():
    """The writer's version-2 files (serialize_v2.c:25-98): with and without the pre-processing block on the input."""
    rt = art.Runtime(REF_SO)
    case = cases.resnet18(N=1, hw=96)
    x = casecpu.random_input(case, 3)
    want = casecpu.run_case(case, x)[case.output.name]
    tf = (0x11, 2, (1.5, 2.5, 3.5), (0.25, 0.5, 0.75), (7.0, 8.0, 9.0))
    for transform in (None, tf):
        ws = rt.workspace("quant")
        p = engine.Parade(rt, engine.write_engine(case, version=2, transform=transform), [ws])
        casecpu.zero_reference_conv_scratch(p)
        got = p.forward(x).reshape(case.output.shape)
        assert np.array_equal(got.view(np.uint8), want.view(np.uint8))
        if transform:
            assert p.transform_param() == (0x11, (1.5, 2.5, 3.5), (0.25, 0.5, 0.75), (7.0, 8.0, 9.0))
        p.delete()


def _probe_source():
    return r'''
#include <stdio.h>
#include <stddef.h>
#ifdef USE_REF
#include "art/module.h"
#include "art/op.h"
#include "art/op_tp.h"
#include "art/op_settings.h"
#include "art/parade.h"
#include "art/serialize.h"
#include "art/transform.h"
#else
#include "art/art.h"
#endif
#define S(t) printf("sizeof " #t " %zu\n", sizeof(t))
#define O(t, f) printf("offsetof " #t "." #f " %zu\n", offsetof(t, f))
int main(void) {
    S(shape_t); O(shape_t, dim_size); O(shape_t, batch_axis); O(shape_t, channel_axis);
    S(tensor_t); O(tensor_t, mem); O(tensor_t, dtype); O(tensor_t, shape); O(tensor_t, with_transform);
    S(mem_tp); O(mem_tp, new_func); O(mem_tp, alloc_func); O(mem_tp, data_func); O(mem_tp, cpu_data_func);
    O(mem_tp, size_func); O(mem_tp, share_from_func); S(mem_t); O(mem_t, refcount);
    S(uvalue_t); S(setting_constraint_t); O(setting_constraint_t, dtype); O(setting_constraint_t, ctp);
    O(setting_constraint_t, constraint); O(setting_constraint_t, name);
    S(setting_entry_t); O(setting_entry_t, tp); O(setting_entry_t, v); S(struct _setting_t); O(struct _setting_t, entries);
    S(op_tp_t); O(op_tp_t, name); O(op_tp_t, min_input_size); O(op_tp_t, infer_output_func); O(op_tp_t, constraints);
    S(op_tp_entry_t); O(op_tp_entry_t, alloc_func); O(op_tp_entry_t, prepare_func);
    S(op_t); O(op_t, workspace); O(op_t, input_size); O(op_t, input_tensors); O(op_t, output_tensors); O(op_t, run_func);
    O(op_t, setting); S(workspace_t); S(module_t); O(module_t, name_func); O(module_t, new_func); O(module_t, op_tp_entry);
    S(deserialize_param_t); O(deserialize_param_t, input_mem_tp);
    S(pixel_t); S(transform_param_t); O(transform_param_t, operators); O(transform_param_t, mats); O(transform_param_t, means);
    O(transform_param_t, paddings); S(transform_tensor_t); O(transform_tensor_t, capacity); O(transform_tensor_t, param);
    printf("codes %llx %llx %llx %llx %llx %llx %llx %llx %llx\n", (unsigned long long)OP_CONV_2D, (unsigned long long)OP_IP,
           (unsigned long long)OP_POOL, (unsigned long long)OP_RELU, (unsigned long long)OP_ADD, (unsigned long long)OP_ELTWISE,
           (unsigned long long)OP_RESHAPE, 0ull, 0ull);
    printf("dt %d %d %d %d %d\n", dtUINT8, dtINT32, dtFLOAT32, dtBOOL, dtSTR);
    printf("set %d %d %d %d %d %d\n", SETTING_CONV_2D_GROUP, SETTING_POOL_CEIL_MODE, SETTING_IP_AXIS, SETTING_ELTWISE_COEFF,
           SETTING_RESHAPE_AXIS, ENUM_SETTING_CONSTRAINT_REPEATED);
    return 0;
}
'''


@pytest.mark.skipif(not os.path.isdir(REF_TREE), reason="reference headers not mounted")
def test_header_layouts_equal_reference(tmp_path):
    src = tmp_path / "probe.c"
    src.write_text(_probe_source())
    outs = []
    for flags in (["-I" + os.path.join(ROOT, "include")],
                  ["-DUSE_REF", "-DART_CONSTRAINT_WITH_NAME", "-DNART_LOG_LEVEL=1", "-I" + os.path.join(REF_TREE, "art", "include")]):
        exe = tmp_path / ("probe%d" % len(outs))
        subprocess.check_call(["gcc", "-std=gnu11", "-w"] + flags + [str(src), "-o", str(exe)])
        outs.append(subprocess.check_output([str(exe)]).decode())
    assert outs[0] == outs[1], "\n".join(a + " | " + b for a, b in zip(outs[0].splitlines(), outs[1].splitlines()) if a != b)
    gold = os.path.join(ROOT, "tests", "golden", "art_abi_layout.txt")
    assert open(gold).read() == outs[1], "regenerate tests/golden/art_abi_layout.txt from the reference headers"


def test_header_layouts_equal_committed_table(tmp_path):
    """Where the reference is absent: the same probe against the committed table taken from its headers."""
    src = tmp_path / "probe.c"
    src.write_text(_probe_source())
    exe = tmp_path / "probe"
    subprocess.check_call(["gcc", "-std=gnu11", "-w", "-I" + os.path.join(ROOT, "include"), str(src), "-o", str(exe)])
    assert subprocess.check_output([str(exe)]).decode() == open(os.path.join(ROOT, "tests", "golden", "art_abi_layout.txt")).read()


def _fake_workspace(rt, lib):
    """A workspace_t that points at hip_module_tp without touching a device: enough for alloc/config/infer."""
    mod = art.module_t.in_dll(lib, "hip_module_tp")
    ws = art.workspace_t(C.pointer(mod))
    return art.Workspace(rt, mod, C.pointer(ws)), ws


def _check_hip_table(rt, lib):
    ws, keep = _fake_workspace(rt, lib)
    core = rt.core
    core.workspace_support_op.restype = C.c_bool
    core.workspace_support_op.argtypes = [C.POINTER(art.workspace_t), C.c_uint64, C.c_bool]
    g = art.OP_GROUP_QUANT << 32
    for code in (art.OP_CONV_2D, art.OP_IP, art.OP_POOL, art.OP_RELU, art.OP_ADD, art.OP_ELTWISE, art.OP_RESHAPE,
                 art.OP_CONCAT, art.OP_SOFTMAX):
        assert core.workspace_support_op(ws.ptr, g | code, True), hex(code)      # strict: group 6
        assert not core.workspace_support_op(ws.ptr, (2 << 32) | code, True)      # another module's group
        assert core.workspace_support_op(ws.ptr, (2 << 32) | code, False)         # by op code alone
    assert core.workspace_support_op(ws.ptr, art.OP_QUANT_QUANTIZE, False)
    assert core.workspace_support_op(ws.ptr, art.OP_QUANT_DEQUANTIZE, True)
    assert not core.workspace_support_op(ws.ptr, g | 0x010D, False)               # scale (op_tp.h:61): not in the table
    # configure a conv and a pool through the public API and read back the inferred shapes
    x = rt.tensor(dtype=np.uint8, shape=(2, 64, 56, 56))
    w = rt.tensor(np.zeros((128, 64, 3, 3), np.uint8))
    b = rt.tensor(np.zeros(128, np.int32))
    q = dict(ialpha=0.02, izp=128, walpha=0.005, wzp=128, oalpha=0.05, ozp=0)
    op = ws.conv2d(x, w, b, 1, 2, 1, q)
    assert op.output(0).shape == (2, 128, 28, 28) and op.output(0).dtype == np.uint8
    pool = ws.pool(op.output(0), 3, 1, 2, 0, False, dict(ialpha=0.05, izp=0, oalpha=0.05, ozp=0))
    assert pool.output(0).shape == (2, 128, 14, 14)
    pool_ceil = ws.pool(op.output(0), 3, 1, 2, 0, True, dict(ialpha=0.05, izp=0, oalpha=0.05, ozp=0))
    assert pool_ceil.output(0).shape == (2, 128, 15, 15)
    gap = ws.pool(pool.output(0), 14, 0, 1, 1, True, dict(ialpha=0.05, izp=0, oalpha=0.05, ozp=0))
    fcw = rt.tensor(np.zeros((10, 128), np.uint8))
    ip = ws.ip(gap.output(0), fcw, None, q)
    assert ip.output(0).shape == (2, 10)
    dq = ws.dequantize(ip.output(0), 0.05, 3)
    assert dq.output(0).shape == (2, 10) and dq.output(0).dtype == np.float32
    xf = rt.tensor(dtype=np.float32, shape=(2, 3, 8, 8))
    qz = ws.quantize(xf, 0.02, 128)
    assert qz.output(0).shape == (2, 3, 8, 8) and qz.output(0).dtype == np.uint8
    add = ws.add(op.output(0), op.output(0), dict(ialpha=[0.05, 0.05], izp=[0, 0], oalpha=0.07, ozp=0))
    assert add.output(0).shape == (2, 128, 28, 28)
    for o in (add, qz, dq, ip, gap, pool_ceil, pool, op):
        o.delete()
    return keep


def test_hip_module_table_and_config_on_own_core():
    rt = art.Runtime(os.path.join(LIB, "libart.so"), [os.path.join(LIB, "libart_module_hip.so")])
    _check_hip_table(rt, rt.libs[1])


@needs_ref
@pytest.mark.skipif(not os.path.isdir(REF_TREE), reason="reference headers not mounted")
def test_hip_module_built_against_nart_headers_plugs_into_reference_runtime():
    """The drop-in claim, CPU part: compile the module against the reference's OWN headers, load it into the
    reference's OWN libart and drive op lookup, settings and shape inference through it."""
    from nart_amd import build
    so = build.build_module(force=True, nart_tree=REF_TREE, out_name="libart_module_hip_narttree.so")[0]
    rt = art.Runtime(REF_SO, [so])
    _check_hip_table(rt, rt.libs[1])


def test_workspace_creation_fails_loudly_without_gpu():
    try:
        import torch
        if torch.cuda.is_available():
            pytest.skip("a GPU is present")
    except ImportError:
        pass
    rt = art.Runtime(os.path.join(LIB, "libart.so"), [os.path.join(LIB, "libart_module_hip.so")])
    with pytest.raises(AssertionError, match="workspace_new failed"):
        rt.workspace("hip")


_MALFORMED_LOADER = r"""
import ctypes as C, os, struct, sys
sys.path.insert(0, sys.argv[1])
from nart_amd import art, cases, engine
rt = art.Runtime(os.path.join(sys.argv[1], "nart_amd", "lib", "libart.so"))
data = bytearray(engine.write_engine(cases.single_fc(M=2, K=64, Nout=16)))
off = 4 + 4 + struct.unpack_from("<i", data, 4)[0]   # version, name -> tensor_count
n_tensors, n_in = struct.unpack_from("<ii", data, off)
how = sys.argv[2]
if how == "inputs_outrun_table":
    struct.pack_into("<i", data, off, 0)             # a table of no tensors, one input declared
elif how == "negative_inputs":
    struct.pack_into("<i", data, off + 4, -3)
elif how == "truncated":
    del data[len(data) // 2:]
pos = [0]
READ = C.CFUNCTYPE(C.c_size_t, C.c_size_t, C.c_void_p, C.c_void_p)
def read(sz, dst, _):
    chunk = bytes(data[pos[0]:pos[0] + sz]); C.memmove(dst, chunk, len(chunk)); pos[0] += len(chunk); return len(chunk)
cb = READ(read)
class Param(C.Structure):
    _fields_ = [("workspaces", C.POINTER(C.POINTER(art.workspace_t))), ("input_mem_tp", C.POINTER(art.mem_tp))]
core = rt.core
core.nart_buffer_new.restype = C.c_void_p; core.nart_buffer_new.argtypes = [C.c_size_t]
core.buffer_set_buffer_read_func.argtypes = [C.c_void_p, READ, C.c_void_p]
core.deserialize_parade.restype = C.c_void_p; core.deserialize_parade.argtypes = [C.c_void_p, C.POINTER(Param)]
buf = core.nart_buffer_new(1 << 16)
core.buffer_set_buffer_read_func(buf, cb, None)
ws = (C.POINTER(art.workspace_t) * 1)(None)
print("loading", how, flush=True)
core.deserialize_parade(buf, C.byref(Param(ws, rt.cpu_mem_tp)))
print("returned", flush=True)
"""


@pytest.mark.parametrize("how", ["inputs_outrun_table", "negative_inputs", "truncated"])
def test_malformed_engine_file_aborts_instead_of_overrunning(how, tmp_path):
    """Counts in an engine file are checked against the tensor table before anything is written through them; a file
    that lies about them ends in the runtime's CHECK failure (abort, the reference's error behaviour:
    art/include/art/log.h CHECK), never in a write past the table."""
    import signal
    import sys
    script = tmp_path / "load.py"
    script.write_text(_MALFORMED_LOADER)
    r = subprocess.run([sys.executable, str(script), ROOT, how], stdout=subprocess.PIPE, stderr=subprocess.PIPE, timeout=120)
    assert b"loading" in r.stdout and b"returned" not in r.stdout
    assert r.returncode == -signal.SIGABRT, (r.returncode, r.stderr[-500:])


def test_art_compat_surface_without_a_gpu():
    """nart_amd.art_compat offers the names of the reference's `nart.art` package (python/nart/art/__init__.py:31-73);
    without a GPU the `hip` module cannot make a workspace, which is reported like any module that fails to load."""
    from nart_amd import art_compat
    for name in ("RuntimeContext", "Parade", "create_context_from_json", "create_context_for_target", "load_parade",
                 "get_empty_io", "set_package_dir"):
        assert hasattr(art_compat, name), name
    for name in ("run", "forward", "reshape", "input_shapes", "output_shapes", "input_dtypes", "output_dtypes",
                 "get_tensor_shape", "get_tensor_dtype", "get_input_names", "get_output_names", "get_raw_tensor_data"):
        assert callable(getattr(art_compat.Parade, name)), name
    try:
        import torch
        if torch.cuda.is_available():
            return
    except ImportError:
        pass
    with pytest.raises(RuntimeError, match="none of the modules"):
        art_compat.RuntimeContext(["no_such_module"], "no_such_module")
