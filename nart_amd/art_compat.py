"""Drop-in for the reference's Python runtime package `nart.art` (python/nart/art/__init__.py:31-73 and its
pybind extension `_art`, python/src/art/module.cpp:98-122, 193-275, 280-527) on top of this repo's libraries.

A script written against the reference -

    from nart import art
    ctx = art.create_context_from_json("engine.bin.json")
    parade = art.load_parade("engine.bin", ctx)
    inputs, outputs = art.get_empty_io(parade)
    inputs["data"][:] = my_data
    parade.run(inputs, outputs)

- runs unchanged with `from nart_amd import art_compat as art`.  Same names, same argument meaning, same return
values, same errors: `RuntimeContext(modules, input_module)` loads `lib art_module_<name>.so` from the package directory
and skips (with a message) the modules it cannot load; `Parade(data, ctx)` deserialises, applies the shapes and
prepares; `run(inputs, outputs)` checks every array's rank, shape and dtype (ValueError with the reference's
messages), copies in through `mem_cpu_data`, runs, copies out.

No arithmetic happens here: every call goes through the art C API (include/art/art.h) into libart.so and the case
modules.
"""
import ctypes as C
import json
import os
import sys

import numpy

from . import art as _abi
from . import engine as _engine

_PACKAGE_DIR = os.path.join(os.path.dirname(os.path.abspath(__file__)), "lib")
_RUNTIME = None

# DTYPE_NAME of module.cpp:262-278
_DTYPE_NAME = {_abi.dtINT8: "int8", _abi.dtINT16: "int16", _abi.dtINT32: "int32", _abi.dtINT64: "int64",
               _abi.dtUINT8: "uint8", _abi.dtUINT16: "uint16", _abi.dtUINT32: "uint32", _abi.dtUINT64: "uint64",
               _abi.dtFLOAT16: "float16", _abi.dtFLOAT32: "float32", _abi.dtFLOAT64: "float64", _abi.dtBOOL: "bool"}


def set_package_dir(path):
    """Directory that holds libart.so and the libart_module_<name>.so files (module.cpp:526)."""
    global _PACKAGE_DIR, _RUNTIME
    _PACKAGE_DIR = str(path)
    _RUNTIME = None


def _runtime():
    global _RUNTIME
    if _RUNTIME is None:
        _RUNTIME = _abi.Runtime(os.path.join(_PACKAGE_DIR, "libart.so"))
    return _RUNTIME


class RuntimeContext:
    """The workspaces a parade needs (module.cpp:75-128): one per module that loads, in the order given; the input
    tensors live in `input_module`'s memory type (the first workspace's if that module is not among them)."""

    _load_failed = set()  # names that failed once are not tried again (module.cpp:93-96)

    def __init__(self, modules, input_module):
        rt = _runtime()
        self._rt = rt
        self._modules, self._workspaces = [], []
        self._input_ws = None
        for name in list(modules):
            if name in RuntimeContext._load_failed:
                continue
            mod = self._find_module(rt, name)
            if mod is None:
                print("fail to load module %s" % name, file=sys.stderr)
                RuntimeContext._load_failed.add(name)
                continue
            ws = mod.new_func(None)
            if not ws:
                print("fail to load module %s" % name, file=sys.stderr)
                RuntimeContext._load_failed.add(name)
                continue
            w = _abi.Workspace(rt, mod, ws)
            self._modules.append(name)
            self._workspaces.append(w)
            if name == input_module:
                self._input_ws = w
        if not self._workspaces:
            raise RuntimeError("RuntimeContext: none of the modules %r could be loaded from %s" % (list(modules), _PACKAGE_DIR))
        if self._input_ws is None:
            self._input_ws = self._workspaces[0]

    @staticmethod
    def _find_module(rt, name):
        try:
            return rt.module(name)  # already loaded (or built into libart, like `default` in the reference)
        except KeyError:
            pass
        path = os.path.join(_PACKAGE_DIR, "libart_module_%s.so" % name)  # module_path(), module.cpp:64-68
        if not os.path.exists(path):
            return None
        try:
            rt.libs.append(C.CDLL(path, mode=C.RTLD_GLOBAL))
            return rt.module(name)
        except (OSError, KeyError) as e:
            print(e, file=sys.stderr)
            return None

    @property
    def loaded_workspaces(self):
        return list(self._modules)

    def __del__(self):
        for w in getattr(self, "_workspaces", []):
            try:
                w.delete()
            except Exception:
                pass
        self._workspaces = []


class Parade:
    """`_art.Parade` (module.cpp:193-275, 284-500)."""

    def __init__(self, data, ctx):
        if not isinstance(data, (bytes, bytearray, memoryview)):
            raise TypeError("Parade(data, ctx): data must be the bytes of an engine file")
        self._ctx = ctx  # keeps the workspaces alive
        core = ctx._rt.core
        self._core = core
        self._p = _engine.Parade(ctx._rt, bytes(data), ctx._workspaces, input_workspace=ctx._input_ws, prepare=False)
        if not core.parade_apply_reshape(self._p.ptr):
            raise RuntimeError("parade_apply_reshape failed")
        core.parade_prepare(self._p.ptr)
        self._collect()

    def _collect(self):
        self._inputs = {t.ptr.contents.name.decode(): t for t in self._p.inputs()}
        self._outputs = {t.ptr.contents.name.decode(): t for t in self._p.outputs()}
        self._by_name = dict(self._inputs)
        self._by_name.update(self._outputs)

    # ---- shapes and dtypes ------------------------------------------------------------------------------
    def input_shapes(self):
        return {k: list(t.shape) for k, t in self._inputs.items()}

    def output_shapes(self):
        return {k: list(t.shape) for k, t in self._outputs.items()}

    def input_dtypes(self):
        return {k: _DTYPE_NAME[t.ptr.contents.dtype] for k, t in self._inputs.items()}

    def output_dtypes(self):
        return {k: _DTYPE_NAME[t.ptr.contents.dtype] for k, t in self._outputs.items()}

    def get_tensor_shape(self, name):
        t = self._by_name.get(name)
        return None if t is None else list(t.shape)

    def get_tensor_dtype(self, name):
        t = self._by_name.get(name)
        return None if t is None else _DTYPE_NAME[t.ptr.contents.dtype]

    def get_input_names(self):
        return list(self._inputs)

    def get_output_names(self):
        return list(self._outputs)

    def get_raw_tensor_data(self, name):
        """mem_data() of the tensor as an integer (a device address for device workspaces), 0 for an unknown name."""
        t = self._by_name.get(name)
        return 0 if t is None else int(t.device_ptr() or 0)

    # ---- execution ----------------------------------------------------------------------------------------
    def forward(self):
        self._core.parade_run(self._p.ptr)

    def reshape(self, shapes):
        """{input name: new shape}; False if a rank differs or the runtime refuses (module.cpp:224-243, 381-400)."""
        for name, t in self._inputs.items():
            if name not in shapes:
                continue
            shape = [int(v) for v in shapes[name]]
            s = t.ptr.contents.shape
            if len(shape) != s.dim_size:
                return False
            for i, v in enumerate(shape):
                s.dim[i] = v
        if not self._core.parade_apply_reshape(self._p.ptr):
            return False
        self._core.parade_prepare(self._p.ptr)
        return True

    @staticmethod
    def _check(kind, t, arr):
        s = t.ptr.contents.shape
        if s.dim_size != arr.ndim:
            raise ValueError("%s dim size not match" % kind)
        if tuple(int(s.dim[i]) for i in range(s.dim_size)) != tuple(arr.shape):
            raise ValueError("%s shape not match" % kind)
        if _DTYPE_NAME[t.ptr.contents.dtype] != str(arr.dtype):
            raise ValueError("%s dtype not match" % kind)

    def run(self, inputs, outputs):
        for name, t in self._inputs.items():
            assert name in inputs, "some input not given when calling parade.run"
            self._check("input", t, numpy.asarray(inputs[name]))
        for name, t in self._outputs.items():
            assert name in outputs, "some output not given when calling parade.run"
            self._check("output", t, outputs[name])
        for name, t in self._inputs.items():
            a = numpy.ascontiguousarray(inputs[name])
            C.memmove(t._host(), a.ctypes.data, a.nbytes)
        self.forward()
        for name, t in self._outputs.items():
            out = outputs[name]
            if out.flags["C_CONTIGUOUS"]:
                C.memmove(out.ctypes.data, t._host(), out.nbytes)
            else:
                out[...] = t.numpy()
        return True

    def __del__(self):
        p = getattr(self, "_p", None)
        if p is not None:
            try:
                p.delete()
            except Exception:
                pass


# ---- python/nart/art/__init__.py:31-73 ---------------------------------------------------------------------------
def create_context_from_json(jsonPath):
    with open(jsonPath, "r") as fp:
        ws_data = json.loads(fp.read())
    return RuntimeContext(list(ws_data["workspaces"].keys()), ws_data["input_workspace"])


def create_context_for_target(target):
    """The reference maps a target name to its module list; the target this package adds is `hip`."""
    modules = {"hip": ["hip"]}
    if target not in modules:
        raise KeyError("unknown target %r (this package provides: %s)" % (target, ", ".join(modules)))
    return RuntimeContext(modules[target], target)


def load_parade(engine_fp, ctx):
    with open(engine_fp, "rb") as fp:
        return Parade(fp.read(), ctx)


def get_empty_io(parade):
    inputs = {k: numpy.zeros(v, dtype=numpy.dtype(parade.get_tensor_dtype(k))) for k, v in parade.input_shapes().items()}
    outputs = {k: numpy.zeros(v, dtype=numpy.dtype(parade.get_tensor_dtype(k))) for k, v in parade.output_shapes().items()}
    return inputs, outputs
