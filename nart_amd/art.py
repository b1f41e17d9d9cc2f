"""ctypes binding of NART's `art` case-runtime C API.

The binding mirrors the public C interface of art/include/art/{module,workspace,op,mem,tensor,
settings}.h (module.h:45-79, op.h:114-186, mem.h:48-101, tensor.h:33-111) and works with any library
that implements that ABI: the repo's own host core + `hip` case module, or the reference core + CPU
`quant` module built for the tests.  It is the Python-side runner (the counterpart of the reference's
pybind `_art` module, python/src/art/module.cpp) and contains no arithmetic of its own.
"""
import ctypes as C
import os

import numpy as np

MAX_DIM = 8

# data_type.h:24-44
dtUNKNOWN, dtINT8, dtINT16, dtINT32, dtINT64 = 0, 1, 2, 3, 4
dtUINT8, dtUINT16, dtUINT32, dtUINT64 = 5, 6, 7, 8
dtFLOAT16, dtFLOAT32, dtFLOAT64 = 9, 10, 11
dtSTR, dtPTR, dtCPTR, dtBOOL = 12, 13, 14, 15

_NP2DT = {np.dtype(np.int8): dtINT8, np.dtype(np.int16): dtINT16, np.dtype(np.int32): dtINT32,
          np.dtype(np.int64): dtINT64, np.dtype(np.uint8): dtUINT8, np.dtype(np.uint16): dtUINT16,
          np.dtype(np.uint32): dtUINT32, np.dtype(np.uint64): dtUINT64,
          np.dtype(np.float32): dtFLOAT32, np.dtype(np.float64): dtFLOAT64}
_DT2NP = {v: k for k, v in _NP2DT.items()}

# op_tp.h:20-129 (group << 32 | code)
OP_GROUP_QUANT = 0x0006
OP_ADD = 0x0011
OP_CONV_2D = 0x0100
OP_RELU = 0x0101
OP_POOL = 0x0102
OP_IP = 0x0104
OP_ELTWISE = 0x010C
OP_RESHAPE = 0x010E
OP_CONCAT, OP_SOFTMAX = 0x0106, 0x010B
SETTING_CONCAT_AXIS = SETTING_SOFTMAX_AXIS = 1
OP_QUANT_QUANTIZE = (OP_GROUP_QUANT << 32) | 0x80000000   # quant_op_tp.h:23
OP_QUANT_DEQUANTIZE = (OP_GROUP_QUANT << 32) | 0x80000001  # quant_op_tp.h:24

# op_settings.h
SETTING_CONV_2D_NUM_OUTPUT, SETTING_CONV_2D_PAD_H, SETTING_CONV_2D_PAD_W = 1, 2, 3
SETTING_CONV_2D_KERNEL_H, SETTING_CONV_2D_KERNEL_W = 4, 5
SETTING_CONV_2D_STRIDE_H, SETTING_CONV_2D_STRIDE_W, SETTING_CONV_2D_GROUP = 6, 7, 8
SETTING_CONV_2D_RELU_FLAG = 9
SETTING_POOL_METHOD, SETTING_POOL_PAD_H, SETTING_POOL_PAD_W = 1, 2, 3
SETTING_POOL_KERNEL_H, SETTING_POOL_KERNEL_W = 4, 5
SETTING_POOL_STRIDE_H, SETTING_POOL_STRIDE_W, SETTING_POOL_CEIL_MODE = 6, 7, 8
SETTING_POOL_MAX, SETTING_POOL_AVE = 0, 1
SETTING_IP_NUM_OUTPUT, SETTING_IP_RELU_FLAG, SETTING_IP_AXIS = 1, 2, 3
SETTING_ELTWISE_OPERATION, SETTING_ELTWISE_COEFF = 1, 2
SETTING_ELTWISE_OP_PROD, SETTING_ELTWISE_OP_SUM, SETTING_ELTWISE_OP_MAX = 0, 1, 2
SETTING_RESHAPE_DIMS, SETTING_RESHAPE_DIM_SIZE, SETTING_RESHAPE_AXIS, SETTING_RESHAPE_NUM_AXES = 1, 2, 3, 4

# quant_op_settings.h:24-40
_Q = OP_GROUP_QUANT << 16
SETTING_QUANT_IALPHA, SETTING_QUANT_IZERO_POINT, SETTING_QUANT_IBITS = _Q | 0x101, _Q | 0x102, _Q | 0x103
SETTING_QUANT_WALPHA, SETTING_QUANT_WZERO_POINT, SETTING_QUANT_WBITS = _Q | 0x104, _Q | 0x105, _Q | 0x106
SETTING_QUANT_OALPHA, SETTING_QUANT_OZERO_POINT, SETTING_QUANT_OBITS = _Q | 0x107, _Q | 0x108, _Q | 0x109
SETTING_QUANT_QTYPE = _Q | 0x10A


class shape_t(C.Structure):  # tensor.h:33-38
    _fields_ = [("dim", C.c_uint32 * MAX_DIM), ("dim_size", C.c_int32), ("batch_axis", C.c_int32),
                ("channel_axis", C.c_int32)]


class mem_t(C.Structure):
    pass


class mem_tp(C.Structure):  # mem.h:48-64
    _fields_ = [("name", C.c_char_p),
                ("new_func", C.CFUNCTYPE(C.POINTER(mem_t))),
                ("delete_func", C.CFUNCTYPE(None, C.POINTER(mem_t))),
                ("alloc_func", C.CFUNCTYPE(C.c_bool, C.POINTER(mem_t), C.c_size_t)),
                ("free_func", C.CFUNCTYPE(None, C.POINTER(mem_t))),
                ("data_func", C.CFUNCTYPE(C.c_void_p, C.POINTER(mem_t))),
                ("cpu_data_func", C.CFUNCTYPE(C.c_void_p, C.POINTER(mem_t))),
                ("size_func", C.CFUNCTYPE(C.c_size_t, C.POINTER(mem_t))),
                ("copy_from_cpu_func", C.c_void_p), ("copy_to_cpu_func", C.c_void_p),
                ("share_from_func", C.c_void_p)]


mem_t._fields_ = [("tp", C.POINTER(mem_tp)), ("refcount", C.c_uint32)]  # mem.h:66-69


class tensor_t(C.Structure):  # tensor.h:40-46
    _fields_ = [("name", C.c_char_p), ("mem", C.POINTER(mem_t)), ("dtype", C.c_uint32),
                ("shape", shape_t), ("with_transform", C.c_int32)]


class op_t(C.Structure):
    pass


op_t._fields_ = [("entry", C.c_void_p), ("workspace", C.c_void_p), ("input_size", C.c_size_t),  # op.h:134-143
                 ("output_size", C.c_size_t), ("input_tensors", C.POINTER(C.POINTER(tensor_t))),
                 ("output_tensors", C.POINTER(tensor_t)),
                 ("run_func", C.CFUNCTYPE(None, C.POINTER(op_t))), ("setting", C.c_void_p)]


class workspace_t(C.Structure):
    pass


class module_t(C.Structure):  # module.h:51-60
    _fields_ = [("op_group", C.c_uint32),
                ("name_func", C.CFUNCTYPE(C.c_char_p, C.POINTER(workspace_t))),
                ("memtype_func", C.CFUNCTYPE(C.POINTER(mem_tp), C.POINTER(workspace_t))),
                ("new_func", C.CFUNCTYPE(C.POINTER(workspace_t), C.c_void_p)),
                ("delete_func", C.CFUNCTYPE(None, C.POINTER(workspace_t))),
                ("op_tp_entry", C.c_void_p)]


workspace_t._fields_ = [("module_type", C.POINTER(module_t))]  # workspace.h:27-29


class Tensor:
    """A tensor_t owned either by Python (tensor_new) or by an op (output)."""

    def __init__(self, rt, ptr, owned):
        self.rt, self.ptr, self.owned = rt, ptr, owned

    @property
    def shape(self):
        s = self.ptr.contents.shape
        return tuple(int(s.dim[i]) for i in range(s.dim_size))

    @property
    def dtype(self):
        return _DT2NP[self.ptr.contents.dtype]

    def set_shape(self, shape, batch_axis=0, channel_axis=None):
        s = self.ptr.contents.shape
        s.dim_size = len(shape)
        for i in range(MAX_DIM):
            s.dim[i] = shape[i] if i < len(shape) else 1
        s.batch_axis = batch_axis
        s.channel_axis = (1 if len(shape) > 1 else -1) if channel_axis is None else channel_axis

    def alloc(self):  # tensor_alloc, tensor.h:96-100
        t = self.ptr.contents
        n = int(np.prod(self.shape)) * self.dtype.itemsize
        ok = t.mem.contents.tp.contents.alloc_func(t.mem, n)
        assert ok
        return n

    def _host(self):
        t = self.ptr.contents
        return t.mem.contents.tp.contents.cpu_data_func(t.mem)  # mem_cpu_data, mem.h:88

    def write(self, arr):
        arr = np.ascontiguousarray(arr, dtype=self.dtype)
        assert arr.shape == self.shape, (arr.shape, self.shape)
        self.alloc()
        C.memmove(self._host(), arr.ctypes.data, arr.nbytes)

    def numpy(self):
        out = np.empty(self.shape, dtype=self.dtype)
        C.memmove(out.ctypes.data, self._host(), out.nbytes)
        return out

    def device_ptr(self):
        t = self.ptr.contents
        return t.mem.contents.tp.contents.data_func(t.mem)  # mem_data, mem.h:86


class Op:
    def __init__(self, rt, ptr):
        self.rt, self.ptr = rt, ptr
        self._keep = []

    def set_single(self, item, dtype, value):
        lib = self.rt.core
        if dtype == dtFLOAT32:
            ok = lib.op_setting_single_set(self.ptr, C.c_uint32(item), C.c_uint32(dtype), C.c_double(value))
        elif dtype in (dtINT64, dtUINT64):
            ok = lib.op_setting_single_set(self.ptr, C.c_uint32(item), C.c_uint32(dtype), C.c_uint64(value))
        else:
            ok = lib.op_setting_single_set(self.ptr, C.c_uint32(item), C.c_uint32(dtype),
                                           C.c_uint32(int(value) & 0xFFFFFFFF))
        assert ok, "op_setting_single_set(%#x) refused" % item
        return self

    def set_array(self, item, dtype, values):
        arr = np.ascontiguousarray(values, dtype=_DT2NP[dtype])
        ok = self.rt.core.op_setting_array_set(self.ptr, C.c_uint32(item), C.c_uint32(dtype),
                                               C.c_size_t(arr.size), C.c_void_p(arr.ctypes.data))
        assert ok, "op_setting_array_set(%#x) refused" % item
        return self

    def set_quant(self, ialpha=None, izp=None, walpha=None, wzp=None, oalpha=None, ozp=None, bits=8, obits=None):
        """The SETTING_QUANT_* arrays every quant op reads (e.g. conv_2d.c:42-69)."""
        obits = bits if obits is None else obits
        if ialpha is not None:
            ia = np.atleast_1d(np.asarray(ialpha, dtype=np.float32))
            self.set_array(SETTING_QUANT_IALPHA, dtFLOAT32, ia)
            self.set_array(SETTING_QUANT_IZERO_POINT, dtUINT8, np.atleast_1d(izp))
            self.set_array(SETTING_QUANT_IBITS, dtUINT8, [bits] * ia.size)
        if walpha is not None:
            # one entry = a per-tensor scale; one entry per output channel = per-channel scales
            self.set_array(SETTING_QUANT_WALPHA, dtFLOAT32, np.atleast_1d(np.asarray(walpha, dtype=np.float32)))
            self.set_array(SETTING_QUANT_WZERO_POINT, dtUINT8, [wzp])
            self.set_array(SETTING_QUANT_WBITS, dtUINT8, [bits])
        if oalpha is not None:
            self.set_array(SETTING_QUANT_OALPHA, dtFLOAT32, [oalpha])
            self.set_array(SETTING_QUANT_OZERO_POINT, dtUINT8, [ozp])
            self.set_array(SETTING_QUANT_OBITS, dtUINT8, [obits])
        return self

    def config(self):
        assert self.rt.core.op_config(self.ptr), "op_config failed"
        return self

    def prepare(self):
        self.rt.core.op_prepare(self.ptr)
        return self

    def run(self):  # op_run is an inline wrapper around run_func (op.h:145-165)
        self.ptr.contents.run_func(self.ptr)
        return self

    def output(self, i=0):
        o = self.ptr.contents
        assert i < o.output_size
        return Tensor(self.rt, C.pointer(o.output_tensors[i]), owned=False)

    def delete(self):
        self.rt.core.op_delete(self.ptr)


class Workspace:
    def __init__(self, rt, module, ptr):
        self.rt, self.module, self.ptr = rt, module, ptr

    @property
    def name(self):
        return self.module.name_func(self.ptr).decode()

    @property
    def memtype(self):
        return self.module.memtype_func(self.ptr)

    def new_op(self, code, inputs):
        arr = (C.POINTER(tensor_t) * len(inputs))(*[t.ptr for t in inputs])
        p = self.rt.core.workspace_new_op(self.ptr, C.c_uint64(code), C.c_uint8(len(inputs)), arr)
        assert p, "workspace_new_op(%#x) failed" % code
        op = Op(self.rt, p)
        op._keep = list(inputs)
        return op

    def tensor(self, arr=None, dtype=None, shape=None, mem="ws"):
        return self.rt.tensor(arr, dtype, shape, self.memtype if mem == "ws" else None)

    def delete(self):
        self.module.delete_func(self.ptr)

    # ---- convenience builders for the quantized operators -------------------------------------
    def conv2d(self, x, w, b, pad, stride, group, q, relu=None):
        K, _, R, S = w.shape
        ph, pw = (pad, pad) if np.isscalar(pad) else pad
        sh, sw = (stride, stride) if np.isscalar(stride) else stride
        op = self.new_op(OP_CONV_2D, [x, w] + ([b] if b is not None else []))
        for item, v in ((SETTING_CONV_2D_NUM_OUTPUT, K), (SETTING_CONV_2D_KERNEL_H, R),
                        (SETTING_CONV_2D_KERNEL_W, S), (SETTING_CONV_2D_PAD_H, ph),
                        (SETTING_CONV_2D_PAD_W, pw), (SETTING_CONV_2D_STRIDE_H, sh),
                        (SETTING_CONV_2D_STRIDE_W, sw), (SETTING_CONV_2D_GROUP, group)):
            op.set_single(item, dtUINT32, v)
        if relu is not None:
            op.set_single(SETTING_CONV_2D_RELU_FLAG, dtBOOL, int(relu))
        op.set_quant(**q)
        return op.config()

    def ip(self, x, w, b, q):
        op = self.new_op(OP_IP, [x, w] + ([b] if b is not None else []))
        op.set_single(SETTING_IP_NUM_OUTPUT, dtUINT32, w.shape[0])
        op.set_quant(**q)
        return op.config()

    def add(self, a, b, q):
        return self.new_op(OP_ADD, [a, b]).set_quant(**q).config()

    def eltwise(self, ins, q, operation=SETTING_ELTWISE_OP_SUM, coeff=None):
        op = self.new_op(OP_ELTWISE, list(ins))
        op.set_single(SETTING_ELTWISE_OPERATION, dtUINT32, operation)
        if coeff is not None:
            op.set_array(SETTING_ELTWISE_COEFF, dtFLOAT32, coeff)
        return op.set_quant(**q).config()

    def relu(self, x, q):
        return self.new_op(OP_RELU, [x]).set_quant(**q).config()

    def pool(self, x, kernel, pad, stride, method, ceil_mode, q):
        op = self.new_op(OP_POOL, [x])
        kh, kw = (kernel, kernel) if np.isscalar(kernel) else kernel
        ph, pw = (pad, pad) if np.isscalar(pad) else pad
        sh, sw = (stride, stride) if np.isscalar(stride) else stride
        for item, v in ((SETTING_POOL_KERNEL_H, kh), (SETTING_POOL_KERNEL_W, kw),
                        (SETTING_POOL_PAD_H, ph), (SETTING_POOL_PAD_W, pw),
                        (SETTING_POOL_STRIDE_H, sh), (SETTING_POOL_STRIDE_W, sw),
                        (SETTING_POOL_METHOD, method)):
            op.set_single(item, dtUINT32, v)
        op.set_single(SETTING_POOL_CEIL_MODE, dtBOOL, int(ceil_mode))
        return op.set_quant(**q).config()

    def quantize(self, x, oalpha, ozp, bits=8, qtype=None):
        op = self.new_op(OP_QUANT_QUANTIZE, [x])
        if qtype is not None:  # SETTING_QUANT_DEFAULT / _BIASED / _SYMMETRIC (quant_op_settings.h:38-41)
            op.set_single(SETTING_QUANT_QTYPE, dtINT32, qtype)
        return op.set_quant(oalpha=oalpha, ozp=ozp, bits=bits).config()

    def dequantize(self, x, ialpha, izp, bits=8, qtype=None):
        op = self.new_op(OP_QUANT_DEQUANTIZE, [x])
        if qtype is not None:
            op.set_single(SETTING_QUANT_QTYPE, dtINT32, qtype)
        return op.set_quant(ialpha=ialpha, izp=izp, bits=bits).config()

    def concat(self, ins, q, axis=1):
        op = self.new_op(OP_CONCAT, list(ins))
        op.set_single(SETTING_CONCAT_AXIS, dtUINT32, axis)
        return op.set_quant(**q).config()

    def softmax(self, x, q, axis=1):
        op = self.new_op(OP_SOFTMAX, [x])
        op.set_single(SETTING_SOFTMAX_AXIS, dtUINT32, axis)
        return op.set_quant(**q).config()

    def reshape_flatten(self, x, axis=1):
        """Caffe-style flatten expressed as `reshape` (dims [0,-1] from `axis` on)."""
        op = self.new_op(OP_RESHAPE, [x])
        op.set_array(SETTING_RESHAPE_DIMS, dtINT32, [-1])
        op.set_single(SETTING_RESHAPE_AXIS, dtINT32, axis)
        return op.config()


class Runtime:
    """Loads a core library (libart) and any number of case-module libraries, RTLD_GLOBAL like the
    reference runners do (tools/promark.cpp:151-167)."""

    def __init__(self, core_path, module_paths=()):
        mode = C.RTLD_GLOBAL
        self.core = C.CDLL(os.path.abspath(core_path), mode=mode)
        self.libs = [self.core] + [C.CDLL(os.path.abspath(p), mode=mode) for p in module_paths]
        c = self.core
        c.tensor_new.restype = C.POINTER(tensor_t)
        c.tensor_new.argtypes = [C.POINTER(mem_tp), C.c_uint32]
        c.tensor_free.argtypes = [C.POINTER(tensor_t)]
        c.tensor_delete.argtypes = [C.POINTER(tensor_t)]
        c.workspace_new_op.restype = C.POINTER(op_t)
        c.workspace_new_op.argtypes = [C.POINTER(workspace_t), C.c_uint64, C.c_uint8,
                                       C.POINTER(C.POINTER(tensor_t))]
        c.op_config.restype = C.c_bool
        c.op_config.argtypes = [C.POINTER(op_t)]
        c.op_prepare.argtypes = [C.POINTER(op_t)]
        c.op_delete.argtypes = [C.POINTER(op_t)]
        c.op_setting_single_set.restype = C.c_bool
        c.op_setting_array_set.restype = C.c_bool
        c.op_setting_array_set.argtypes = [C.POINTER(op_t), C.c_uint32, C.c_uint32, C.c_size_t, C.c_void_p]
        self.cpu_mem_tp = C.POINTER(mem_tp).in_dll(c, "cpu_mem_tp")

    def module(self, name):
        for lib in self.libs:
            try:
                return module_t.in_dll(lib, name + "_module_tp")
            except ValueError:
                continue
        raise KeyError(name + "_module_tp")

    def workspace(self, name):
        m = self.module(name)
        ws = m.new_func(None)  # both reference runners pass NULL settings
        assert ws, "workspace_new failed"
        return Workspace(self, m, ws)

    def tensor(self, arr=None, dtype=None, shape=None, memtype=None):
        if arr is not None:
            arr = np.ascontiguousarray(arr)
            dtype, shape = arr.dtype, arr.shape
        p = self.core.tensor_new(memtype if memtype is not None else self.cpu_mem_tp,
                                 _NP2DT[np.dtype(dtype)])
        t = Tensor(self, p, owned=True)
        t.set_shape(shape)
        if arr is not None:
            t.write(arr)
        return t
