"""engine.bin (version 1) writer for synthetic cases, and a loader that hands the file to an art runtime.

The byte layout is the one NART's converter writes and its runtime reads (writer: src/serialize.cpp:67-176,
reader: art/src/serialize_v1.c:203-340, shape field order art/src/serialize.c:230-240):

    int32 version (1) | string name
    int32 tensor_count                      (inputs + weights + every op output)
    int32 n_inputs  { uint32 dtype | string name | shape }
    int32 n_weights { uint32 dtype | string name | shape | raw little-endian data }
    int32 n_ops     { int32 n_in | int32 n_out | uint64 op code | int32 input tensor index [n_in]
                      int32 n_settings { int32 repeated | int32 item | int32 dtype | value  or  int32 count + values } }
    int32 n_outputs { int32 tensor index | string name }
    int32 n_shares  { int32 from | int32 to }
    string = int32 length + bytes;   shape = int32 dim_size | uint32 dim[dim_size] | int32 channel_axis | int32 batch_axis

Every op is stamped with the quant group (6), exactly as the quant converter does (python/nart/modules/
quant.py:216), so the file loads unchanged with {"workspaces": ["quant"]} on the reference runtime and with
{"workspaces": ["hip"]} on this one.
"""
import ctypes as C
import struct

import numpy as np

from . import art

GROUP = art.OP_GROUP_QUANT << 32


def _i32(v):
    return struct.pack("<i", int(v))


def _str(s):
    b = (s or "").encode()
    return _i32(len(b)) + b


def _shape(dims, channel_axis=None, batch_axis=0):
    dims = list(dims)
    if channel_axis is None:
        channel_axis = 1 if len(dims) > 1 else -1
    return _i32(len(dims)) + b"".join(struct.pack("<I", d) for d in dims) + _i32(channel_axis) + _i32(batch_axis)


def _single(item, dtype, value):
    fmt = {art.dtUINT32: "<I", art.dtINT32: "<i", art.dtBOOL: "<?", art.dtFLOAT32: "<f", art.dtUINT8: "<B"}[dtype]
    return _i32(0) + _i32(item) + _i32(dtype) + struct.pack(fmt, value)


def _array(item, dtype, values):
    arr = np.ascontiguousarray(values, dtype=art._DT2NP[dtype])
    return _i32(1) + _i32(item) + _i32(dtype) + _i32(arr.size) + arr.tobytes()


def _quant(ialpha=None, izp=None, walpha=None, wzp=None, oalpha=None, ozp=None, bits=8):
    out = []
    if ialpha is not None:
        ia = np.atleast_1d(np.asarray(ialpha, np.float32))
        out += [_array(art.SETTING_QUANT_IALPHA, art.dtFLOAT32, ia),
                _array(art.SETTING_QUANT_IZERO_POINT, art.dtUINT8, np.atleast_1d(izp)),
                _array(art.SETTING_QUANT_IBITS, art.dtUINT8, [bits] * ia.size)]
    if walpha is not None:
        out += [_array(art.SETTING_QUANT_WALPHA, art.dtFLOAT32, [walpha]), _array(art.SETTING_QUANT_WZERO_POINT, art.dtUINT8, [wzp]),
                _array(art.SETTING_QUANT_WBITS, art.dtUINT8, [bits])]
    if oalpha is not None:
        out += [_array(art.SETTING_QUANT_OALPHA, art.dtFLOAT32, [oalpha]), _array(art.SETTING_QUANT_OZERO_POINT, art.dtUINT8, [ozp]),
                _array(art.SETTING_QUANT_OBITS, art.dtUINT8, [bits])]
    return out


def write_engine(case, version=1, transform=None):
    """Serialise a Case (nart_amd/cases.py).  A conv with relu=True becomes conv_2d followed by a relu op with
    equal scales and zero point — the reference CPU module has no fused ReLU.
    version=2 writes the format of serialize_v2.c:25-98: each input is followed by a flag and, with
    transform = (operators, frame_type, mean_rgb, std_rgb, padding_rgb), by that pre-processing block."""
    T = case.tensors
    index = {case.input.name: 0}
    inputs = [case.input]
    weights, ops = [], []
    # weights first: they follow the inputs in the tensor index space
    for node in case.nodes:
        if node.kind in ("conv", "ip"):
            for key in ("w", "b"):
                index[node.attrs[key]] = len(inputs) + len(weights)
                weights.append((node.attrs[key], case.weights[node.attrs[key]]))
    nxt = len(inputs) + len(weights)
    for node in case.nodes:
        y, xs, a = T[node.output], [T[i] for i in node.inputs], node.attrs
        ins = [index[i] for i in node.inputs]
        if node.kind == "quantize":
            ops.append((art.OP_QUANT_QUANTIZE, ins, _quant(oalpha=y.alpha, ozp=y.zp)))
        elif node.kind == "dequantize":
            ops.append((art.OP_QUANT_DEQUANTIZE, ins, _quant(ialpha=xs[0].alpha, izp=xs[0].zp)))
        elif node.kind == "conv":
            k = a["k"]
            s = [_single(art.SETTING_CONV_2D_NUM_OUTPUT, art.dtUINT32, a["K"]), _single(art.SETTING_CONV_2D_KERNEL_H, art.dtUINT32, k),
                 _single(art.SETTING_CONV_2D_KERNEL_W, art.dtUINT32, k), _single(art.SETTING_CONV_2D_PAD_H, art.dtUINT32, a["pad"]),
                 _single(art.SETTING_CONV_2D_PAD_W, art.dtUINT32, a["pad"]), _single(art.SETTING_CONV_2D_STRIDE_H, art.dtUINT32, a["stride"]),
                 _single(art.SETTING_CONV_2D_STRIDE_W, art.dtUINT32, a["stride"]), _single(art.SETTING_CONV_2D_GROUP, art.dtUINT32, a["group"])]
            s += _quant(ialpha=xs[0].alpha, izp=xs[0].zp, walpha=a["walpha"], wzp=a["wzp"], oalpha=y.alpha, ozp=y.zp)
            ops.append((GROUP | art.OP_CONV_2D, ins + [index[a["w"]], index[a["b"]]], s))
            if a["relu"]:
                nxt += 1  # the conv's own output tensor; the relu's output takes the node's name below
                ops.append((GROUP | art.OP_RELU, [nxt - 1], _quant(ialpha=y.alpha, izp=y.zp, oalpha=y.alpha, ozp=y.zp)))
        elif node.kind == "ip":
            s = [_single(art.SETTING_IP_NUM_OUTPUT, art.dtUINT32, a["K"])]
            s += _quant(ialpha=xs[0].alpha, izp=xs[0].zp, walpha=a["walpha"], wzp=a["wzp"], oalpha=y.alpha, ozp=y.zp)
            ops.append((GROUP | art.OP_IP, ins + [index[a["w"]], index[a["b"]]], s))
        elif node.kind == "pool":
            s = [_single(art.SETTING_POOL_KERNEL_H, art.dtUINT32, a["k"]), _single(art.SETTING_POOL_KERNEL_W, art.dtUINT32, a["k"]),
                 _single(art.SETTING_POOL_PAD_H, art.dtUINT32, a["pad"]), _single(art.SETTING_POOL_PAD_W, art.dtUINT32, a["pad"]),
                 _single(art.SETTING_POOL_STRIDE_H, art.dtUINT32, a["stride"]), _single(art.SETTING_POOL_STRIDE_W, art.dtUINT32, a["stride"]),
                 _single(art.SETTING_POOL_METHOD, art.dtUINT32, a["method"]), _single(art.SETTING_POOL_CEIL_MODE, art.dtBOOL, bool(a["ceil_mode"]))]
            s += _quant(ialpha=xs[0].alpha, izp=xs[0].zp, oalpha=y.alpha, ozp=y.zp)
            ops.append((GROUP | art.OP_POOL, ins, s))
        elif node.kind == "add":
            s = _quant(ialpha=[xs[0].alpha, xs[1].alpha], izp=[xs[0].zp, xs[1].zp], oalpha=y.alpha, ozp=y.zp)
            ops.append((GROUP | art.OP_ADD, ins, s))
        else:
            raise ValueError(node.kind)
        index[y.name] = nxt
        nxt += 1

    assert version in (1, 2) and (transform is None or version == 2)
    out = [_i32(version), _str(case.name), _i32(nxt)]
    out.append(_i32(len(inputs)))
    for t in inputs:
        out += [struct.pack("<I", art.dtFLOAT32 if t.dtype == "f32" else art.dtUINT8), _str(t.name), _shape(t.shape)]
        if version == 2:
            out.append(_i32(1 if transform else 0))
            if transform:
                oprs, frame_type, mean, std, pad = transform
                out += [struct.pack("<Ii", oprs, frame_type), struct.pack("<9f", *mean, *std, *pad)]
    out.append(_i32(len(weights)))
    for name, arr in weights:
        arr = np.ascontiguousarray(arr)
        out += [struct.pack("<I", art._NP2DT[arr.dtype]), _str(name), _shape(arr.shape), arr.tobytes()]
    out.append(_i32(len(ops)))
    for code, ins, settings in ops:
        out += [_i32(len(ins)), _i32(1), struct.pack("<Q", code)] + [_i32(i) for i in ins] + [_i32(len(settings))] + settings
    out += [_i32(1), _i32(index[case.output.name]), _str(case.output.name), _i32(0)]
    return b"".join(out)


class Parade:
    """A loaded case: deserialize_parade + parade_prepare on any art-ABI runtime (the counterpart of the
    reference's `_art.Parade`, python/src/art/module.cpp:193-216)."""

    _READ = C.CFUNCTYPE(C.c_size_t, C.c_size_t, C.c_void_p, C.c_void_p)

    class _Param(C.Structure):
        _fields_ = [("workspaces", C.POINTER(C.POINTER(art.workspace_t))), ("input_mem_tp", C.POINTER(art.mem_tp))]

    def __init__(self, rt, data, workspaces, input_workspace=None, prepare=True):
        core = rt.core
        self.rt, self.workspaces = rt, list(workspaces)
        pos = [0]

        def read(sz, dst, _):
            chunk = data[pos[0]:pos[0] + sz]
            C.memmove(dst, chunk, len(chunk))
            pos[0] += len(chunk)
            return len(chunk)
        cb = self._READ(read)
        core.nart_buffer_new.restype = C.c_void_p
        core.nart_buffer_new.argtypes = [C.c_size_t]
        core.buffer_set_buffer_read_func.argtypes = [C.c_void_p, self._READ, C.c_void_p]
        core.nart_buffer_delete.argtypes = [C.c_void_p]
        core.deserialize_parade.restype = C.c_void_p
        core.deserialize_parade.argtypes = [C.c_void_p, C.POINTER(self._Param)]
        for f in ("parade_prepare", "parade_run", "parade_delete"):
            getattr(core, f).argtypes = [C.c_void_p]
        core.parade_apply_reshape.argtypes = [C.c_void_p]
        core.parade_apply_reshape.restype = C.c_bool
        gt = [C.c_void_p, C.POINTER(C.c_size_t), C.POINTER(C.POINTER(C.POINTER(art.tensor_t)))]
        core.parade_get_input_tensors.argtypes = gt
        core.parade_get_output_tensors.argtypes = gt
        buf = core.nart_buffer_new(1 << 20)
        core.buffer_set_buffer_read_func(buf, cb, None)
        ws_arr = (C.POINTER(art.workspace_t) * (len(workspaces) + 1))(*[w.ptr for w in workspaces], None)
        iw = input_workspace or workspaces[0]
        param = self._Param(ws_arr, iw.memtype)
        self.ptr = core.deserialize_parade(buf, C.byref(param))
        core.nart_buffer_delete(buf)
        assert self.ptr, "deserialize_parade failed"
        if prepare:
            core.parade_prepare(self.ptr)

    def transform_param(self):
        """(operators, means, stds, paddings) of input 0's pre-processing block (parade_get_transfrom_param, parade.c:128-138;
        only meaningful for a version-2 file whose input carries one)."""
        class Pixel(C.Structure):
            _fields_ = [("r", C.c_float), ("g", C.c_float), ("b", C.c_float)]

        class Param(C.Structure):  # transform_param_t, transform.h:54-67
            _fields_ = [("tensor_name", C.c_char_p), ("operators", C.c_uint32), ("batch", C.c_size_t), ("frames", C.c_void_p),
                        ("tensor_type", C.c_int32), ("rois", C.c_void_p), ("dst_rois", C.c_void_p), ("mats", C.c_void_p),
                        ("means", Pixel), ("stds", Pixel), ("paddings", Pixel)]
        f = self.rt.core.parade_get_transfrom_param
        f.restype, f.argtypes = C.c_bool, [C.c_void_p, C.POINTER(C.c_size_t), C.POINTER(Param)]
        n, prm = C.c_size_t(), Param()
        assert f(self.ptr, C.byref(n), C.byref(prm))
        px = lambda q: (q.r, q.g, q.b)  # noqa: E731
        return prm.operators, px(prm.means), px(prm.stds), px(prm.paddings)

    def _tensors(self, getter):
        n, arr = C.c_size_t(), C.POINTER(C.POINTER(art.tensor_t))()
        getter(self.ptr, C.byref(n), C.byref(arr))
        return [art.Tensor(self.rt, arr[i], owned=False) for i in range(n.value)]

    def inputs(self):
        return self._tensors(self.rt.core.parade_get_input_tensors)

    def outputs(self):
        return self._tensors(self.rt.core.parade_get_output_tensors)

    def run(self):
        self.rt.core.parade_run(self.ptr)

    def forward(self, x):
        self.inputs()[0].write(x)
        self.run()
        return self.outputs()[0].numpy()

    def delete(self):
        if self.ptr:
            self.rt.core.parade_delete(self.ptr)
            self.ptr = None
