"""numpy-facing wrapper of the CPU oracle (oracle/quant_oracle.c).

TEST INFRASTRUCTURE ONLY: imported by tests/, by the smoke check and by the benchmark's cpu_baseline
leg; never by the product package.  Tensors are NCHW numpy arrays, exactly as the reference CPU
`quant` module sees them.
"""
import ctypes as C
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB = None


def build():
    subprocess.check_call(["make", "-s", "-C", _HERE, "oracle"])


def lib():
    global _LIB
    if _LIB is None:
        path = os.path.join(_HERE, "liborc.so")
        if not os.path.exists(path):
            build()
        L = C.CDLL(path)
        L.orc_rshift_rn.restype = C.c_int64
        L.orc_rshift_rn.argtypes = [C.c_int64, C.c_int]
        L.orc_sat_bits.restype = C.c_uint8
        L.orc_conv_out_dim.restype = C.c_int
        L.orc_pool_out_dim.restype = C.c_int
        L.orc_fnv1a64.restype = C.c_uint64
        L.orc_fnv1a64.argtypes = [C.c_void_p, C.c_size_t]
        L.orc_quant_scale.argtypes = [C.c_float, C.c_int, C.POINTER(C.c_uint32), C.POINTER(C.c_int)]
        L.orc_requant_per_channel_u8.argtypes = [C.c_void_p, C.c_void_p, C.c_size_t, C.c_size_t, C.c_size_t, C.c_float,
                                                 C.c_void_p, C.c_float, C.c_int, C.c_int]
        L.orc_requant_per_channel_i8.argtypes = [C.c_void_p, C.c_void_p, C.c_size_t, C.c_size_t, C.c_size_t, C.c_float,
                                                 C.c_void_p, C.c_float, C.c_int]
        _LIB = L
    return _LIB


def _p(a):
    return C.c_void_p(a.ctypes.data) if a is not None else C.c_void_p(0)


def _f(v):
    return C.c_float(np.float32(v))


def quant_scale(x, bits):
    m, s = C.c_uint32(), C.c_int()
    lib().orc_quant_scale(_f(x), bits, C.byref(m), C.byref(s))
    return m.value, s.value


def rshift_rn(x, bits):
    return lib().orc_rshift_rn(int(x), int(bits))


def conv_out_dim(i, pad, k, stride):
    return lib().orc_conv_out_dim(i, pad, k, stride)


def pool_out_dim(i, pad, k, stride, ceil_mode, any_pad=None):
    any_pad = pad if any_pad is None else any_pad
    return lib().orc_pool_out_dim(i, pad, k, stride, int(bool(ceil_mode)), int(bool(any_pad)))


def fnv1a64(a):
    a = np.ascontiguousarray(a)
    return lib().orc_fnv1a64(_p(a), a.nbytes)


def _pair(v):
    return (v, v) if np.isscalar(v) else tuple(v)


def conv2d_u8(x, w, bias, pad, stride, group, ialpha, izp, walpha, wzp, oalpha, ozp, obits=8,
              return_acc=False, refshape=False):
    x = np.ascontiguousarray(x, np.uint8)
    w = np.ascontiguousarray(w, np.uint8)
    bias = None if bias is None else np.ascontiguousarray(bias, np.int32)
    N, Cc, H, W = x.shape
    K, _, R, S = w.shape
    (ph, pw), (sh, sw) = _pair(pad), _pair(stride)
    OH, OW = conv_out_dim(H, ph, R, sh), conv_out_dim(W, pw, S, sw)
    y = np.empty((N, K, OH, OW), np.uint8)
    if refshape:
        lib().orc_conv2d_u8_refshape(_p(x), _p(w), _p(bias), _p(y), N, Cc, H, W, K, R, S, ph, pw, sh,
                                     sw, group, _f(ialpha), int(izp), _f(walpha), int(wzp),
                                     _f(oalpha), int(ozp), int(obits))
        return y
    acc = np.empty((N, K, OH, OW), np.int32) if return_acc else None
    lib().orc_conv2d_u8(_p(x), _p(w), _p(bias), _p(y), _p(acc), N, Cc, H, W, K, R, S, ph, pw, sh, sw,
                        group, _f(ialpha), int(izp), _f(walpha), int(wzp), _f(oalpha), int(ozp),
                        int(obits))
    return (y, acc) if return_acc else y


def ip_u8(x, w, bias, ialpha, izp, walpha, wzp, oalpha, ozp, obits=8, return_acc=False):
    x = np.ascontiguousarray(x, np.uint8)
    w = np.ascontiguousarray(w, np.uint8)
    bias = None if bias is None else np.ascontiguousarray(bias, np.int32)
    M = x.shape[0]
    Kd = int(np.prod(x.shape[1:]))
    Nout = w.shape[0]
    assert int(np.prod(w.shape[1:])) == Kd
    y = np.empty((M, Nout), np.uint8)
    acc = np.empty((M, Nout), np.int32) if return_acc else None
    lib().orc_ip_u8(_p(x), _p(w), _p(bias), _p(y), _p(acc), M, Kd, Nout, _f(ialpha), int(izp),
                    _f(walpha), int(wzp), _f(oalpha), int(ozp), int(obits))
    return (y, acc) if return_acc else y


def add_u8(a, b, ialpha0, izp0, ialpha1, izp1, oalpha, ozp, obits=8):
    a = np.ascontiguousarray(a, np.uint8)
    b = np.ascontiguousarray(b, np.uint8)
    y = np.empty_like(a)
    lib().orc_add_u8(_p(a), _p(b), _p(y), C.c_size_t(a.size), _f(ialpha0), int(izp0), _f(ialpha1),
                     int(izp1), _f(oalpha), int(ozp), int(obits))
    return y


def eltwise_u8(ins, ialpha, izp, oalpha, ozp, operation=1, coeff=None, obits=8):
    ins = [np.ascontiguousarray(a, np.uint8) for a in ins]
    n = len(ins)
    ptrs = (C.c_void_p * n)(*[a.ctypes.data for a in ins])
    ia = np.ascontiguousarray(ialpha, np.float32)
    iz = np.ascontiguousarray(izp, np.uint8)
    cf = None if coeff is None else np.ascontiguousarray(coeff, np.float32)
    y = np.empty_like(ins[0])
    lib().orc_eltwise_u8(ptrs, n, _p(cf), _p(ia), _p(iz), _p(y), C.c_size_t(y.size), int(operation),
                         _f(oalpha), int(ozp), int(obits))
    return y


def relu_u8(x, ialpha, izp, oalpha, ozp, obits=8):
    x = np.ascontiguousarray(x, np.uint8)
    y = np.empty_like(x)
    lib().orc_relu_u8(_p(x), _p(y), C.c_size_t(x.size), _f(ialpha), int(izp), _f(oalpha), int(ozp),
                      int(obits))
    return y


def pool_u8(x, kernel, pad, stride, method, ceil_mode, ialpha, izp, oalpha, ozp, obits=8):
    x = np.ascontiguousarray(x, np.uint8)
    N, Cc, H, W = x.shape
    (kh, kw), (ph, pw), (sh, sw) = _pair(kernel), _pair(pad), _pair(stride)
    OH = pool_out_dim(H, ph, kh, sh, ceil_mode, ph or pw)
    OW = pool_out_dim(W, pw, kw, sw, ceil_mode, ph or pw)
    if (OH - 1) * sh - ph >= H + ph or (OW - 1) * sw - pw >= W + pw:
        # an empty last window (ceil mode without padding): the average's divisor is 0 and the reference's scale search
        # (quant_helper.h:60-118) never ends on the infinite scale
        raise ValueError("pool_u8: a window lies outside the image")
    y = np.empty((N, Cc, OH, OW), np.uint8)
    lib().orc_pool_u8(_p(x), _p(y), N, Cc, H, W, OH, OW, kh, kw, ph, pw, sh, sw, int(method),
                      _f(ialpha), int(izp), _f(oalpha), int(ozp), int(obits))
    return y


def quantize_u8(x, oalpha, ozp, obits=8):
    x = np.ascontiguousarray(x, np.float32)
    y = np.empty(x.shape, np.uint8)
    lib().orc_quantize_u8(_p(x), _p(y), C.c_size_t(x.size), _f(oalpha), int(ozp), int(obits))
    return y


def dequantize_u8(x, ialpha, izp):
    x = np.ascontiguousarray(x, np.uint8)
    y = np.empty(x.shape, np.float32)
    lib().orc_dequantize_u8(_p(x), _p(y), C.c_size_t(x.size), _f(ialpha), int(izp))
    return y


def dequantize_i32(acc, alpha):
    """int32 accumulators -> fp32: (float)acc * alpha.  No counterpart in the reference (closed form only)."""
    acc = np.ascontiguousarray(acc, np.int32)
    y = np.empty(acc.shape, np.float32)
    lib().orc_dequantize_i32(_p(acc), _p(y), C.c_size_t(acc.size), _f(alpha))
    return y


def concat_u8(ins, ialpha, izp, oalpha, ozp, obits=8):
    """Concatenation along dimension 1 with per-input rescaling (the reference ignores `axis`, concat.c:99-121)."""
    ins = [np.ascontiguousarray(a, np.uint8) for a in ins]
    n = len(ins)
    N = ins[0].shape[0]
    per = (C.c_size_t * n)(*[a.size // N for a in ins])
    ptrs = (C.c_void_p * n)(*[a.ctypes.data for a in ins])
    ia = np.ascontiguousarray(ialpha, np.float32)
    iz = np.ascontiguousarray(izp, np.uint8)
    shape = list(ins[0].shape)
    shape[1] = sum(a.shape[1] for a in ins)
    y = np.empty(shape, np.uint8)
    lib().orc_concat_u8(ptrs, n, per, _p(ia), _p(iz), _p(y), N, _f(oalpha), int(ozp), int(obits))
    return y


def softmax_u8(x, axis, ialpha, izp, oalpha, ozp, obits=8):
    x = np.ascontiguousarray(x, np.uint8)
    ch = x.shape[axis]
    outer = int(np.prod(x.shape[:axis], dtype=np.int64))
    inner = int(np.prod(x.shape[axis + 1:], dtype=np.int64))
    y = np.empty(x.shape, np.uint8)
    lib().orc_softmax_u8(_p(x), _p(y), C.c_size_t(outer), C.c_size_t(ch), C.c_size_t(inner), _f(ialpha), int(izp),
                         _f(oalpha), int(ozp), int(obits))
    return y


def conv2d_i8(x, w, bias, pad, stride, group, ialpha, walpha, oalpha, obits=8, return_acc=False):
    x = np.ascontiguousarray(x, np.int8)
    w = np.ascontiguousarray(w, np.int8)
    bias = None if bias is None else np.ascontiguousarray(bias, np.int32)
    N, Cc, H, W = x.shape
    K, _, R, S = w.shape
    (ph, pw), (sh, sw) = _pair(pad), _pair(stride)
    OH, OW = conv_out_dim(H, ph, R, sh), conv_out_dim(W, pw, S, sw)
    y = np.empty((N, K, OH, OW), np.int8)
    acc = np.empty((N, K, OH, OW), np.int32) if return_acc else None
    lib().orc_conv2d_i8(_p(x), _p(w), _p(bias), _p(y), _p(acc), N, Cc, H, W, K, R, S, ph, pw, sh, sw, group,
                        _f(ialpha), _f(walpha), _f(oalpha), int(obits))
    return (y, acc) if return_acc else y


def ip_i8(x, w, bias, ialpha, walpha, oalpha, obits=8, return_acc=False):
    x = np.ascontiguousarray(x, np.int8)
    w = np.ascontiguousarray(w, np.int8)
    bias = None if bias is None else np.ascontiguousarray(bias, np.int32)
    M = x.shape[0]
    Kd = int(np.prod(x.shape[1:]))
    Nout = w.shape[0]
    assert int(np.prod(w.shape[1:])) == Kd
    y = np.empty((M, Nout), np.int8)
    acc = np.empty((M, Nout), np.int32) if return_acc else None
    lib().orc_ip_i8(_p(x), _p(w), _p(bias), _p(y), _p(acc), M, Kd, Nout, _f(ialpha), _f(walpha), _f(oalpha),
                    int(obits))
    return (y, acc) if return_acc else y


def quantize_i8(x, oalpha, obits=8):
    x = np.ascontiguousarray(x, np.float32)
    y = np.empty(x.shape, np.int8)
    lib().orc_quantize_i8(_p(x), _p(y), C.c_size_t(x.size), _f(oalpha), int(obits))
    return y


def dequantize_i8(x, ialpha):
    x = np.ascontiguousarray(x, np.int8)
    y = np.empty(x.shape, np.float32)
    lib().orc_dequantize_i8(_p(x), _p(y), C.c_size_t(x.size), _f(ialpha))
    return y


def requant_per_channel_u8(acc, ialpha, walpha, oalpha, ozp, obits=8):
    """acc: int32 [N, K, ...] (or [M, K]); walpha: K floats.  See quant_oracle.h."""
    acc = np.ascontiguousarray(acc, np.int32)
    wa = np.ascontiguousarray(walpha, np.float32).reshape(-1)
    outer, K = acc.shape[0], acc.shape[1]
    assert wa.size == K
    inner = int(np.prod(acc.shape[2:])) if acc.ndim > 2 else 1
    y = np.empty(acc.shape, np.uint8)
    lib().orc_requant_per_channel_u8(_p(acc), _p(y), outer, K, inner, _f(ialpha), _p(wa), _f(oalpha), int(ozp), int(obits))
    return y


def requant_per_channel_i8(acc, ialpha, walpha, oalpha, obits=8):
    acc = np.ascontiguousarray(acc, np.int32)
    wa = np.ascontiguousarray(walpha, np.float32).reshape(-1)
    outer, K = acc.shape[0], acc.shape[1]
    assert wa.size == K
    inner = int(np.prod(acc.shape[2:])) if acc.ndim > 2 else 1
    y = np.empty(acc.shape, np.int8)
    lib().orc_requant_per_channel_i8(_p(acc), _p(y), outer, K, inner, _f(ialpha), _p(wa), _f(oalpha), int(obits))
    return y


def conv2d_u8_per_channel(x, w, bias, pad, stride, group, ialpha, izp, walpha, wzp, oalpha, ozp, obits=8):
    """walpha: K floats.  The accumulators do not depend on the scales."""
    _, acc = conv2d_u8(x, w, bias, pad, stride, group, ialpha, izp, float(np.float32(walpha[0])), wzp, oalpha, ozp, obits,
                       return_acc=True)
    return requant_per_channel_u8(acc, ialpha, walpha, oalpha, ozp, obits)


class XorShift:
    """The generator of the recorded conv known answers (state 0x9E3779B97F4A7C15 at the start of a case)."""

    def __init__(self, seed=0x9E3779B97F4A7C15):
        self.state = C.c_uint64(seed)

    def u32(self, n):
        out = np.empty(n, np.uint32)
        lib().orc_xorshift_fill(C.byref(self.state), _p(out), C.c_size_t(n))
        return out
