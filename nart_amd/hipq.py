"""ctypes binding of the hipq C ABI (include/hipq.h) for Python callers.

PyTorch is used for one thing only: owning device memory and streams (torch.uint8 / float32 CUDA
tensors whose data_ptr() is handed to the library).  All arithmetic happens in the HIP kernels; there
is no host fallback — loading fails loudly if the library has not been built.
"""
import ctypes as C
import os
import re

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "lib", "libhipq.so")
_LIB = None


class HipqError(RuntimeError):
    pass


class ConvDesc(C.Structure):  # hipq_conv2d_desc
    _fields_ = [(n, C.c_int32) for n in ("N", "C", "H", "W", "K", "R", "S", "pad_h", "pad_w", "stride_h",
                                         "stride_w", "group", "in_cs", "out_cs")] \
        + [(n, C.c_float) for n in ("ialpha", "walpha", "oalpha")] \
        + [(n, C.c_int32) for n in ("izp", "wzp", "ozp", "obits", "relu", "dtype")]


DTYPE_U8, DTYPE_I8 = 0, 1
TILE_INDEX = {"128x128": 0, "256x64": 1, "128x64": 2, "64x128": 3, "64x64": 4}  # hipq_conv2d_plan_select


# every symbol include/hipq.h declares, with its signature
_SIGS = {
    "hipq_abi_version": (C.c_int, []),
    "hipq_last_error": (C.c_char_p, []),
    "hipq_quant_scale": (None, [C.c_float, C.c_int, C.POINTER(C.c_uint32), C.POINTER(C.c_int)]),
    "hipq_channel_stride": (C.c_int, [C.c_int]),
    "hipq_div_magic": (C.c_int, [C.c_uint32, C.POINTER(C.c_uint32), C.POINTER(C.c_int)]),
    "hipq_nchw_to_nhwc_u8": (C.c_int, [C.c_void_p, C.c_void_p] + [C.c_int] * 5 + [C.c_void_p]),
    "hipq_nhwc_to_nchw_u8": (C.c_int, [C.c_void_p, C.c_void_p] + [C.c_int] * 5 + [C.c_void_p]),
    "hipq_conv2d_plan_create": (C.c_int, [C.POINTER(ConvDesc), C.c_void_p, C.c_void_p, C.POINTER(C.c_void_p)]),
    "hipq_conv2d_plan_create_per_channel": (C.c_int, [C.POINTER(ConvDesc), C.c_void_p, C.c_void_p, C.c_void_p,
                                                      C.POINTER(C.c_void_p)]),
    "hipq_conv2d_plan_destroy": (None, [C.c_void_p]),
    "hipq_conv2d_plan_kernel": (C.c_char_p, [C.c_void_p]),
    "hipq_conv2d_plan_kernel_add": (C.c_char_p, [C.c_void_p]),
    "hipq_conv2d_dequant_fusable": (C.c_int, [C.c_void_p, C.c_float, C.c_int]),
    "hipq_conv2d_run_dequant": (C.c_int, [C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p]),
    "hipq_conv2d_plan_select": (C.c_int, [C.c_void_p, C.c_int, C.c_int]),
    "hipq_conv2d_plan_special": (C.c_int, [C.c_void_p, C.c_int]),
    "hipq_conv2d_plan_stream": (C.c_int, [C.c_void_p, C.c_int, C.c_int, C.c_int]),
    "hipq_conv2d_run_relu": (C.c_int, [C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p]),
    "hipq_conv2d_run": (C.c_int, [C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p]),
    "hipq_conv2d_run_add": (C.c_int, [C.c_void_p, C.c_void_p, C.c_void_p, C.c_int, C.c_float, C.c_int, C.c_float, C.c_int,
                                      C.c_int, C.c_void_p, C.c_void_p]),
    "hipq_conv2d_add_conv_fusable": (C.c_int, [C.c_void_p, C.c_int, C.c_float, C.c_int, C.c_float, C.c_int, C.c_int, C.c_void_p]),
    "hipq_conv2d_run_add_conv": (C.c_int, [C.c_void_p, C.c_void_p, C.c_void_p, C.c_int, C.c_float, C.c_int, C.c_float, C.c_int,
                                           C.c_int, C.c_void_p, C.c_void_p, C.c_int, C.c_void_p, C.c_void_p]),
    "hipq_conv2d_add2_fusable": (C.c_int, [C.c_void_p, C.c_void_p, C.c_int, C.c_float, C.c_int, C.c_int]),
    "hipq_conv2d_run_add2": (C.c_int, [C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_int, C.c_float, C.c_int, C.c_int,
                                       C.c_void_p, C.c_void_p]),
    "hipq_bottleneck_fusable": (C.c_int, [C.c_void_p, C.c_void_p, C.c_void_p, C.c_int, C.c_float, C.c_int, C.c_int]),
    "hipq_bottleneck_conv_fusable": (C.c_int, [C.c_void_p, C.c_void_p, C.c_void_p, C.c_int, C.c_float, C.c_int, C.c_int, C.c_void_p]),
    "hipq_bottleneck_run_conv": (C.c_int, [C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_int, C.c_float, C.c_int, C.c_int,
                                           C.c_void_p, C.c_void_p, C.c_int, C.c_void_p, C.c_void_p]),
    "hipq_bottleneck_run": (C.c_int, [C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_int, C.c_float, C.c_int, C.c_int,
                                      C.c_void_p, C.c_void_p]),
    "hipq_bottleneck_tail_fusable": (C.c_int, [C.c_void_p, C.c_void_p, C.c_int, C.c_float, C.c_int, C.c_float, C.c_int, C.c_int,
                                               C.c_void_p]),
    "hipq_bottleneck_tail_run": (C.c_int, [C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_int, C.c_float, C.c_int, C.c_float,
                                           C.c_int, C.c_int, C.c_void_p, C.c_void_p, C.c_int, C.c_void_p, C.c_void_p]),
    "hipq_conv2d_maxpool_fusable": (C.c_int, [C.c_void_p] + [C.c_int] * 5 + [C.c_float, C.c_int, C.c_float, C.c_int, C.c_int]),
    "hipq_conv2d_run_maxpool": (C.c_int, [C.c_void_p, C.c_void_p, C.c_void_p, C.c_int, C.c_int, C.c_int, C.c_void_p]),
    "hipq_conv2d_maxpool_conv_fusable": (C.c_int, [C.c_void_p, C.c_int, C.c_int, C.c_void_p, C.c_void_p]),
    "hipq_conv2d_run_maxpool_conv": (C.c_int, [C.c_void_p, C.c_void_p, C.c_void_p, C.c_int, C.c_int, C.c_int, C.c_void_p, C.c_int,
                                               C.c_void_p, C.c_void_p, C.c_int, C.c_void_p, C.c_void_p]),
    "hipq_ip_reorder_weights": (C.c_int, [C.c_void_p, C.c_void_p] + [C.c_int] * 6),
    "hipq_add_u8": (C.c_int, [C.c_void_p, C.c_void_p, C.c_void_p, C.c_size_t, C.c_float, C.c_int, C.c_float,
                              C.c_int, C.c_float, C.c_int, C.c_int, C.c_void_p]),
    "hipq_eltwise_u8": (C.c_int, [C.POINTER(C.c_void_p), C.c_int, C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p,
                                  C.c_size_t, C.c_int, C.c_float, C.c_int, C.c_int, C.c_void_p]),
    "hipq_relu_u8": (C.c_int, [C.c_void_p, C.c_void_p, C.c_size_t, C.c_float, C.c_int, C.c_float, C.c_int,
                               C.c_int, C.c_void_p]),
    "hipq_concat_u8": (C.c_int, [C.POINTER(C.c_void_p), C.c_int, C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_size_t,
                                 C.c_float, C.c_int, C.c_int, C.c_void_p]),
    "hipq_softmax_u8": (C.c_int, [C.c_void_p, C.c_void_p, C.c_size_t, C.c_int, C.c_int, C.c_float, C.c_int, C.c_float,
                                  C.c_int, C.c_int, C.c_void_p]),
    "hipq_pool_u8": (C.c_int, [C.c_void_p, C.c_void_p] + [C.c_int] * 14 + [C.c_float, C.c_int, C.c_float, C.c_int,
                                                                          C.c_int, C.c_void_p]),
    "hipq_quantize_u8": (C.c_int, [C.c_void_p, C.c_void_p] + [C.c_int] * 5 + [C.c_float, C.c_int, C.c_int, C.c_void_p]),
    "hipq_dequantize_u8": (C.c_int, [C.c_void_p, C.c_void_p] + [C.c_int] * 5 + [C.c_float, C.c_int, C.c_void_p]),
    "hipq_quantize_i8": (C.c_int, [C.c_void_p, C.c_void_p] + [C.c_int] * 5 + [C.c_float, C.c_int, C.c_void_p]),
    "hipq_dequantize_i8": (C.c_int, [C.c_void_p, C.c_void_p] + [C.c_int] * 5 + [C.c_float, C.c_void_p]),
    "hipq_dequantize_i32": (C.c_int, [C.c_void_p, C.c_void_p] + [C.c_int] * 5 + [C.c_float, C.c_void_p]),
    "hipq_copy_bytes": (C.c_int, [C.c_void_p, C.c_void_p, C.c_size_t, C.c_void_p]),
}
EXPORTS = tuple(_SIGS)


def lib():
    global _LIB
    if _LIB is None:
        if not os.path.exists(LIB_PATH):
            raise HipqError("%s is missing: build it with `python -m nart_amd.build`" % LIB_PATH)
        L = C.CDLL(LIB_PATH)
        for name, (res, args) in _SIGS.items():
            f = getattr(L, name)  # AttributeError here = the library does not export a declared symbol
            f.restype, f.argtypes = res, args
        _LIB = L
    return _LIB


def check(rc):
    if rc != 0:
        raise HipqError(lib().hipq_last_error().decode() or "hipq call failed (%d)" % rc)


def channel_stride(c):
    return lib().hipq_channel_stride(int(c))


def quant_scale(x, bits):
    m, s = C.c_uint32(), C.c_int()
    lib().hipq_quant_scale(C.c_float(np.float32(x)), bits, C.byref(m), C.byref(s))
    return m.value, s.value


def _stream():
    import torch
    return C.c_void_p(torch.cuda.current_stream().cuda_stream)


def _ptr(t):
    return C.c_void_p(t.data_ptr()) if t is not None else C.c_void_p(0)


def conv_out_dim(i, pad, k, stride):
    return (i + 2 * pad - k) // stride + 1


# ---- device tensors in the library's layout -------------------------------------------------------
def to_device_nhwc(x_nchw):
    """numpy uint8 [N,C,H,W] -> CUDA uint8 [N,H,W,cs] (channels-last, padded channel stride)."""
    import torch
    x = np.ascontiguousarray(x_nchw)
    x = x.view(np.uint8) if x.dtype == np.int8 else np.ascontiguousarray(x, np.uint8)  # int8 travels as its bytes
    N, Cc, H, W = x.shape
    cs = channel_stride(Cc)
    src = torch.from_numpy(x).cuda()
    dst = torch.empty((N, H, W, cs), dtype=torch.uint8, device="cuda")
    check(lib().hipq_nchw_to_nhwc_u8(_ptr(src), _ptr(dst), N, Cc, H, W, cs, _stream()))
    return dst


def from_device_nhwc(t, Cc):
    """CUDA uint8 [N,H,W,cs] -> numpy uint8 [N,C,H,W]."""
    import torch
    N, H, W, cs = t.shape
    dst = torch.empty((N, Cc, H, W), dtype=torch.uint8, device="cuda")
    check(lib().hipq_nhwc_to_nchw_u8(_ptr(t), _ptr(dst), N, Cc, H, W, cs, _stream()))
    return dst.cpu().numpy()


class Conv2d:
    """A convolution plan (weights packed and resident on the device) plus its launch."""

    def __init__(self, x_shape, w, bias, pad, stride, group, ialpha, izp, walpha, wzp, oalpha, ozp, obits=8,
                 relu=False, in_cs=None, out_cs=None, dtype=DTYPE_U8):
        """dtype=DTYPE_I8: int8 symmetric tensors (w is an int8 array, zero points are ignored).
        walpha: a float, or an array of K floats = one weight scale per output channel."""
        N, Cc, H, W = x_shape
        wa_pc = None
        if not np.isscalar(walpha):
            wa_pc = np.ascontiguousarray(walpha, np.float32).reshape(-1)
            assert wa_pc.size == np.asarray(w).shape[0], "one weight scale per output channel"
            walpha = float(wa_pc[0])
        w = np.ascontiguousarray(w, np.int8 if dtype == DTYPE_I8 else np.uint8)
        K, _, R, S = w.shape
        ph, pw = (pad, pad) if np.isscalar(pad) else pad
        sh, sw = (stride, stride) if np.isscalar(stride) else stride
        d = ConvDesc(N=N, C=Cc, H=H, W=W, K=K, R=R, S=S, pad_h=ph, pad_w=pw, stride_h=sh, stride_w=sw, group=group,
                     in_cs=in_cs or channel_stride(Cc), out_cs=out_cs or channel_stride(K),
                     ialpha=ialpha, walpha=walpha, oalpha=oalpha, izp=izp, wzp=wzp, ozp=ozp, obits=obits,
                     relu=int(relu), dtype=dtype)
        self.desc = d
        self.OH, self.OW = conv_out_dim(H, ph, R, sh), conv_out_dim(W, pw, S, sw)
        b = None if bias is None else np.ascontiguousarray(bias, np.int32)
        h = C.c_void_p()
        bp = C.c_void_p(b.ctypes.data) if b is not None else None
        if wa_pc is None:
            check(lib().hipq_conv2d_plan_create(C.byref(d), C.c_void_p(w.ctypes.data), bp, C.byref(h)))
        else:
            check(lib().hipq_conv2d_plan_create_per_channel(C.byref(d), C.c_void_p(w.ctypes.data), bp,
                                                            C.c_void_p(wa_pc.ctypes.data), C.byref(h)))
        self.handle = h
        self.kernel = lib().hipq_conv2d_plan_kernel(h).decode()
        m = re.match(r"conv_mfma_i8_(\d+x\d+)", self.kernel)
        self._tile0 = TILE_INDEX.get(m.group(1), -1) if m else -1  # the built-in choice, for the tuner to return to
        self.ops = 2 * N * K * self.OH * self.OW * (Cc // group) * R * S

    @property
    def kernel_add(self):
        """Name of the kernel run_add dispatches to ("" when the plan cannot fuse the add)."""
        return lib().hipq_conv2d_plan_kernel_add(self.handle).decode()

    def select(self, tile=-1, stages=0):
        """Tuning hook: work-group tile index and load stages of the MFMA kernel (include/hipq.h)."""
        check(lib().hipq_conv2d_plan_select(self.handle, tile, stages))
        self.kernel = lib().hipq_conv2d_plan_kernel(self.handle).decode()
        return self

    def dequant_fusable(self, alpha, zp):
        """True if run_dequant serves this plan and a dequantize with these settings (include/hipq.h)."""
        return bool(lib().hipq_conv2d_dequant_fusable(self.handle, float(alpha), int(zp)))

    def run_dequant(self, x, y):
        """The layer and the dequantize of its output in one launch: y (float32, N x K) receives the values."""
        import torch
        assert y.dtype == torch.float32 and y.is_contiguous() and y.numel() == self.desc.N * self.desc.K
        check(lib().hipq_conv2d_run_dequant(self.handle, _ptr(x), _ptr(y), _stream()))
        return y

    def special(self, mode=1):
        """Tuning hook: the halo-tile (3x3 stride 1), pointwise (small 1x1) and two-group (few tiles, long reduction)
        kernels: 0 never, 1 built-in rule, 2 wherever they apply (include/hipq.h)."""
        check(lib().hipq_conv2d_plan_special(self.handle, int(mode)))
        self.kernel = lib().hipq_conv2d_plan_kernel(self.handle).decode()
        return self

    def stream(self, rows=0, cols=0, waves=0):
        """Tuning hook: shape of the streaming (fully-connected) kernel's work-groups (include/hipq.h)."""
        check(lib().hipq_conv2d_plan_stream(self.handle, rows, cols, waves))
        self.kernel = lib().hipq_conv2d_plan_kernel(self.handle).decode()
        return self

    def empty_output(self):
        import torch
        d = self.desc
        return torch.empty((d.N, self.OH, self.OW, d.out_cs), dtype=torch.uint8, device="cuda")

    def __call__(self, x, y=None, acc=None):
        if y is None:
            y = self.empty_output()
        check(lib().hipq_conv2d_run(self.handle, _ptr(x), _ptr(y), _ptr(acc), _stream()))
        return y

    def run_relu(self, x, y=None):
        """y = max(conv(x), ozp) from a plan created without relu (include/hipq.h: hipq_conv2d_run_relu)."""
        if y is None:
            y = self.empty_output()
        check(lib().hipq_conv2d_run_relu(self.handle, _ptr(x), _ptr(y), _stream()))
        return y

    def run_add(self, x, residual, residual_first, res_alpha, res_zp, oalpha, ozp, y, obits=8):
        """y = add(conv(x), residual) in one launch (include/hipq.h: hipq_conv2d_run_add)."""
        check(lib().hipq_conv2d_run_add(self.handle, _ptr(x), _ptr(residual), int(bool(residual_first)), res_alpha, res_zp,
                                        oalpha, ozp, obits, _ptr(y), _stream()))
        return y

    def add_conv_fusable(self, residual_first, res_alpha, res_zp, oalpha, ozp, nxt, obits=8):
        """Can run_add and the 1x1 convolution `nxt` that reads the sum run as one kernel (include/hipq.h)?"""
        return bool(lib().hipq_conv2d_add_conv_fusable(self.handle, int(bool(residual_first)), res_alpha, res_zp, oalpha, ozp,
                                                       obits, nxt.handle))

    def run_add_conv(self, x, residual, residual_first, res_alpha, res_zp, oalpha, ozp, y, nxt, y_next, obits=8, next_relu=False):
        """y = add(conv(x), residual) and y_next = nxt(y) in one launch (include/hipq.h: hipq_conv2d_run_add_conv)."""
        check(lib().hipq_conv2d_run_add_conv(self.handle, _ptr(x), _ptr(residual), int(bool(residual_first)), res_alpha, res_zp,
                                             oalpha, ozp, obits, _ptr(y), nxt.handle, int(bool(next_relu)), _ptr(y_next), _stream()))
        return y, y_next

    def maxpool_fusable(self, OH, OW, kernel, stride, pad, ialpha, izp, oalpha, ozp, obits=8):
        """Can the 3x3 / stride 2 / pad 1 max pooling that follows run inside this convolution's kernel (include/hipq.h)?"""
        return bool(lib().hipq_conv2d_maxpool_fusable(self.handle, OH, OW, kernel, stride, pad, ialpha, izp, oalpha, ozp, obits))

    def run_maxpool(self, x, y, relu=False):
        """y = maxpool3x3/2/1(conv(x)) in one launch, with the ReLU clamp in between if relu; y: [N, OH, OW, 64]
        (include/hipq.h: hipq_conv2d_run_maxpool)."""
        check(lib().hipq_conv2d_run_maxpool(self.handle, _ptr(x), _ptr(y), y.shape[1], y.shape[2], int(bool(relu)), _stream()))
        return y

    def maxpool_conv_fusable(self, OH, OW, nxt, nxt2=None):
        """Can that pooling AND the 1x1 convolutions `nxt` (and `nxt2`) that read the pooled tensor run inside this
        convolution's kernel?"""
        return bool(lib().hipq_conv2d_maxpool_conv_fusable(self.handle, OH, OW, nxt.handle, nxt2.handle if nxt2 else None))

    def run_maxpool_conv(self, x, y, nxt, y_next, relu=False, next_relu=False, nxt2=None, y_next2=None, next2_relu=False):
        """y = maxpool3x3/2/1(conv(x)), y_next = nxt(y) and - given - y_next2 = nxt2(y) in one launch (include/hipq.h:
        hipq_conv2d_run_maxpool_conv)."""
        check(lib().hipq_conv2d_run_maxpool_conv(self.handle, _ptr(x), _ptr(y), y.shape[1], y.shape[2], int(bool(relu)),
                                                 nxt.handle, int(bool(next_relu)), _ptr(y_next), nxt2.handle if nxt2 else None,
                                                 int(bool(next2_relu)), _ptr(y_next2) if y_next2 is not None else None, _stream()))
        return y, y_next, y_next2

    def close(self):
        if self.handle:
            lib().hipq_conv2d_plan_destroy(self.handle)
            self.handle = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass


def add2_fusable(plan, shortcut, shortcut_first, oalpha, ozp, obits=8):
    """Can add(plan(x), shortcut(x_shortcut)) run as one kernel (include/hipq.h: hipq_conv2d_add2_fusable)?"""
    return bool(lib().hipq_conv2d_add2_fusable(plan.handle, shortcut.handle, int(bool(shortcut_first)), oalpha, ozp, obits))


def run_add2(plan, x, shortcut, x_shortcut, shortcut_first, oalpha, ozp, y, obits=8):
    """y = add(plan(x), shortcut(x_shortcut)) in one launch (include/hipq.h: hipq_conv2d_run_add2)."""
    check(lib().hipq_conv2d_run_add2(plan.handle, _ptr(x), shortcut.handle, _ptr(x_shortcut), int(bool(shortcut_first)), oalpha, ozp,
                                     obits, _ptr(y), _stream()))
    return y


def bottleneck_fusable(reduce, mid, widen, residual_first, oalpha, ozp, obits=8):
    """Can the identity bottleneck block reduce -> mid -> widen -> add(., x) run as one kernel (include/hipq.h)?"""
    return bool(lib().hipq_bottleneck_fusable(reduce.handle, mid.handle, widen.handle, int(bool(residual_first)), oalpha, ozp, obits))


def bottleneck_run(reduce, mid, widen, x, residual_first, oalpha, ozp, y, obits=8):
    """y = add(widen(mid(reduce(x))), x) in one launch (include/hipq.h: hipq_bottleneck_run)."""
    check(lib().hipq_bottleneck_run(reduce.handle, mid.handle, widen.handle, _ptr(x), int(bool(residual_first)), oalpha, ozp,
                                    obits, _ptr(y), _stream()))
    return y


def bottleneck_conv_fusable(reduce, mid, widen, residual_first, oalpha, ozp, nxt, obits=8):
    """Can that block AND the 1x1 convolution `nxt` that reads its sum run as one kernel (include/hipq.h)?"""
    return bool(lib().hipq_bottleneck_conv_fusable(reduce.handle, mid.handle, widen.handle, int(bool(residual_first)), oalpha, ozp,
                                                   obits, nxt.handle))


def bottleneck_run_conv(reduce, mid, widen, x, residual_first, oalpha, ozp, y, nxt, y_next, obits=8, next_relu=False):
    """y = add(widen(mid(reduce(x))), x) and y_next = nxt(y) in one launch (include/hipq.h: hipq_bottleneck_run_conv)."""
    check(lib().hipq_bottleneck_run_conv(reduce.handle, mid.handle, widen.handle, _ptr(x), int(bool(residual_first)), oalpha, ozp,
                                         obits, _ptr(y), nxt.handle, int(bool(next_relu)), _ptr(y_next), _stream()))
    return y, y_next


def bottleneck_tail_fusable(mid, widen, residual_first, res_alpha, res_zp, oalpha, ozp, nxt=None, obits=8):
    """Can mid (3x3) -> widen (1x1) -> add(., residual) [-> nxt (1x1)] run as one kernel (include/hipq.h)?"""
    return bool(lib().hipq_bottleneck_tail_fusable(mid.handle, widen.handle, int(bool(residual_first)), res_alpha, res_zp, oalpha,
                                                   ozp, obits, nxt.handle if nxt is not None else None))


def bottleneck_tail_run(mid, widen, x, residual, residual_first, res_alpha, res_zp, oalpha, ozp, y, nxt=None, y_next=None,
                        next_relu=False, obits=8):
    """y = add(widen(mid(x)), residual) and y_next = nxt(y) in one launch (include/hipq.h: hipq_bottleneck_tail_run)."""
    check(lib().hipq_bottleneck_tail_run(mid.handle, widen.handle, _ptr(x), _ptr(residual), int(bool(residual_first)), res_alpha,
                                         res_zp, oalpha, ozp, obits, _ptr(y), nxt.handle if nxt is not None else None,
                                         int(bool(next_relu)), _ptr(y_next), _stream()))
    return y


def add_u8(a, b, y, ialpha0, izp0, ialpha1, izp1, oalpha, ozp, obits=8):
    check(lib().hipq_add_u8(_ptr(a), _ptr(b), _ptr(y), a.numel(), ialpha0, izp0, ialpha1, izp1, oalpha, ozp, obits,
                            _stream()))
    return y


def eltwise_u8(ins, y, ialpha, izp, oalpha, ozp, operation=1, coeff=None, obits=8):
    n = len(ins)
    ptrs = (C.c_void_p * n)(*[t.data_ptr() for t in ins])
    ia = np.ascontiguousarray(ialpha, np.float32)
    iz = np.ascontiguousarray(izp, np.uint8)
    cf = None if coeff is None else np.ascontiguousarray(coeff, np.float32)
    check(lib().hipq_eltwise_u8(ptrs, n, C.c_void_p(cf.ctypes.data) if cf is not None else None,
                                C.c_void_p(ia.ctypes.data), C.c_void_p(iz.ctypes.data), _ptr(y), y.numel(),
                                operation, oalpha, ozp, obits, _stream()))
    return y


def relu_u8(x, y, ialpha, izp, oalpha, ozp, obits=8):
    check(lib().hipq_relu_u8(_ptr(x), _ptr(y), x.numel(), ialpha, izp, oalpha, ozp, obits, _stream()))
    return y


def concat_u8(ins, channels, y, ialpha, izp, oalpha, ozp, obits=8):
    n = len(ins)
    ptrs = (C.c_void_p * n)(*[t.data_ptr() for t in ins])
    ch = np.ascontiguousarray(channels, np.int32)
    ia = np.ascontiguousarray(ialpha, np.float32)
    iz = np.ascontiguousarray(izp, np.uint8)
    N, H, W, _ = y.shape
    check(lib().hipq_concat_u8(ptrs, n, C.c_void_p(ch.ctypes.data), C.c_void_p(ia.ctypes.data), C.c_void_p(iz.ctypes.data),
                               _ptr(y), N * H * W, oalpha, ozp, obits, _stream()))
    return y


def softmax_u8(x, y, Cc, ialpha, izp, oalpha, ozp, obits=8):
    N, H, W, cs = x.shape
    check(lib().hipq_softmax_u8(_ptr(x), _ptr(y), N * H * W, Cc, cs, ialpha, izp, oalpha, ozp, obits, _stream()))
    return y


def pool_u8(x, y, Cc, kernel, pad, stride, method, ialpha, izp, oalpha, ozp, obits=8):
    N, H, W, cs = x.shape
    _, OH, OW, _ = y.shape
    (kh, kw) = (kernel, kernel) if np.isscalar(kernel) else kernel
    (ph, pw) = (pad, pad) if np.isscalar(pad) else pad
    (sh, sw) = (stride, stride) if np.isscalar(stride) else stride
    check(lib().hipq_pool_u8(_ptr(x), _ptr(y), N, Cc, H, W, OH, OW, cs, kh, kw, ph, pw, sh, sw, method, ialpha, izp,
                             oalpha, ozp, obits, _stream()))
    return y


def quantize_u8(x_nchw, y, oalpha, ozp, obits=8):
    N, Cc, H, W = x_nchw.shape
    check(lib().hipq_quantize_u8(_ptr(x_nchw), _ptr(y), N, Cc, H, W, y.shape[-1], oalpha, ozp, obits, _stream()))
    return y


def quantize_i8(x_nchw, y, oalpha, obits=8):
    N, Cc, H, W = x_nchw.shape
    check(lib().hipq_quantize_i8(_ptr(x_nchw), _ptr(y), N, Cc, H, W, y.shape[-1], oalpha, obits, _stream()))
    return y


def dequantize_i8(x, y_nchw, ialpha):
    N, Cc, H, W = y_nchw.shape
    check(lib().hipq_dequantize_i8(_ptr(x), _ptr(y_nchw), N, Cc, H, W, x.shape[-1], ialpha, _stream()))
    return y_nchw


def dequantize_i32(acc, y_nchw, alpha):
    """int32 accumulators NHWC -> fp32 NCHW: (float)acc * alpha (include/hipq.h: hipq_dequantize_i32)."""
    N, Cc, H, W = y_nchw.shape
    check(lib().hipq_dequantize_i32(_ptr(acc), _ptr(y_nchw), N, Cc, H, W, acc.shape[-1], float(np.float32(alpha)), _stream()))
    return y_nchw


def dequantize_u8(x, y_nchw, ialpha, izp):
    N, Cc, H, W = y_nchw.shape
    check(lib().hipq_dequantize_u8(_ptr(x), _ptr(y_nchw), N, Cc, H, W, x.shape[-1], ialpha, izp, _stream()))
    return y_nchw
