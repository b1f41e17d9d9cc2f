"""Synthetic quantized cases (graphs + seeded weights + per-layer quantisation parameters).

A case is what the reference's converter would hand to the runtime for a quantized network: a flat,
topologically ordered list of quant-module operators (quantize, conv_2d, pool, add, ip, dequantize —
art/modules/quant/src/quant_module.c:49-89) with SETTING_QUANT_* parameters per operator.  The shapes
follow BASELINE.json's configurations; weights are random-init from a seed (there are no checkpoints).

Conventions (reference semantics, see conv_2d_uint8_impl.c / add.c):
  * int8-symmetric weights are stored as uint8 with wzp = 128;
  * a ReLU after a conv or add is expressed the reference's implicit way where the graph allows it:
    output zero point 0, so the saturation at 0 is the ReLU; where activations carry random zero points
    (MobileNetV2 case) the conv carries relu=True, which means "followed by a quant relu op with equal
    scales and zero point";
  * biases are int32 in units of ialpha*walpha.
Output scales are chosen from the fan-in so that activations neither collapse nor saturate, then
jittered by the seed.
"""
import math

import numpy as np


class Tensor:
    def __init__(self, name, shape, alpha=None, zp=None, dtype="u8"):
        self.name, self.shape, self.alpha, self.zp, self.dtype = name, tuple(shape), alpha, zp, dtype


class Node:
    def __init__(self, kind, inputs, output, **attrs):
        self.kind, self.inputs, self.output, self.attrs = kind, list(inputs), output, attrs


class Case:
    def __init__(self, name, seed):
        self.name = name
        self.rng = np.random.default_rng(seed)
        self.tensors, self.nodes, self.weights = {}, [], {}
        self.input = self.output = None
        self._n = 0

    # -- helpers -----------------------------------------------------------------------------------
    def _t(self, prefix, shape, alpha=None, zp=None, dtype="u8"):
        self._n += 1
        t = Tensor("%s_%d" % (prefix, self._n), shape, alpha, zp, dtype)
        self.tensors[t.name] = t
        return t

    def _jitter(self, lo=0.75, hi=1.35):
        return float(self.rng.uniform(lo, hi))

    def input_f32(self, shape):
        self.input = self._t("input", shape, dtype="f32")
        return self.input

    def input_u8(self, shape, alpha, zp):
        self.input = self._t("input", shape, alpha, zp)
        return self.input

    def quantize(self, x, alpha, zp):
        y = self._t("q", x.shape, alpha, zp)
        self.nodes.append(Node("quantize", [x.name], y.name))
        return y

    def dequantize(self, x):
        y = self._t("dq", x.shape, dtype="f32")
        self.nodes.append(Node("dequantize", [x.name], y.name))
        self.output = y
        return y

    def conv(self, x, K, k, stride=1, pad=None, group=1, relu=False, ozp=None, wzp=128, w_lo=1, w_hi=255,
             implicit_relu=False):
        """implicit_relu: ozp = 0 (the clamp at 0 is the ReLU).  relu: explicit fused flag."""
        N, C, H, W = x.shape
        pad = k // 2 if pad is None else pad
        OH, OW = (H + 2 * pad - k) // stride + 1, (W + 2 * pad - k) // stride + 1
        cg = C // group
        w = self.rng.integers(w_lo, w_hi + 1, (K, cg, k, k), dtype=np.uint8)
        fan = cg * k * k
        # accumulator spread: uniform bytes around their zero points have sigma ~ 74
        acc_sigma = 74.0 * 74.0 * math.sqrt(fan)
        bias = self.rng.integers(-int(acc_sigma), int(acc_sigma) + 1, K).astype(np.int32)
        if implicit_relu:
            ozp = 0
        elif ozp is None:
            ozp = int(self.rng.integers(96, 160))
        target = 48.0 if (implicit_relu or relu) else 36.0  # output sigma in LSB
        # keep the activation scale of the same order from layer to layer (seeded jitter) and derive
        # the weight scale from it, so that ialpha*walpha/oalpha maps the accumulator spread to `target`
        oalpha = float(np.float32(x.alpha * self._jitter()))
        walpha = float(np.float32(oalpha * target / (x.alpha * acc_sigma)))
        y = self._t("conv", (N, K, OH, OW), oalpha, ozp)
        wn, bn = y.name + ".w", y.name + ".b"
        self.weights[wn], self.weights[bn] = w, bias
        self.nodes.append(Node("conv", [x.name], y.name, w=wn, b=bn, K=K, k=k, stride=stride, pad=pad, group=group,
                               relu=bool(relu), walpha=walpha, wzp=wzp))
        return y

    def pool(self, x, k, stride, pad, method, ceil_mode, alpha=None, zp=None):
        N, C, H, W = x.shape

        def od(i):
            v = (i + 2 * pad - k) / stride + 1
            o = math.ceil(v) if ceil_mode else math.floor(v)
            if pad and (o - 1) * stride >= i + pad:
                o -= 1
            return o
        y = self._t("pool", (N, C, od(H), od(W)), x.alpha if alpha is None else alpha, x.zp if zp is None else zp)
        self.nodes.append(Node("pool", [x.name], y.name, k=k, stride=stride, pad=pad, method=method, ceil_mode=ceil_mode))
        return y

    def add(self, a, b, implicit_relu=True, ozp=None):
        oalpha = float(np.float32(math.hypot(a.alpha, b.alpha) * 1.1 * self._jitter(0.9, 1.2)))
        if implicit_relu:
            ozp = 0
        elif ozp is None:
            ozp = int(self.rng.integers(96, 160))
        y = self._t("add", a.shape, oalpha, ozp)
        self.nodes.append(Node("add", [a.name, b.name], y.name))
        return y

    def ip(self, x, Nout, ozp=None):
        N = x.shape[0]
        Kd = int(np.prod(x.shape[1:]))
        w = self.rng.integers(0, 256, (Nout, Kd), dtype=np.uint8)
        walpha = float(np.float32(math.exp(self.rng.uniform(math.log(1e-3), math.log(1e-1)))))
        acc_sigma = 74.0 * 74.0 * math.sqrt(Kd)
        bias = self.rng.integers(-int(acc_sigma), int(acc_sigma) + 1, Nout).astype(np.int32)
        oalpha = float(np.float32(x.alpha * walpha * acc_sigma / 36.0 * self._jitter()))
        y = self._t("ip", (N, Nout, 1, 1), oalpha, int(self.rng.integers(96, 160)) if ozp is None else ozp)
        wn, bn = y.name + ".w", y.name + ".b"
        self.weights[wn], self.weights[bn] = w, bias
        self.nodes.append(Node("ip", [x.name], y.name, w=wn, b=bn, K=Nout, walpha=walpha, wzp=128))
        return y

    # -- accounting --------------------------------------------------------------------------------
    def conv_ops(self):
        """Algorithmic integer ops of the contractions: 2*N*K*OH*OW*(C/g)*R*S per conv, 2*M*K*N per ip."""
        total = 0
        for n in self.nodes:
            y = self.tensors[n.output]
            if n.kind == "conv":
                x = self.tensors[n.inputs[0]]
                total += 2 * int(np.prod(y.shape)) * (x.shape[1] // n.attrs["group"]) * n.attrs["k"] ** 2
            elif n.kind == "ip":
                x = self.tensors[n.inputs[0]]
                total += 2 * int(np.prod(y.shape)) * int(np.prod(x.shape[1:]))
        return total


# ---- the BASELINE configurations ---------------------------------------------------------------------
def single_conv(N=1, seed=1):
    """configs[0]: 3x3/s1/p1 conv 64->64 at 56x56, izp 128 / 0.02, wzp 128 / 0.005, out 0.05 / zp 0."""
    c = Case("conv3x3_64_56_n%d" % N, seed)
    x = c.input_u8((N, 64, 56, 56), 0.02, 128)
    w = (c.rng.integers(-127, 128, (64, 64, 3, 3)) + 128).astype(np.uint8)
    b = c.rng.integers(-1000, 1001, 64).astype(np.int32)
    y = c._t("conv", (N, 64, 56, 56), 0.05, 0)
    c.weights[y.name + ".w"], c.weights[y.name + ".b"] = w, b
    c.nodes.append(Node("conv", [x.name], y.name, w=y.name + ".w", b=y.name + ".b", K=64, k=3, stride=1, pad=1, group=1,
                        relu=False, walpha=0.005, wzp=128))
    c.output = y
    return c


def single_fc(M=128, K=4096, Nout=4096, seed=2):
    """configs[1]: FC M x K x Nout, activations zp 128, int8-symmetric weights, log-uniform scales."""
    c = Case("fc_%dx%dx%d" % (M, K, Nout), seed)
    ia = float(np.float32(math.exp(c.rng.uniform(math.log(1e-3), math.log(1e-1)))))
    x = c.input_u8((M, K, 1, 1), ia, 128)
    c.output = c.ip(x, Nout)
    return c


def _bottleneck(c, x, width, stride, downsample):
    y = c.conv(x, width, 1, implicit_relu=True)
    y = c.conv(y, width, 3, stride=stride, implicit_relu=True)
    y = c.conv(y, width * 4, 1)
    sc = c.conv(x, width * 4, 1, stride=stride, pad=0) if downsample else x
    return c.add(y, sc, implicit_relu=True)


def resnet50(N=64, seed=50, hw=224, with_quantize=True):
    """configs[4]: ResNet-50-shaped (v1.5: stride on the 3x3), bottlenecks [3,4,6,3], FC 2048->1000,
    explicit quantize (fp32 -> uint8) and dequantize (uint8 -> fp32) at the graph ends."""
    c = Case("resnet50_n%d" % N, seed)
    if with_quantize:
        x = c.quantize(c.input_f32((N, 3, hw, hw)), 0.0186, int(c.rng.integers(100, 140)))
    else:
        x = c.input_u8((N, 3, hw, hw), 0.0186, 114)
    x = c.conv(x, 64, 7, stride=2, pad=3, implicit_relu=True)
    x = c.pool(x, 3, 2, 1, 0, False)
    for width, blocks, stride in ((64, 3, 1), (128, 4, 2), (256, 6, 2), (512, 3, 2)):
        for b in range(blocks):
            x = _bottleneck(c, x, width, stride if b == 0 else 1, b == 0)
    x = c.pool(x, x.shape[2], 1, 0, 1, True)
    x = c.ip(x, 1000)
    if with_quantize:
        c.dequantize(x)
    else:
        c.output = x
    return c


def resnet18(N=1, seed=18, hw=224):
    """configs[2]: 7x7/s2 stem, 4 stages of 2 basic blocks (64..512), 1x1/s2 downsample, FC 512->1000."""
    c = Case("resnet18_n%d" % N, seed)
    x = c.input_u8((N, 3, hw, hw), 0.0186, 114)
    x = c.conv(x, 64, 7, stride=2, pad=3, implicit_relu=True)
    x = c.pool(x, 3, 2, 1, 0, False)
    for width, stride in ((64, 1), (128, 2), (256, 2), (512, 2)):
        for b in range(2):
            s = stride if b == 0 else 1
            y = c.conv(x, width, 3, stride=s, implicit_relu=True)
            y = c.conv(y, width, 3)
            sc = c.conv(x, width, 1, stride=s, pad=0) if (b == 0 and (s != 1 or x.shape[1] != width)) else x
            x = c.add(y, sc, implicit_relu=True)
    x = c.pool(x, x.shape[2], 1, 0, 1, True)
    c.output = c.ip(x, 1000)
    return c


def mobilenet_v2(N=64, seed=22, hw=224):
    """configs[3]: inverted residuals (expansion 6: 1x1 expand, 3x3 depthwise, 1x1 project), widths 16..320,
    quantized residual adds, random activation zero points (ReLU as an explicit fused flag)."""
    c = Case("mobilenetv2_n%d" % N, seed)
    rz = lambda: int(c.rng.integers(0, 256))  # noqa: E731
    x = c.input_u8((N, 3, hw, hw), 0.0186, rz())
    x = c.conv(x, 32, 3, stride=2, relu=True, ozp=int(c.rng.integers(0, 64)))
    cin = 32
    for t, cout, n, s in ((1, 16, 1, 1), (6, 24, 2, 2), (6, 32, 3, 2), (6, 64, 4, 2), (6, 96, 3, 1), (6, 160, 3, 2),
                          (6, 320, 1, 1)):
        for i in range(n):
            stride = s if i == 0 else 1
            y = x
            if t != 1:
                y = c.conv(y, cin * t, 1, relu=True, ozp=int(c.rng.integers(0, 64)))
            y = c.conv(y, y.shape[1], 3, stride=stride, group=y.shape[1], relu=True, ozp=int(c.rng.integers(0, 64)))
            y = c.conv(y, cout, 1, ozp=rz())
            x = c.add(x, y, implicit_relu=False, ozp=rz()) if (stride == 1 and cin == cout) else y
            cin = cout
    x = c.conv(x, 1280, 1, relu=True, ozp=int(c.rng.integers(0, 64)))
    x = c.pool(x, x.shape[2], 1, 0, 1, True)
    c.output = c.ip(x, 1000)
    return c
