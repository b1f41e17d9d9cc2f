"""CPU-side checks of the C-ABI libraries: they load without a GPU, export every symbol their headers
declare, and their host-only entry points agree with the oracle.  No kernel is launched here."""
import os
import re

import numpy as np
import pytest

from nart_amd import hipq
from oracle import orc

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def declared_functions(header):
    text = open(os.path.join(ROOT, "include", header)).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return set(re.findall(r"\b(hipq_[a-z0-9_]+)\s*\(", text))


def test_hipq_exports_every_declared_symbol():
    L = hipq.lib()  # raises if the library is missing or lacks a symbol of hipq.EXPORTS
    declared = declared_functions("hipq.h")
    assert declared == set(hipq.EXPORTS), declared ^ set(hipq.EXPORTS)
    for name in declared:
        assert getattr(L, name) is not None
    assert L.hipq_abi_version() == 4


def test_quant_scale_matches_oracle():
    rng = np.random.default_rng(0)
    for bits in (16, 23, 24, 32):
        for _ in range(500):
            f = np.float32(np.exp(rng.uniform(np.log(1e-7), np.log(100.0))))
            assert hipq.quant_scale(f, bits) == orc.quant_scale(f, bits)
    assert hipq.quant_scale(0.0, 32) == (0, 0)


def test_channel_stride_rule():
    assert [hipq.channel_stride(c) for c in (1, 3, 4, 5, 16, 17, 24, 64, 1000)] == [4, 4, 4, 16, 16, 32, 32, 64, 1008]


def test_division_reciprocals_are_exact():
    """hipq_div_magic: the multiply-and-shift that replaces a division by a run-time constant inside the kernels equals
    the division for every dividend below 2^31 - checked at the dividends where a rounded-up reciprocal fails first (one
    below and exactly at multiples of the divisor), at the ends of the range and at random ones, for small divisors,
    powers of two and their neighbours, and large ones."""
    import ctypes
    rng = np.random.default_rng(5)
    ds = list(range(1, 700)) + [2 ** k + e for k in range(2, 31) for e in (-1, 0, 1)] + [int(v) for v in rng.integers(1, 2 ** 31 - 1, 300)]
    m, s = ctypes.c_uint32(), ctypes.c_int()
    for d in ds:
        assert hipq.lib().hipq_div_magic(d, ctypes.byref(m), ctypes.byref(s)) == 0
        q = np.unique(np.concatenate([np.arange(0, min(2 ** 31 // d + 1, 3000)), rng.integers(0, 2 ** 31 // d + 1, 3000)])).astype(np.uint64)
        x = np.concatenate([q * np.uint64(d), q * np.uint64(d) + np.uint64(d - 1), rng.integers(0, 2 ** 31, 3000).astype(np.uint64),
                            np.array([0, 1, 2 ** 31 - 1], np.uint64)])
        x = x[x < 2 ** 31]
        got = ((x * np.uint64(m.value)) >> np.uint64(32)) >> np.uint64(s.value) if m.value else x
        assert np.array_equal(got, x // np.uint64(d)), (d, m.value, s.value)
    assert hipq.lib().hipq_div_magic(0, ctypes.byref(m), ctypes.byref(s)) == -1


def test_ip_weight_reorder_host():
    rng = np.random.default_rng(1)
    No, C, H, W, cs = 5, 6, 2, 3, 16
    w = rng.integers(0, 256, (No, C, H, W), dtype=np.uint8)
    out = np.empty((No, H, W, cs), np.uint8)
    hipq.check(hipq.lib().hipq_ip_reorder_weights(w.ctypes.data, out.ctypes.data, No, C, H, W, cs, 77))
    assert np.array_equal(out[..., :C], w.transpose(0, 2, 3, 1)) and (out[..., C:] == 77).all()


def test_compute_entry_points_fail_loudly_without_gpu():
    try:
        import torch
        if torch.cuda.is_available():
            pytest.skip("a GPU is present")
    except ImportError:
        pass
    with pytest.raises(hipq.HipqError):
        hipq.Conv2d((1, 16, 4, 4), np.zeros((16, 16, 1, 1), np.uint8), None, 0, 1, 1, 0.1, 0, 0.1, 0, 0.1, 0)


def test_no_kernel_uses_scratch_memory():
    """The build records every kernel's register, LDS and scratch use (nart_amd/lib/kernel_resources.json) and refuses
    kernels with scratch memory; the record must be there and clean, and the MFMA tile kernels must fit the register
    budget their occupancy assumes."""
    import json
    path = os.path.join(ROOT, "nart_amd", "lib", "kernel_resources.json")
    assert os.path.exists(path), "run `python -m nart_amd.build` (it writes the record)"
    usage = json.load(open(path))
    assert len(usage) > 50
    assert all(v["scratch"] == 0 for v in usage.values())
    tiles = {k: v for k, v in usage.items() if "conv_mfma_dma_kernel" in k}
    assert tiles and all(v["vgprs"] <= 168 for v in tiles.values())  # three waves per SIMD at least
