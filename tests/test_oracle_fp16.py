"""The oracle's software fp16 conversions against numpy's IEEE conversions."""
import ctypes

import numpy as np


def test_half_to_float_exhaustive(oracle):
    h = np.arange(65536, dtype=np.uint16)
    f = np.empty(65536, dtype=np.float32)
    oracle.lib().exl3o_half_to_float(
        h.ctypes.data_as(ctypes.POINTER(ctypes.c_uint16)),
        f.ctypes.data_as(ctypes.POINTER(ctypes.c_float)), 65536)
    ref = h.view(np.float16).astype(np.float32)
    np.testing.assert_array_equal(f.view(np.uint32)[~np.isnan(ref)], ref.view(np.uint32)[~np.isnan(ref)])
    assert np.isnan(f[np.isnan(ref)]).all()


def test_float_to_half_rounding(oracle):
    rng = np.random.default_rng(0)
    # random floats across the half range, plus every midpoint between adjacent halves
    f = (rng.standard_normal(200000) * np.exp(rng.uniform(-18, 11, 200000))).astype(np.float32)
    h = np.arange(0, 0x7BFF, dtype=np.uint16)
    mid = (h.view(np.float16).astype(np.float64) + (h + 1).view(np.float16).astype(np.float64)) / 2
    f = np.concatenate([f, mid.astype(np.float32), -mid.astype(np.float32),
                        np.array([0.0, -0.0, 65504.0, 65519.9, 65520.0, 1e9, -1e9, 6e-8, 2.9e-8, 3.0e-8],
                                 dtype=np.float32)])
    out = np.empty(f.size, dtype=np.uint16)
    oracle.lib().exl3o_float_to_half(
        f.ctypes.data_as(ctypes.POINTER(ctypes.c_float)),
        out.ctypes.data_as(ctypes.POINTER(ctypes.c_uint16)), f.size)
    with np.errstate(over="ignore"):
        ref = f.astype(np.float16).view(np.uint16)
    np.testing.assert_array_equal(out, ref)


def test_double_to_half_single_rounding(oracle):
    # values where float32-then-half would double round: half midpoint + tiny epsilon
    h = np.arange(0x3C00, 0x4000, dtype=np.uint16)
    a = h.view(np.float16).astype(np.float64)
    b = (h + 1).view(np.float16).astype(np.float64)
    d = (a + b) / 2 + 1e-12
    out = np.empty(d.size, dtype=np.uint16)
    oracle.lib().exl3o_double_to_half(
        d.ctypes.data_as(ctypes.POINTER(ctypes.c_double)),
        out.ctypes.data_as(ctypes.POINTER(ctypes.c_uint16)), d.size)
    np.testing.assert_array_equal(out, h + 1)
