"""The 64-bit accumulator words of the atomic split reductions (count << 56 | fixed-point
sum), compiled for the host: counts up to 255 contributors, negative sums, the clamp and
non-finite partial sums."""
import ctypes
import math
import os
import subprocess

import numpy as np
import pytest

HERE = os.path.dirname(os.path.abspath(__file__))
MASK = (1 << 64) - 1


@pytest.fixture(scope="module")
def shim(tmp_path_factory):
    so = str(tmp_path_factory.mktemp("fixpoint") / "fixpoint_shim.so")
    subprocess.run(["g++", "-O2", "-std=c++17", "-shared", "-fPIC", os.path.join(HERE, "fixpoint_shim.cpp"),
                    "-o", so], check=True)
    lib = ctypes.CDLL(so)
    lib.shim_fix_word.restype = ctypes.c_uint64
    lib.shim_fix_word.argtypes = [ctypes.c_float]
    lib.shim_fix_count.restype = ctypes.c_int
    lib.shim_fix_count.argtypes = [ctypes.c_uint64]
    lib.shim_fix_value.restype = ctypes.c_float
    lib.shim_fix_value.argtypes = [ctypes.c_uint64]
    return lib


def _accumulate(lib, values):
    w = 0
    for v in values:
        w = (w + lib.shim_fix_word(float(v))) & MASK  # what the 64-bit atomic add does
    return w


@pytest.mark.parametrize("n", [1, 2, 127, 128, 129, 200, 255])
@pytest.mark.parametrize("sign", [1.0, -1.0])
def test_count_and_sum_survive_up_to_255_contributors(shim, n, sign):
    rng = np.random.default_rng(n)
    vals = (sign * np.abs(rng.standard_normal(n)) * 300.0).astype(np.float32)
    w = _accumulate(shim, vals)
    assert shim.shim_fix_count(w) == n
    total = float(np.sum(vals.astype(np.float64)))
    assert abs(shim.shim_fix_value(w) - total) <= n * 2.0 ** -20 + abs(total) * 2.0 ** -23


def test_mixed_signs_cancel_exactly_on_grid_values(shim):
    vals = [1.5, -1.5, 1024.25, -1024.25, -0.125]
    w = _accumulate(shim, vals)
    assert shim.shim_fix_count(w) == 5 and shim.shim_fix_value(w) == -0.125
    # every intermediate count is visible to a lane that reads the word back
    w = 0
    for i, v in enumerate(vals):
        w = (w + shim.shim_fix_word(v)) & MASK
        assert shim.shim_fix_count(w) == i + 1


def test_order_independence(shim):
    rng = np.random.default_rng(3)
    vals = (rng.standard_normal(40) * 100).astype(np.float32)
    a = _accumulate(shim, vals)
    b = _accumulate(shim, vals[::-1])
    c = _accumulate(shim, rng.permutation(vals))
    assert a == b == c


def test_clamp_rounds_to_infinity_in_fp16(shim):
    w = _accumulate(shim, [1e9, 3.0])
    assert shim.shim_fix_count(w) == 2
    with np.errstate(over="ignore"):
        assert np.isinf(np.float16(shim.shim_fix_value(w)))
    w = _accumulate(shim, [-1e9] * 255)
    assert shim.shim_fix_count(w) == 255
    with np.errstate(over="ignore"):
        assert np.float16(shim.shim_fix_value(w)) == -np.inf


@pytest.mark.parametrize("bad", [math.nan, math.inf, -math.inf])
@pytest.mark.parametrize("n_bad,n_ok", [(1, 0), (1, 254), (255, 0), (3, 100)])
def test_non_finite_partial_sums_poison_the_total(shim, bad, n_bad, n_ok):
    vals = [bad] * n_bad + [-262144.0] * n_ok  # the most negative legitimate partial sums
    w = _accumulate(shim, vals)
    assert shim.shim_fix_count(w) == n_bad + n_ok
    assert math.isnan(shim.shim_fix_value(w))


def test_preseeded_count_never_completes(shim):
    """A word that starts with count 255 ends one short of the number of contributors:
    what the GPU test of the bounded wait relies on."""
    w = 0xFF << 56
    for _ in range(5):
        w = (w + shim.shim_fix_word(1.0)) & MASK
    assert shim.shim_fix_count(w) == 4
