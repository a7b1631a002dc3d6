"""Pins exl3o_hadamard128 (ponyexl3/ref/hadamard.py:50-80)."""
import numpy as np
import scipy.linalg

from conftest import rel_l2


def test_matches_dense_sylvester(oracle):
    rng = np.random.default_rng(0)
    x = rng.standard_normal((5, 384)).astype(np.float32)
    pre = np.where(rng.random(384) > 0.5, -1, 1).astype(np.float16)
    post = (rng.standard_normal(384) * 0.5).astype(np.float16)
    H = scipy.linalg.hadamard(128).astype(np.float64) / np.sqrt(128.0)
    ref = np.empty((5, 384))
    for j in range(0, 384, 128):
        blk = x[:, j : j + 128].astype(np.float64) * pre[j : j + 128].astype(np.float64)
        ref[:, j : j + 128] = (blk @ H) * post[j : j + 128].astype(np.float64)
    got = oracle.had_r_128(x, pre_scale=pre, post_scale=post)
    assert got.dtype == np.float32
    np.testing.assert_allclose(got, ref, rtol=2e-6, atol=2e-6)


def test_involution_and_parseval(oracle):
    rng = np.random.default_rng(1)
    x = rng.standard_normal((3, 256)).astype(np.float32)
    y = oracle.had_r_128(x)
    np.testing.assert_allclose(np.linalg.norm(y, axis=1), np.linalg.norm(x, axis=1), rtol=1e-6)
    assert rel_l2(oracle.had_r_128(y), x) < 1e-6


def test_unit_vectors_give_signed_rows(oracle):
    e = np.zeros((1, 128), dtype=np.float32)
    e[0, 5] = 1.0
    y = oracle.had_r_128(e)[0]
    H = scipy.linalg.hadamard(128)
    np.testing.assert_allclose(y, H[5] / np.sqrt(128.0), rtol=1e-7)


def test_rejects_bad_width(oracle):
    import pytest

    with pytest.raises(ValueError):
        oracle.had_r_128(np.zeros((1, 100), dtype=np.float32))
