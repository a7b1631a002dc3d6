"""Pins exl3o_linear_forward (ponyexl3/ref/forward.py:14-49) against outputs
written by the reference, and against the public-weight identity."""
import numpy as np
import pytest

from conftest import golden, rel_l2

# The reference sums the Hadamard and the matmul in fp32 BLAS order, the oracle
# in double; after the fp16 casts that is at most an ulp on a few elements.
TOL = 1e-3


def _cases():
    g = golden("forwards.npz")
    return sorted({n[:-2] for n in g.files if n.endswith("_y")})


@pytest.mark.parametrize("tag", _cases())
def test_golden_forward(oracle, tag):
    g = golden("forwards.npz")
    k = int(tag[1])
    cb = int(tag.split("_")[1][2])
    suh, svh = g[tag + "_suh"], g[tag + "_svh"]
    if not tag.endswith("_bf"):
        suh, svh = suh.view(np.float16), svh.view(np.float16)
    bias = g[tag + "_bias"].view(np.float16) if tag + "_bias" in g.files else None
    y = oracle.linear_forward(g[tag + "_trellis"], k, cb, suh, svh, g[tag + "_x"].view(np.float16), bias=bias)
    ref = g[tag + "_y"].view(np.float16)
    assert y.shape == ref.shape
    assert rel_l2(y, ref) <= TOL
    d = np.abs(y.astype(np.float64) - ref.astype(np.float64)).max()
    assert d <= 2e-3 * np.abs(ref.astype(np.float64)).max()


def test_public_weights_match_reference(oracle):
    g = golden("forwards.npz")
    w = oracle.reconstruct_public_weights(g["pub_trellis"], g["pub_suh"].view(np.float16),
                                          g["pub_svh"].view(np.float16), 4, 0)
    ref = g["pub_w"].view(np.float16)
    assert rel_l2(w, ref) < 1e-3
    assert (w.view(np.uint16) != ref.view(np.uint16)).mean() < 0.02


def test_inner_path_matches_public_weight_path(oracle):
    """tests/test_decode_reconstruct.py:40-69: x @ W_pub ~= had(had(x*suh) @ W)*svh."""
    rng = np.random.default_rng(7)
    tr = rng.integers(0, 65536, size=(8, 8, 48), dtype=np.uint16)
    suh = np.where(rng.random(128) > 0.5, -1, 1).astype(np.float16)
    svh = np.where(rng.random(128) > 0.5, -1, 1).astype(np.float16)
    x = rng.standard_normal((2, 128)).astype(np.float16)
    y = oracle.linear_forward(tr, 3, 0, suh, svh, x)
    w_pub = oracle.reconstruct_public_weights(tr, suh, svh, 3, 0)
    y2 = x.astype(np.float32) @ w_pub.astype(np.float32)
    assert rel_l2(y, y2) < 5e-3


def test_forward_is_plain_gemm_of_decoded_weights(oracle):
    rng = np.random.default_rng(11)
    tr = rng.integers(0, 65536, size=(16, 8, 64), dtype=np.uint16)
    x = rng.standard_normal((4, 256)).astype(np.float16)
    y, xh, yraw = oracle.linear_forward(tr, 4, 1, None, None, x, taps=True)
    w = oracle.decode_trellis(tr, 4, 1).astype(np.float64)
    ref = xh.astype(np.float64) @ w
    assert rel_l2(yraw, ref) < 5e-4
    assert rel_l2(xh, oracle.had_r_128(x.astype(np.float32))) < 5e-4


def test_bs1_streaming_variant_equals_forward(oracle):
    rng = np.random.default_rng(12)
    tr = rng.integers(0, 65536, size=(16, 24, 80), dtype=np.uint16)
    suh = np.where(rng.random(256) > 0.5, -1, 1).astype(np.float16)
    svh = np.where(rng.random(384) > 0.5, -1, 1).astype(np.float16)
    x = rng.standard_normal(256).astype(np.float16)
    a = oracle.linear_forward(tr, 5, 0, suh, svh, x[None])[0]
    b = oracle.linear_forward_bs1(tr, 5, 0, suh, svh, x)
    assert rel_l2(b, a) < 2e-4


def test_shape_errors(oracle):
    tr = np.zeros((2, 8, 64), dtype=np.uint16)  # in = 32: not a multiple of 128
    with pytest.raises(ValueError):
        oracle.linear_forward(tr, 4, 0, None, None, np.zeros((1, 32), dtype=np.float16))


def test_glu_reference_values(oracle):
    g = np.array([-2.0, -0.5, 0.0, 1.0, 3.0], dtype=np.float16)
    u = np.array([0.25, 1.0, -1.0, 2.0, 0.5], dtype=np.float16)
    silu = g.astype(np.float64) / (1 + np.exp(-g.astype(np.float64))) * u.astype(np.float64)
    np.testing.assert_allclose(oracle.glu(g, u, "silu").astype(np.float64), silu, atol=1e-3)
    assert not np.allclose(oracle.glu(g, u, "gelu"), oracle.glu(g, u, "silu"))
