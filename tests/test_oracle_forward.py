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


def test_geglu_closed_form(oracle):
    """GeGLU = u * 0.5 g (1 + tanh(sqrt(2/pi) (g + 0.044715 g^3))), the tanh form of
    ponyexl3/mlx/exl3_moe.py:62-75, evaluated here in float64 at fixed points and on a
    grid; the oracle's fp32 evaluation rounded to fp16 must agree to an fp16 ulp. A
    wrong constant (0.044715, sqrt(2/pi), the 0.5) moves the values by far more."""
    g = np.array([-6.0, -3.0, -1.5, -0.75, -0.1, 0.0, 0.1, 0.5, 1.0, 2.0, 4.0], dtype=np.float16)
    u = np.array([1.0, -2.0, 0.5, 3.0, -1.0, 7.0, 1.0, -0.25, 2.0, 1.5, -1.0], dtype=np.float16)
    g64, u64 = g.astype(np.float64), u.astype(np.float64)
    want = 0.5 * g64 * (1.0 + np.tanh(np.sqrt(2.0 / np.pi) * (g64 + 0.044715 * g64**3))) * u64
    got = oracle.glu(g, u, "gelu").astype(np.float64)
    np.testing.assert_allclose(got, want, rtol=1.0 / 1024, atol=1e-4)
    # known values of gelu_tanh: gelu(1) = 0.841192, gelu(-1) = -0.158808, gelu(2) = 1.954598
    one = np.ones(3, dtype=np.float16)
    k = oracle.glu(np.array([1.0, -1.0, 2.0], dtype=np.float16), one, "gelu").astype(np.float64)
    np.testing.assert_allclose(k, [0.841192, -0.158808, 1.954598], atol=1e-3)
    grid = np.linspace(-8, 8, 4001).astype(np.float16)
    g64 = grid.astype(np.float64)
    want = 0.5 * g64 * (1.0 + np.tanh(np.sqrt(2.0 / np.pi) * (g64 + 0.044715 * g64**3)))
    got = oracle.glu(grid, np.ones_like(grid), "gelu").astype(np.float64)
    np.testing.assert_allclose(got, want, rtol=1.0 / 1024, atol=1e-4)


def _expert(rng, k, n_in, n_out):
    tr = rng.integers(0, 65536, size=(n_in // 16, n_out // 16, 16 * k), dtype=np.uint16)
    suh = (np.where(rng.random(n_in) > 0.5, -1, 1) * rng.uniform(0.5, 1.5, n_in)).astype(np.float16)
    svh = (np.where(rng.random(n_out) > 0.5, -1, 1) * rng.uniform(0.5, 1.5, n_out)).astype(np.float16)
    return tr, suh, svh


@pytest.mark.parametrize("activation", ["silu", "gelu"])
def test_moe_chain_against_public_weight_composition(oracle, activation):
    """The oracle's expert chain (ponyexl3/mlx/exl3_moe.py:648-682) against a
    composition written another way: every expert's three projections folded into
    dense public weights diag(suh) H W H diag(svh) (ponyexl3/ref/reconstruct.py:26-49)
    and applied as plain float64 matrix products, y = (act(x Wg) * (x Wu)) Wd. The two
    routes round at different points (the chain hands fp16 between its linears), so
    they agree to a few fp16 ulps; picking the wrong expert, swapping gate and up or
    dropping the activation is off by order one."""
    rng = np.random.default_rng(2024)
    k, cb, E, D, H, T, kk = 4, 1, 5, 256, 128, 3, 2
    experts = [{"gate": _expert(rng, k, D, H), "up": _expert(rng, k, D, H), "down": _expert(rng, k, H, D)}
               for _ in range(E)]
    x = (rng.standard_normal((T, D)) * 0.05).astype(np.float16)
    indices = np.array([[4, 1], [0, 3], [2, 2]], dtype=np.int32)
    got = oracle.moe_experts_forward(experts, x, indices, k, cb, activation=activation).astype(np.float64)
    assert got.shape == (T, kk, D)

    pub = [{n: oracle.reconstruct_public_weights(e[n][0], e[n][1], e[n][2], k, cb).astype(np.float64)
            for n in ("gate", "up", "down")} for e in experts]

    def act(g):
        if activation == "silu":
            return g / (1.0 + np.exp(-g))
        return 0.5 * g * (1.0 + np.tanh(np.sqrt(2.0 / np.pi) * (g + 0.044715 * g**3)))

    def dense(t, e, swap=False, no_act=False):
        xt = x[t].astype(np.float64)
        g, u = xt @ pub[e]["gate"], xt @ pub[e]["up"]
        if swap:
            g, u = u, g
        return ((g if no_act else act(g)) * u) @ pub[e]["down"]

    for t in range(T):
        for s in range(kk):
            e = int(indices[t, s])
            want = dense(t, e)
            assert rel_l2(got[t, s], want) < 4e-3, (t, s)
            assert rel_l2(got[t, s], dense(t, (e + 1) % E)) > 0.5      # another expert
            assert rel_l2(got[t, s], dense(t, e, swap=True)) > 0.3     # gate and up exchanged
            assert rel_l2(got[t, s], dense(t, e, no_act=True)) > 0.3   # activation dropped
    # the intermediate is handed over as fp16: the chain equals itself with that cast
    # made explicit, bit for bit
    e = experts[4]
    g = oracle.linear_forward(e["gate"][0], k, cb, e["gate"][1], e["gate"][2], x[:1])
    u = oracle.linear_forward(e["up"][0], k, cb, e["up"][1], e["up"][2], x[:1])
    h = oracle.glu(g, u, activation)
    assert h.dtype == np.float16
    y = oracle.linear_forward(e["down"][0], k, cb, e["down"][1], e["down"][2], h)
    np.testing.assert_array_equal(y[0].view(np.uint16),
                                  oracle.moe_experts_forward(experts, x[:1], indices[:1, :1], k, cb,
                                                             activation=activation)[0, 0].view(np.uint16))
