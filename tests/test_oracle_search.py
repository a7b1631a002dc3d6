"""The oracle's two trellis searches (encoder side), pinned without the reference:
brute force over every path of a short trellis, the tail-biting closure, recovery
of exactly representable tiles, the pack -> unpack round trip of the found states
and the quality bound between the two searches -- the assertions of the
reference's own tests/test_convert_metal.py:25-86."""
import math

import numpy as np
import pytest

MCG, DEFAULT, MUL1 = 1, 0, 2


def _tail_biting(states, k):
    return (int(states[0]) >> k) == (int(states[-1]) & ((1 << (16 - k)) - 1))


def _chain_valid(states, k):
    """Every state is its predecessor shifted by K with fresh low bits."""
    s = states.astype(np.uint32)
    return bool(np.all((s[1:] >> k) == (s[:-1] & ((1 << (16 - k)) - 1))))


def valid_tail_biting_indices(k, seed):
    """A random closed path: every 16-bit state is the last 16 bits of the circular
    stream of K-bit symbols (same construction as the reference's test helper)."""
    rng = np.random.default_rng(seed)
    fresh = rng.integers(0, 1 << k, size=256, dtype=np.uint32)
    out = np.zeros(256, dtype=np.uint32)
    for i in range(256):
        x = 0
        for shift in range(int(math.ceil(16 / k))):
            x |= int(fresh[(i - shift) % 256]) << (k * shift)
        out[i] = x & 0xFFFF
    return out.astype(np.uint16)


@pytest.mark.parametrize("k,cb", [(4, MCG), (4, DEFAULT), (3, MUL1)])
def test_free_pass_is_the_optimum_over_all_open_paths(oracle, k, cb):
    """Two steps: the start state (16 bits) and two fresh symbols enumerate every
    open path; the free Viterbi pass must find the cheapest one."""
    lut = oracle.decode_table(cb).astype(np.float32).astype(np.float64)
    rng = np.random.default_rng(7 + k + cb)
    w = (rng.standard_normal(2) * 1.2).astype(np.float32)
    s0 = np.arange(65536, dtype=np.uint32)
    best = np.inf
    for f1 in range(1 << k):
        s1 = ((s0 << k) | f1) & 0xFFFF
        c1 = (lut[s1] - float(w[0])) ** 2
        for f2 in range(1 << k):
            s2 = ((s1 << k) | f2) & 0xFFFF
            best = min(best, float((c1 + (lut[s2] - float(w[1])) ** 2).min()))
    states, decoded = oracle.quantize_tile_exact(w, k, cb, max_pins=0)
    assert _chain_valid(states, k)
    got = float(((decoded.astype(np.float64) - w.astype(np.float64)) ** 2).sum())
    assert got == pytest.approx(best, rel=1e-12, abs=1e-15)
    np.testing.assert_array_equal(decoded, lut[states].astype(np.float32))


@pytest.mark.parametrize("seed", [0, 1, 2])
def test_pinned_passes_cannot_beat_the_closed_optimum(oracle, seed):
    """Five steps at K=4: 2^20 closed paths, brute-forced. The pinning scheme does
    not force the last state, so on so short a trellis it may stop unclosed; when it
    does close, its path is one of the enumerated ones."""
    k, n = 4, 5
    lut = oracle.decode_table(MCG).astype(np.float32).astype(np.float64)
    rng = np.random.default_rng(seed)
    w = (rng.standard_normal(n) * 1.2).astype(np.float32)
    seq = np.arange(1 << (k * n), dtype=np.uint32)
    sym = [(seq >> (k * i)) & 15 for i in range(n)]  # symbol appended at step i
    total = np.zeros(seq.size)
    for t in range(n):
        st = np.zeros(seq.size, dtype=np.uint32)
        for back in range(4):  # 16 bits = 4 symbols, newest lowest
            st |= sym[(t - back) % n] << (k * back)
        total += (lut[st] - float(w[t])) ** 2
    opt = float(total.min())
    states, decoded = oracle.quantize_tile_exact(w, k, MCG, max_pins=4)
    assert _chain_valid(states, k)
    got = float(((decoded.astype(np.float64) - w.astype(np.float64)) ** 2).sum())
    if _tail_biting(states, k):
        assert got >= opt - 1e-12
    free_states, free_dec = oracle.quantize_tile_exact(w, k, MCG, max_pins=0)
    free = float(((free_dec.astype(np.float64) - w.astype(np.float64)) ** 2).sum())
    assert free <= opt + 1e-12 and free <= got + 1e-12  # fewer constraints, never worse


@pytest.mark.parametrize("k", [2, 3, 4, 5, 8])
def test_production_search_recovers_an_exactly_representable_tile(oracle, k):
    encoded = valid_tail_biting_indices(k, seed=k)
    assert _tail_biting(encoded, k) and _chain_valid(encoded, k)
    decoded = oracle.decode_table(MCG)[encoded].astype(np.float32).reshape(1, 256)
    q, states = oracle.quantize_tiles_search(decoded, k, MCG)
    assert _tail_biting(states[0], k)
    np.testing.assert_array_equal(states[0], encoded)
    np.testing.assert_array_equal(q[0], decoded[0])


@pytest.mark.parametrize("k", [2, 3, 4])
def test_exact_search_recovers_an_exactly_representable_tile(oracle, k):
    encoded = valid_tail_biting_indices(k, seed=40 + k)
    decoded = oracle.decode_table(MCG)[encoded].astype(np.float32)
    states, q = oracle.quantize_tile_exact(decoded, k, MCG)
    np.testing.assert_array_equal(states, encoded)
    np.testing.assert_array_equal(q, decoded)


@pytest.mark.parametrize("k,cb", [(2, MCG), (3, MCG), (4, DEFAULT), (4, MCG), (4, MUL1)])
def test_production_search_quality_against_the_exact_search(oracle, k, cb):
    """Same seeds, scale and bound as tests/test_convert_metal.py:44-71."""
    scale = 1.0 if cb == MUL1 else 1.24371088
    rng = np.random.default_rng(100 + 10 * k + cb)
    tile = (rng.standard_normal((1, 256)) * scale).astype(np.float32)
    q, states = oracle.quantize_tiles_search(tile, k, cb)
    ref_states, ref_tile = oracle.quantize_tile_exact(tile[0], k, cb)
    assert _tail_biting(states[0], k) and _chain_valid(states[0], k)
    # the exact search stops after four pinned passes whether or not the path has
    # closed (reference_search.py:77-84), so only its chain is checked
    assert _chain_valid(ref_states, k)
    packed = oracle.pack_tile((states[0] & ((1 << k) - 1)).astype(np.uint16), k)
    np.testing.assert_array_equal(oracle.unpack_tile(packed, k), states[0])
    np.testing.assert_array_equal(q[0], oracle.decode_table(cb)[states[0]].astype(np.float32))
    mse = float(np.mean((q[0] - tile[0]) ** 2))
    ref_mse = float(np.mean((ref_tile - tile[0]) ** 2))
    assert mse <= ref_mse * 1.10
    # K bits per weight buy roughly 6 dB each: a sanity bound on both searches
    assert ref_mse < 1.6 * scale * scale * 4.0 ** -k * 3.0


def test_search_argument_errors(oracle):
    tile = np.zeros((1, 256), dtype=np.float32)
    with pytest.raises(ValueError, match=r"supports K in \[2, 8\]"):
        oracle.quantize_tiles_search(tile, 1, MCG)
    with pytest.raises(ValueError):
        oracle.quantize_tiles_search(np.zeros((2, 100), dtype=np.float32), 4, MCG)
    q, idx = oracle.quantize_tiles_search(np.zeros((3, 256), dtype=np.float32), 4, DEFAULT)
    assert q.shape == (3, 256) and idx.shape == (3, 256)
    assert (idx[0] == idx[1]).all() and (idx[1] == idx[2]).all()


@pytest.mark.parametrize("k,cb", [(2, MCG), (3, MCG), (4, DEFAULT), (4, MCG), (4, MUL1), (5, MCG)])
def test_exact_search_equals_reference_vectors(oracle, k, cb):
    """States and decoded values written by the reference's quantize_tile_reference
    (tests/golden/make_golden_search.py): same path bit for bit, including the
    closing passes and the tie-breaking."""
    from conftest import golden

    g = golden("search_exact.npz")
    tag = f"k{k}_cb{cb}"
    states, decoded = oracle.quantize_tile_exact(g[tag + "_tile"], k, cb)
    np.testing.assert_array_equal(states, g[tag + "_states"])
    np.testing.assert_array_equal(decoded.view(np.uint32), g[tag + "_decoded"].view(np.uint32))
