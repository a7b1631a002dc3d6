"""Pins oracle.exl3o_unpack_tile / exl3o_pack_tile (ponyexl3/ref/trellis.py)."""
import numpy as np
import pytest

from conftest import golden

KS = [1, 2, 3, 4, 5, 6, 7, 8]


def sliding_window_states(packed, k):
    """Independent statement of the format (tests/test_trellis.py:9-22 and
    ref/trellis.py:179-202): undo the uint16 swap inside each uint32, read the
    words as one MSB-first bit string, and run state = ((state << K) | fresh)
    & 0xFFFF for two laps."""
    w = packed.astype(np.uint16).reshape(-1, 2)[:, ::-1].reshape(-1)
    bits = ((w[:, None] >> np.arange(15, -1, -1)) & 1).reshape(-1)
    fresh = bits.reshape(256, k)
    fresh = (fresh * (1 << np.arange(k - 1, -1, -1))).sum(axis=1)
    states = np.zeros(256, dtype=np.uint16)
    state = 0
    for t in list(range(256)) * 2:
        state = ((state << k) | int(fresh[t])) & 0xFFFF
        states[t] = state
    return states


@pytest.mark.parametrize("k", KS)
def test_golden_pack_unpack(oracle, k):
    g = golden("tiles.npz")
    for s in range(4):
        np.testing.assert_array_equal(oracle.pack_tile(g[f"k{k}_encoded"][s], k), g[f"k{k}_packed"][s])
        np.testing.assert_array_equal(oracle.unpack_tile(g[f"k{k}_packed"][s], k), g[f"k{k}_unpacked"][s])
        np.testing.assert_array_equal(oracle.unpack_tile(g[f"k{k}_raw"][s], k), g[f"k{k}_raw_unpacked"][s])
        # the reference's tensor-level formulation agrees with its tile one
        np.testing.assert_array_equal(g[f"k{k}_raw_unpacked_tensor"][s], g[f"k{k}_raw_unpacked"][s])


@pytest.mark.parametrize("k", KS)
def test_unpack_matches_sliding_window_model(oracle, k):
    rng = np.random.default_rng(500 + k)
    for _ in range(8):
        packed = rng.integers(0, 65536, size=16 * k, dtype=np.uint16)
        np.testing.assert_array_equal(oracle.unpack_tile(packed, k), sliding_window_states(packed, k))


@pytest.mark.parametrize("k", KS)
def test_pack_unpack_roundtrip(oracle, k):
    rng = np.random.default_rng(k)
    mask = (1 << k) - 1
    enc = (rng.integers(0, 2**16, size=256, dtype=np.uint32) & mask).astype(np.uint16)
    dec = oracle.unpack_tile(oracle.pack_tile(enc, k), k)
    np.testing.assert_array_equal(dec & mask, enc)


@pytest.mark.parametrize("k", KS)
def test_states_shift_consistent(oracle, k):
    rng = np.random.default_rng(1000 + k)
    packed = rng.integers(0, 65536, size=16 * k, dtype=np.uint16)
    st = oracle.unpack_tile(packed, k).astype(np.uint32)
    keep = (1 << (16 - k)) - 1
    for t in range(256):
        assert st[(t + 1) % 256] >> k == (st[t] & keep), t


@pytest.mark.parametrize("k", KS)
def test_constant_tiles(oracle, k):
    assert (oracle.unpack_tile(np.zeros(16 * k, dtype=np.uint16), k) == 0).all()
    assert (oracle.unpack_tile(np.full(16 * k, 0xFFFF, dtype=np.uint16), k) == 0xFFFF).all()


def test_bad_k_raises(oracle):
    with pytest.raises(ValueError):
        oracle.unpack_tile(np.zeros(16 * 9, dtype=np.uint16), 9)
    with pytest.raises(ValueError):
        oracle.unpack_tile(np.zeros(10, dtype=np.uint16), 4)
