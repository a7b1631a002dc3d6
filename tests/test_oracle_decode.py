"""Pins the tile permutation and exl3o_decode_trellis
(ponyexl3/ref/perm.py, ponyexl3/ref/decode.py)."""
import numpy as np
import pytest

from conftest import golden


def test_perm_matches_reference_and_is_bijection(oracle):
    g = golden("perm.npz")
    perm = oracle.tensor_core_perm()
    np.testing.assert_array_equal(perm, g["perm"])
    assert sorted(perm.tolist()) == list(range(256))
    inv = np.empty(256, dtype=np.int32)
    inv[perm] = np.arange(256)
    np.testing.assert_array_equal(inv, g["inverse"])


def test_perm_is_mma_fragment_map(oracle):
    """mma.m16n8k16 B-fragment order: codewords 4l..4l+3 of 'lane' l share column
    (l>>3) + 8*(l&1) and cover rows {2q, 2q+1, 2q+8, 2q+9}, q = (l>>1)&3."""
    perm = oracle.tensor_core_perm()
    for l in range(64):
        q = (l >> 1) & 3
        rows = [2 * q, 2 * q + 1, 2 * q + 8, 2 * q + 9]
        col = (l >> 3) + 8 * (l & 1)
        assert [int(p) for p in perm[4 * l : 4 * l + 4]] == [r * 16 + col for r in rows]


@pytest.mark.parametrize("k", range(1, 9))
@pytest.mark.parametrize("cb", [0, 1, 2])
def test_golden_decoded_layers(oracle, k, cb):
    g = golden("decoded_layers.npz")
    w = oracle.decode_trellis(g[f"k{k}_cb{cb}_trellis"], k, cb)
    assert w.shape == (32, 48) and w.dtype == np.float16
    np.testing.assert_array_equal(w.view(np.uint16), g[f"k{k}_cb{cb}_w"])


def test_zero_tile_decodes_to_constant(oracle):
    for cb, bits in ((0, 0x3A25), (1, 0x3F60), (2, 0xC2E8)):
        t = oracle.decode_tile(np.zeros(64, dtype=np.uint16), 4, cb)
        assert (t.view(np.uint16) == bits).all()


def test_column_slice(oracle):
    rng = np.random.default_rng(3)
    tr = rng.integers(0, 65536, size=(2, 5, 48), dtype=np.uint16)
    full = oracle.decode_trellis(tr, 3, 1)
    part = oracle.decode_trellis(tr, 3, 1, tn_offset=1, tn_count=3)
    np.testing.assert_array_equal(part.view(np.uint16), full[:, 16:64].view(np.uint16))
    with pytest.raises(ValueError):
        oracle.decode_trellis(tr, 3, 1, tn_offset=4, tn_count=2)
    with pytest.raises(ValueError):
        oracle.decode_trellis(tr, 4, 1)


def test_decode_tile_places_by_perm(oracle):
    rng = np.random.default_rng(9)
    packed = rng.integers(0, 65536, size=80, dtype=np.uint16)
    cw = oracle.unpack_tile(packed, 5)
    tab = oracle.decode_table(0)
    perm = oracle.tensor_core_perm()
    expect = np.empty(256, dtype=np.float16)
    expect[perm] = tab[cw]
    np.testing.assert_array_equal(oracle.decode_tile(packed, 5, 0).reshape(-1).view(np.uint16),
                                  expect.view(np.uint16))
