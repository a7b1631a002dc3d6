"""exl3_quantize_tiles / exl3_pack_trellis on the GPU against the oracle's
restatement of the production search (same path, bit for bit), the reference's
own assertions (tests/test_convert_metal.py:25-120) and the decoder."""
import numpy as np
import pytest
import torch

from test_oracle_search import _chain_valid, _tail_biting, valid_tail_biting_indices

pytestmark = pytest.mark.gpu
DEFAULT, MCG, MUL1 = 0, 1, 2


def _tiles(seed, n, scale=1.24371088):
    rng = np.random.default_rng(seed)
    return (rng.standard_normal((n, 256)) * scale).astype(np.float32)


@pytest.mark.parametrize("k,cb", [(2, MCG), (3, MCG), (4, DEFAULT), (4, MCG), (4, MUL1), (5, DEFAULT),
                                  (6, MCG), (7, MUL1), (7, MCG), (8, MCG), (8, DEFAULT)])
def test_same_path_as_the_oracle_search(cuda, oracle, k, cb):
    """Integer outputs: bit-exact. The first tile of each case uses the seed and
    scale of the reference's quality test."""
    from ponyexl3_amd import search

    scale = 1.0 if cb == MUL1 else 1.24371088
    tiles = np.concatenate([_tiles(100 + 10 * k + cb, 1, scale), _tiles(7 * k + cb, 2, 0.7 * scale),
                            np.zeros((1, 256), np.float32), np.full((1, 256), 9.0, np.float32)])
    print(f"search k={k} cb={cb}", flush=True)
    q, idx = search.quantize_tiles_np(tiles, k, cb, device=cuda)
    q_ref, idx_ref = oracle.quantize_tiles_search(tiles, k, cb)
    np.testing.assert_array_equal(idx, idx_ref)
    np.testing.assert_array_equal(q.view(np.uint32), q_ref.view(np.uint32))
    for row in idx:
        assert _tail_biting(row, k) and _chain_valid(row, k)
    np.testing.assert_array_equal(q, oracle.decode_table(cb)[idx].astype(np.float32))


@pytest.mark.parametrize("k,cb", [(2, MCG), (3, MCG), (4, DEFAULT), (4, MCG), (4, MUL1)])
def test_quality_against_the_exact_search(cuda, oracle, k, cb):
    """mse <= 1.10 x the exact float64 Viterbi (tests/test_convert_metal.py:44-71)."""
    from ponyexl3_amd import search

    scale = 1.0 if cb == MUL1 else 1.24371088
    tile = _tiles(100 + 10 * k + cb, 1, scale)
    q, idx = search.quantize_tiles_np(tile, k, cb, device=cuda)
    _, ref_tile = oracle.quantize_tile_exact(tile[0], k, cb)
    mse = float(np.mean((q[0] - tile[0]) ** 2))
    ref_mse = float(np.mean((ref_tile - tile[0]) ** 2))
    assert mse <= ref_mse * 1.10


@pytest.mark.parametrize("k", [2, 3, 4, 5, 8])
def test_recovers_an_exactly_representable_tile(cuda, oracle, k):
    from ponyexl3_amd import search

    encoded = valid_tail_biting_indices(k, seed=k)
    decoded = oracle.decode_table(MCG)[encoded].astype(np.float32).reshape(1, 256)
    q, idx = search.quantize_tiles_np(decoded, k, MCG, device=cuda)
    np.testing.assert_array_equal(idx[0], encoded)
    np.testing.assert_array_equal(q[0], decoded[0])


def test_small_scratch_budget_walks_the_batch_with_few_slots(cuda, oracle):
    """13 tiles through 3 backpointer slots (tests/test_convert_metal.py:89-103):
    same result as with every tile resident."""
    from ponyexl3_amd import search

    tiles = _tiles(333, 13, 1.0)
    q, idx = search.quantize_tiles_np(tiles, 2, MCG, device=cuda,
                                      max_scratch_bytes=3 * search.scratch_bytes_per_tile(2))
    q_all, idx_all = search.quantize_tiles_np(tiles, 2, MCG, device=cuda)
    assert q.shape == tiles.shape and idx.shape == tiles.shape and np.isfinite(q).all()
    np.testing.assert_array_equal(idx, idx_all)
    np.testing.assert_array_equal(q, q_all)
    for row in idx:
        assert _tail_biting(row, 2)
    q1, idx1 = search.quantize_tiles_np(tiles, 2, MCG, device=cuda, max_scratch_bytes=1)  # one slot
    np.testing.assert_array_equal(idx1, idx_all)


def test_argument_errors(cuda):
    from ponyexl3_amd import search

    tile = np.zeros((1, 256), dtype=np.float32)
    with pytest.raises(ValueError, match=r"supports K in \[2, 8\]"):
        search.quantize_tiles_np(tile, 1, MCG, device=cuda)
    with pytest.raises(ValueError):
        search.quantize_tiles_np(np.zeros((2, 100), np.float32), 4, MCG, device=cuda)
    with pytest.raises(ValueError):
        search.quantize_tiles_np(np.zeros((0, 256), np.float32), 4, MCG, device=cuda)
    with pytest.raises(ValueError):
        search.quantize_tiles_np(tile, 4, MCG, device=cuda, max_scratch_bytes=0)
    with pytest.raises(ValueError):
        search.pack_trellis(np.zeros((2, 100), np.uint16), 4, device=cuda)
    with pytest.raises(ValueError):
        search.pack_trellis(np.zeros((2, 256), np.uint16), 9, device=cuda)
    assert tuple(search.quantize_tiles(np.zeros(256, np.float32), 4, device=cuda)[0].shape) == (1, 256)


@pytest.mark.parametrize("k", [1, 2, 3, 4, 5, 6, 7, 8])
def test_pack_trellis_bit_exact(cuda, oracle, k):
    """tests/test_convert_metal.py:112-120, plus values with bits above K set
    (only the low K bits may be used)."""
    from ponyexl3_amd import search

    rng = np.random.default_rng(800 + k)
    encoded = rng.integers(0, 1 << k, size=(3, 5, 256), dtype=np.uint16)
    packed = search.pack_trellis(encoded, k, device=cuda).cpu().numpy().view(np.uint16)
    assert packed.shape == (3, 5, 16 * k)
    np.testing.assert_array_equal(packed, oracle.pack_trellis(encoded, k))
    np.testing.assert_array_equal(oracle.unpack_trellis(packed, k) & ((1 << k) - 1), encoded)
    noisy = encoded | (rng.integers(0, 65536, size=encoded.shape, dtype=np.uint16) << k).astype(np.uint16)
    packed2 = search.pack_trellis(noisy, k, device=cuda).cpu().numpy().view(np.uint16)
    np.testing.assert_array_equal(packed2, packed)


@pytest.mark.parametrize("k,cb", [(3, MCG), (4, DEFAULT), (6, MUL1)])
def test_search_pack_decode_round_trip(cuda, oracle, k, cb):
    """Encoder and decoder meet: searching an inner weight matrix tile by tile,
    packing the symbols and decoding the trellis with exl3_decode_full returns
    the search's quantized values at their row-major places."""
    from ponyexl3_amd import ops, search

    rng = np.random.default_rng(60 + k)
    tk, tn = 2, 3
    w = (rng.standard_normal((tk * 16, tn * 16)) * (1.0 if cb == MUL1 else 1.24)).astype(np.float32)
    perm = oracle.tensor_core_perm()  # kernel[i] = row_major[perm[i]]
    tiles = w.reshape(tk, 16, tn, 16).transpose(0, 2, 1, 3).reshape(tk * tn, 256)[:, perm]
    q, idx = search.quantize_tiles(tiles, k, cb, device=cuda)
    packed = search.pack_trellis((idx & ((1 << k) - 1)).reshape(tk, tn, 256), k, device=cuda)
    np.testing.assert_array_equal(oracle.unpack_trellis(packed.cpu().numpy().view(np.uint16), k),
                                  idx.cpu().numpy().view(np.uint16).reshape(tk, tn, 256))
    w_q = ops.decode_full(packed, k, cb).float().cpu().numpy()
    got = w_q.reshape(tk, 16, tn, 16).transpose(0, 2, 1, 3).reshape(tk * tn, 256)[:, perm]
    np.testing.assert_array_equal(got, q.cpu().numpy())
    assert float(np.mean((w_q - w) ** 2)) < 0.5 * float(np.mean(w ** 2))


def test_quantize_inner_matrix_feeds_the_forward_kernels(cuda, oracle):
    """Matrix in, trellis out: the packed result decodes (GPU and oracle) to the
    reconstruction the search reports, and an EXL3Linear built on it multiplies by
    exactly that matrix (no signs: suh = svh = 1)."""
    from ponyexl3_amd import EXL3Layer, EXL3Linear, ops, search

    rng = np.random.default_rng(11)
    n_in, n_out, k = 128, 256, 4
    w = (rng.standard_normal((n_in, n_out)) * 1.24).astype(np.float32)
    packed, states, recon = search.quantize_inner_matrix_direct(w, k=k, cb=MCG, return_states=True, device=cuda)
    assert tuple(packed.shape) == (n_in // 16, n_out // 16, 16 * k) and tuple(states.shape) == (8, 16, 256)
    packed_np = packed.cpu().numpy().view(np.uint16)
    np.testing.assert_array_equal(oracle.decode_trellis(packed_np, k, MCG).astype(np.float32), recon.cpu().numpy())
    np.testing.assert_array_equal(ops.decode_full(packed, k, MCG).float().cpu().numpy(), recon.cpu().numpy())
    tiles = search.inner_to_kernel_tiles(torch.from_numpy(w).to(cuda))
    np.testing.assert_array_equal(search.kernel_tiles_to_inner(tiles, n_in, n_out).cpu().numpy(), w)
    rel = float(np.linalg.norm(recon.cpu().numpy() - w) / np.linalg.norm(w))
    assert rel < 0.1  # 4 bits per weight: about 7 % relative error on Gaussian weights
    ones_in, ones_out = np.ones(n_in, np.float16), np.ones(n_out, np.float16)
    layer = EXL3Layer("q", n_in, n_out, k, packed_np, ones_in, ones_out, None, mcg=True, mul1=False)
    x = rng.standard_normal((3, n_in)).astype(np.float16)
    y = EXL3Linear(layer)(torch.from_numpy(x).to(cuda)).cpu().numpy()
    ref = oracle.linear_forward(packed_np, k, MCG, ones_in, ones_out, x)
    np.testing.assert_allclose(y.astype(np.float32), ref.astype(np.float32), rtol=2e-3, atol=2e-2)
    packed2, none_states, _ = search.quantize_inner_matrix_direct(w, k=k, cb=MCG, device=cuda,
                                                                  verify_roundtrip=True)
    assert none_states is None and torch.equal(packed2, packed)
    with pytest.raises(ValueError):
        search.quantize_inner_matrix_direct(np.zeros((100, 256), np.float32), k=4, device=cuda)


@pytest.mark.parametrize("k", [1, 2, 3, 4, 5, 6, 7, 8])
def test_unpack_trellis_bit_exact(cuda, oracle, k):
    """Raw random words (every fill is a legal bitstream), 37 tiles = a partly filled
    last wavefront: codewords equal the oracle's unpack; pack(unpack & mask) is the
    identity."""
    from ponyexl3_amd import search

    rng = np.random.default_rng(500 + k)
    packed = rng.integers(0, 65536, size=(37, 16 * k), dtype=np.uint16)
    got = search.unpack_trellis(packed, k, device=cuda)
    ref = np.stack([oracle.unpack_tile(t, k) for t in packed])
    np.testing.assert_array_equal(got.cpu().numpy().view(np.uint16), ref)
    again = search.pack_trellis(got & ((1 << k) - 1), k, device=cuda)
    np.testing.assert_array_equal(again.cpu().numpy().view(np.uint16), packed)
    with pytest.raises(ValueError):
        search.unpack_trellis(packed, k % 8 + 1, device=cuda)
