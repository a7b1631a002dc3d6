"""exl3_decode_full on the GPU must be bit-exact with the oracle's decode."""
import numpy as np
import pytest
import torch

from conftest import golden

pytestmark = pytest.mark.gpu


def _decode(trellis_np, k, cb, device, **kw):
    from ponyexl3_amd import ops

    w = ops.decode_full(ops.as_trellis_tensor(trellis_np, device), k, cb, **kw)
    torch.cuda.synchronize()
    return w.cpu().numpy()


@pytest.mark.parametrize("k", range(1, 9))
@pytest.mark.parametrize("cb", [0, 1, 2])
def test_golden_layers_bit_exact(cuda, k, cb):
    g = golden("decoded_layers.npz")
    w = _decode(g[f"k{k}_cb{cb}_trellis"], k, cb, cuda)
    np.testing.assert_array_equal(w.view(np.uint16), g[f"k{k}_cb{cb}_w"])


@pytest.mark.parametrize("k", range(1, 9))
@pytest.mark.parametrize("cb", [0, 1, 2])
def test_random_trellis_bit_exact(cuda, oracle, k, cb):
    rng = np.random.default_rng(100 * k + cb)
    tr = rng.integers(0, 65536, size=(9, 21, 16 * k), dtype=np.uint16)  # ragged: 21 tile columns
    print(f"decode k={k} cb={cb}", flush=True)
    w = _decode(tr, k, cb, cuda)
    np.testing.assert_array_equal(w.view(np.uint16), oracle.decode_trellis(tr, k, cb).view(np.uint16))


def test_column_slices(cuda, oracle):
    rng = np.random.default_rng(5)
    tr = rng.integers(0, 65536, size=(4, 19, 80), dtype=np.uint16)
    full = oracle.decode_trellis(tr, 5, 1)
    for off, cnt in [(0, 1), (3, 9), (18, 1), (8, 8), (1, 18), (0, 0)]:
        w = _decode(tr, 5, 1, cuda, tn_offset=off, tn_count=cnt)
        assert w.shape == (64, 16 * cnt)
        np.testing.assert_array_equal(w.view(np.uint16), full[:, 16 * off : 16 * (off + cnt)].view(np.uint16))


def test_constant_tiles(cuda):
    for cb, bits in ((0, 0x3A25), (1, 0x3F60), (2, 0xC2E8)):
        w = _decode(np.zeros((2, 3, 64), dtype=np.uint16), 4, cb, cuda)
        assert (w.view(np.uint16) == bits).all()


def test_config1_full_size_bit_exact(cuda, oracle):
    """4096 -> 4096, K=4, 3INST: trellis [256, 256, 64]."""
    rng = np.random.default_rng(10_000 + 4)
    tr = rng.integers(0, 65536, size=(256, 256, 64), dtype=np.uint16)
    w = _decode(tr, 4, 0, cuda)
    np.testing.assert_array_equal(w.view(np.uint16), oracle.decode_trellis(tr, 4, 0).view(np.uint16))


def test_errors(cuda):
    from ponyexl3_amd import ops

    tr = torch.zeros((2, 3, 64), dtype=torch.int16, device=cuda)
    with pytest.raises(ValueError):
        ops.decode_full(tr, 3, 0)  # packed size does not match K
    with pytest.raises(ValueError):
        ops.decode_full(tr, 4, 0, tn_offset=2, tn_count=2)
    with pytest.raises(ValueError):
        ops.decode_full(tr, 4, 5)
