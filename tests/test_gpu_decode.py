"""exl3_decode_full on the GPU must be bit-exact with the oracle's decode."""
import numpy as np
import pytest
import torch

from conftest import golden, rel_l2

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


def test_reconstruct_public_weights(cuda, oracle):
    """diag(suh).H.W.H.diag(svh) against the oracle (ref/reconstruct.py:26-49), and
    the reference's own check that x @ W_pub reproduces the layer forward
    (tests/test_decode_reconstruct.py:40-69)."""
    from ponyexl3_amd import EXL3Linear, make_exl3_layer, ops

    layer = make_exl3_layer(k=3, in_features=256, out_features=384, seed=77, mcg=True)
    tr = ops.as_trellis_tensor(layer.trellis, cuda)
    suh, svh = torch.from_numpy(layer.suh).to(cuda), torch.from_numpy(layer.svh).to(cuda)
    w_pub = ops.reconstruct_public_weights(tr, suh, svh, 3, int(layer.codebook_mode))
    ref = oracle.reconstruct_public_weights(layer.trellis, layer.suh, layer.svh, 3, int(layer.codebook_mode))
    assert w_pub.dtype == torch.float16 and tuple(w_pub.shape) == (256, 384)
    assert rel_l2(w_pub.cpu().numpy(), ref) < 1e-3
    inner = ops.reconstruct_inner(tr, 3, int(layer.codebook_mode), n_offset=128, n_count=128)
    np.testing.assert_array_equal(
        inner.cpu().numpy().view(np.uint16),
        oracle.decode_trellis(layer.trellis, 3, int(layer.codebook_mode), tn_offset=8, tn_count=8).view(np.uint16))
    rng = np.random.default_rng(5)
    x = torch.from_numpy(rng.standard_normal((4, 256)).astype(np.float16)).to(cuda)
    y = EXL3Linear(layer)(x).float()
    y_pub = x.float() @ w_pub.float()
    assert float((y - y_pub).norm() / y_pub.norm()) < 5e-3
    with pytest.raises(ValueError):
        ops.reconstruct_inner(tr, 3, int(layer.codebook_mode), n_offset=64)


@pytest.mark.parametrize("k", range(1, 9))
@pytest.mark.parametrize("cb", [0, 1, 2])
def test_transposed_and_expert_grouped_layouts_bit_exact(cuda, oracle, k, cb):
    """The (out, in) and (E, in, out_e) layouts hold exactly the weights of the
    row-major decode (decode_full_t_mlx / decode_full_eg_mlx,
    ponyexl3/mlx/gemv_metal.py:746-866); 11 tile rows and 21 / 12 tile columns
    leave partly filled wavefronts in both kernels."""
    from ponyexl3_amd import ops

    rng = np.random.default_rng(900 + 10 * k + cb)
    tr = rng.integers(0, 65536, size=(11, 12, 16 * k), dtype=np.uint16)
    full = oracle.decode_trellis(tr, k, cb).view(np.uint16)  # (176, 192)
    trt = ops.as_trellis_tensor(tr, cuda)
    print(f"layouts k={k} cb={cb}", flush=True)
    wt = ops.decode_full_t(trt, k, cb).cpu().numpy().view(np.uint16)
    np.testing.assert_array_equal(wt, full.T)
    for off, cnt in ((5, 3), (0, 1), (11, 1), (2, 9)):
        wt = ops.decode_full_t(trt, k, cb, tn_offset=off, tn_count=cnt).cpu().numpy().view(np.uint16)
        assert wt.shape == (16 * cnt, 176)
        np.testing.assert_array_equal(wt, full[:, 16 * off:16 * (off + cnt)].T)
    for tpe in (1, 3, 4, 12):
        eg = ops.decode_full_eg(trt, k, cb, tiles_per_e=tpe).cpu().numpy().view(np.uint16)
        assert eg.shape == (12 // tpe, 176, 16 * tpe)
        for e in range(12 // tpe):
            np.testing.assert_array_equal(eg[e], full[:, 16 * tpe * e:16 * tpe * (e + 1)])


def test_layout_variant_errors(cuda):
    from ponyexl3_amd import ops

    tr = torch.zeros((2, 6, 64), dtype=torch.int16, device=cuda)
    with pytest.raises(ValueError):
        ops.decode_full_eg(tr, 4, 0, tiles_per_e=4)  # 6 tile columns do not split into fours
    with pytest.raises(ValueError):
        ops.decode_full_eg(tr, 4, 0, tiles_per_e=0)
    with pytest.raises(ValueError):
        ops.decode_full_t(tr, 4, 0, tn_offset=5, tn_count=2)
    assert tuple(ops.decode_full_t(tr, 4, 0, tn_offset=6, tn_count=0).shape) == (0, 32)
