"""Fused decode GEMV (rows 1..8) against the oracle's decode + fp64 matmul."""
import numpy as np
import pytest
import torch

from conftest import rel_l2

pytestmark = pytest.mark.gpu
TOL = 1e-3  # rel-L2 bar; the kernel accumulates in fp32 and normally lands near 1e-6


def _t(a, device):
    return torch.from_numpy(np.ascontiguousarray(a)).to(device)


def _ref(oracle, tr, k, cb, xh):
    w = oracle.decode_trellis(tr, k, cb).astype(np.float64)
    return xh.astype(np.float64) @ w


@pytest.mark.parametrize("k", range(1, 9))
@pytest.mark.parametrize("cb", [0, 1, 2])
def test_gemv_all_k_cb(cuda, oracle, k, cb):
    from ponyexl3_amd import ops

    rng = np.random.default_rng(200 + 10 * k + cb)
    tr = rng.integers(0, 65536, size=(24, 16, 16 * k), dtype=np.uint16)  # 384 -> 256
    xh = rng.standard_normal(384).astype(np.float16)
    print(f"gemv k={k} cb={cb}", flush=True)
    y = ops.inner_gemv(_t(xh, cuda), ops.as_trellis_tensor(tr, cuda), k, cb).cpu().numpy()
    assert y.dtype == np.float32 and y.shape == (256,)
    assert rel_l2(y, _ref(oracle, tr, k, cb, xh)) < 1e-5


@pytest.mark.parametrize("rows", [1, 2, 3, 4, 5, 8])
@pytest.mark.parametrize("k,cb", [(4, 0), (3, 1), (6, 0), (2, 1), (8, 0), (5, 1)])
def test_small_batch_rows(cuda, oracle, rows, k, cb):
    from ponyexl3_amd import ops

    rng = np.random.default_rng(300 + rows + 10 * k)
    tr = rng.integers(0, 65536, size=(64, 24, 16 * k), dtype=np.uint16)  # 1024 -> 384, split-K active
    xh = rng.standard_normal((rows, 1024)).astype(np.float16)
    print(f"gemm rows={rows} k={k} cb={cb}", flush=True)
    y = ops.inner_gemm(_t(xh, cuda), ops.as_trellis_tensor(tr, cuda), k, cb).cpu().numpy()
    assert y.shape == (rows, 384)
    assert rel_l2(y, _ref(oracle, tr, k, cb, xh)) < 1e-5


def test_fused_groups_and_tile_map(cuda, oracle):
    from ponyexl3_amd import ops

    rng = np.random.default_rng(7)
    k, cb = 4, 1
    tr = rng.integers(0, 65536, size=(16, 40, 64), dtype=np.uint16)  # 256 -> 640 = 5 groups
    xh = rng.standard_normal((2, 3, 256)).astype(np.float16)
    sub = np.array([0, 0, 1, 2, 2], dtype=np.int32)
    y = ops.inner_gem_fused(_t(xh, cuda), ops.as_trellis_tensor(tr, cuda), k, cb,
                            group_sub=_t(sub, cuda)).cpu().numpy()
    w = oracle.decode_trellis(tr, k, cb).astype(np.float64)
    for g in range(5):
        ref = xh[:, sub[g]].astype(np.float64) @ w[:, 128 * g : 128 * (g + 1)]
        assert rel_l2(y[:, 128 * g : 128 * (g + 1)], ref) < 1e-5
    # tile_map: gather groups 4 and 1 only
    tile = np.array([32, 8], dtype=np.int32)
    sub2 = np.array([1, 0], dtype=np.int32)
    y2 = ops.inner_gem_fused(_t(xh, cuda), ops.as_trellis_tensor(tr, cuda), k, cb,
                             group_sub=_t(sub2, cuda), group_tile=_t(tile, cuda)).cpu().numpy()
    assert y2.shape == (2, 256)
    assert rel_l2(y2[:, :128], xh[:, 1].astype(np.float64) @ w[:, 512:640]) < 1e-5
    assert rel_l2(y2[:, 128:], xh[:, 0].astype(np.float64) @ w[:, 128:256]) < 1e-5


def test_deterministic(cuda):
    from ponyexl3_amd import ops

    rng = np.random.default_rng(8)
    tr = ops.as_trellis_tensor(rng.integers(0, 65536, size=(320, 64, 64), dtype=np.uint16), cuda)
    xh = _t(rng.standard_normal(5120).astype(np.float16), cuda)
    a = ops.inner_gemv(xh, tr, 4, 0)
    b = ops.inner_gemv(xh, tr, 4, 0)
    assert torch.equal(a, b)


def test_config1_gemv_full_size(cuda, oracle):
    from ponyexl3_amd import ops

    rng = np.random.default_rng(10_004)
    tr = rng.integers(0, 65536, size=(256, 256, 64), dtype=np.uint16)
    xh = rng.standard_normal(4096).astype(np.float16)
    y = ops.inner_gemv(_t(xh, cuda), ops.as_trellis_tensor(tr, cuda), 4, 0).cpu().numpy()
    assert rel_l2(y, _ref(oracle, tr, 4, 0, xh)) < 1e-5


def test_linearity_at_config2_size(cuda):
    """down_proj shape 17408 -> 5120: W(a + b) == W a + W b within fp16 input rounding."""
    from ponyexl3_amd import ops

    rng = np.random.default_rng(9)
    tr = ops.as_trellis_tensor(rng.integers(0, 65536, size=(1088, 320, 64), dtype=np.uint16), cuda)
    a = np.round(rng.standard_normal(17408) * 8) / 8  # exactly representable, sums stay exact in fp16
    b = np.round(rng.standard_normal(17408) * 8) / 8
    ya = ops.inner_gemv(_t(a.astype(np.float16), cuda), tr, 4, 0).cpu().numpy().astype(np.float64)
    yb = ops.inner_gemv(_t(b.astype(np.float16), cuda), tr, 4, 0).cpu().numpy().astype(np.float64)
    yab = ops.inner_gemv(_t((a + b).astype(np.float16), cuda), tr, 4, 0).cpu().numpy().astype(np.float64)
    assert rel_l2(yab, ya + yb) < 1e-5


def test_errors(cuda):
    from ponyexl3_amd import ops

    tr = torch.zeros((8, 8, 64), dtype=torch.int16, device=cuda)
    with pytest.raises(ValueError):
        ops.inner_gemv(torch.zeros(64, dtype=torch.float16, device=cuda), tr, 4, 0)
    with pytest.raises(ValueError):
        ops.inner_gem_fused(torch.zeros((9, 1, 128), dtype=torch.float16, device=cuda), tr, 4, 0)
    with pytest.raises(ValueError):
        ops.inner_gem_fused(torch.zeros((1, 2, 128), dtype=torch.float16, device=cuda), tr, 4, 0)


@pytest.mark.parametrize("k,cb", [(1, 0), (2, 1), (3, 0), (4, 0), (4, 1), (4, 2), (5, 1), (6, 0), (7, 1), (8, 0)])
def test_one_hot_activations_reproduce_the_decoded_weights_exactly(cuda, oracle, k, cb):
    """A one-hot activation row selects one row of W: the fp32 result must equal the
    oracle's decoded fp16 weight exactly, for every row count of the kernel."""
    from ponyexl3_amd import ops

    rng = np.random.default_rng(700 + 10 * k + cb)
    tr_np = rng.integers(0, 65536, size=(16, 16, 16 * k), dtype=np.uint16)  # 256 -> 256
    tr = ops.as_trellis_tensor(tr_np, cuda)
    w = oracle.decode_trellis(tr_np, k, cb).astype(np.float32)
    for rows in (1, 2, 3, 4, 8):
        pick = rng.permutation(256)[:rows]
        xh = torch.zeros((rows, 1, 256), dtype=torch.float16, device=cuda)
        xh[torch.arange(rows), 0, torch.from_numpy(pick).to(cuda)] = 1.0
        y = ops.inner_gem_fused(xh, tr, k, cb).cpu().numpy()
        np.testing.assert_array_equal(y, w[pick])
