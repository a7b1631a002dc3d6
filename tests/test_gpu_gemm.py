"""MFMA prefill GEMM against the oracle-decoded fp16 weights times xh
(fp32 accumulation, rel-L2 <= 1e-3)."""
import ctypes

import numpy as np
import pytest
import torch

from conftest import rel_l2

pytestmark = pytest.mark.gpu
TOL = 1e-3


def _t(a, device):
    return torch.from_numpy(np.ascontiguousarray(a)).to(device)


@pytest.mark.parametrize("rows", [9, 17, 100, 256, 300, 513])
@pytest.mark.parametrize("k,cb", [(4, 0), (3, 1), (5, 0), (8, 1), (1, 0), (7, 1), (4, 2)])
def test_gemm_matches_oracle(cuda, oracle, rows, k, cb):
    from ponyexl3_amd import ops

    rng = np.random.default_rng(400 + rows + k)
    tr = rng.integers(0, 65536, size=(24, 24, 16 * k), dtype=np.uint16)  # 384 -> 384
    xh = rng.standard_normal((rows, 384)).astype(np.float16)
    print(f"gemm rows={rows} k={k} cb={cb}", flush=True)
    y = ops.inner_gemm(_t(xh, cuda), ops.as_trellis_tensor(tr, cuda), k, cb).cpu().numpy()
    assert y.dtype == np.float16 and y.shape == (rows, 384)
    w = oracle.decode_trellis(tr, k, cb).astype(np.float64)
    ref = xh.astype(np.float64) @ w
    assert rel_l2(y, ref) < 5e-4  # one fp16 rounding of the result


@pytest.mark.parametrize("k", [1, 2, 3, 4, 5, 6, 7, 8])
@pytest.mark.parametrize("cb", [0, 1, 2])
def test_identity_activations_reproduce_the_decoded_weights_bit_for_bit(cuda, oracle, k, cb):
    """x = I makes every output the sum of one weight and zeros, which fp32 MFMA
    accumulation and the single fp16 cast keep exact: the GEMM's in-kernel decode,
    LDS layout and fragment mapping against the oracle's decoded weights, every bit
    width and codebook, 64-, 128- and 256-row blocks."""
    from ponyexl3_amd import ops

    rng = np.random.default_rng(600 + 10 * k + cb)
    tr_np = rng.integers(0, 65536, size=(24, 24, 16 * k), dtype=np.uint16)  # 384 -> 384
    tr = ops.as_trellis_tensor(tr_np, cuda)
    w = oracle.decode_trellis(tr_np, k, cb).view(np.uint16)
    eye = torch.eye(384, dtype=torch.float16, device=cuda)
    print(f"gemm identity k={k} cb={cb}", flush=True)
    for rows in (384, 100, 40):  # MI = 8, 4, 2
        y = ops.inner_gemm(eye[:rows].contiguous(), tr, k, cb).cpu().numpy().view(np.uint16)
        np.testing.assert_array_equal(y, w[:rows])


def test_gemm_column_slice(cuda, oracle):
    from ponyexl3_amd import ops

    rng = np.random.default_rng(41)
    tr = rng.integers(0, 65536, size=(16, 40, 64), dtype=np.uint16)
    xh = rng.standard_normal((64, 256)).astype(np.float16)
    y = ops.inner_gemm(_t(xh, cuda), ops.as_trellis_tensor(tr, cuda), 4, 0, tn_offset=16, tn_count=16).cpu().numpy()
    w = oracle.decode_trellis(tr, 4, 0, tn_offset=16, tn_count=16).astype(np.float64)
    assert rel_l2(y, xh.astype(np.float64) @ w) < 5e-4


def test_slice_with_half_width_last_block_and_split_tiles(cuda, oracle):
    """A column slice that starts inside the matrix, ends with a half-width
    (128-column) block and is few enough tiles that every tile is split along the
    reduction dimension; the columns outside the slice must stay untouched."""
    from ponyexl3_amd import _lib, ops

    rng = np.random.default_rng(45)
    tr_np = rng.integers(0, 65536, size=(128, 48, 64), dtype=np.uint16)  # 2048 -> 768
    tr = ops.as_trellis_tensor(tr_np, cuda)
    xh_np = rng.standard_normal((300, 2048)).astype(np.float16)
    assert _lib.load().exl3_gemm_workspace_bytes(300, 128, 24) > 0
    y = ops.inner_gemm(_t(xh_np, cuda), tr, 4, 0, tn_offset=8, tn_count=24).cpu().numpy()
    assert y.shape == (300, 384)
    w = oracle.decode_trellis(tr_np, 4, 0, tn_offset=8, tn_count=24).astype(np.float64)
    assert rel_l2(y, xh_np.astype(np.float64) @ w) < 5e-4


def test_small_batch_and_prefill_kernels_agree(cuda):
    from ponyexl3_amd import ops

    rng = np.random.default_rng(42)
    tr = ops.as_trellis_tensor(rng.integers(0, 65536, size=(64, 32, 64), dtype=np.uint16), cuda)
    xh = _t(rng.standard_normal((16, 1024)).astype(np.float16), cuda)
    big = ops.inner_gemm(xh, tr, 4, 0).float().cpu().numpy()
    small = torch.cat([ops.inner_gemm(xh[:8].contiguous(), tr, 4, 0), ops.inner_gemm(xh[8:].contiguous(), tr, 4, 0)])
    assert rel_l2(big, small.cpu().numpy()) < 5e-4


def test_config3_prefill_against_decoded_weights(cuda, oracle):
    """M = 2048 on the q_proj shape 5120 -> 8192: compare with the decoded fp16
    weights times xh in fp32; the decoded matrix (all 41.9 M weights) is first
    checked bit for bit against the oracle's decode."""
    from ponyexl3_amd import ops

    rng = np.random.default_rng(30_004)
    tr_np = rng.integers(0, 65536, size=(320, 512, 64), dtype=np.uint16)
    tr = ops.as_trellis_tensor(tr_np, cuda)
    g = torch.Generator().manual_seed(5)
    xh = torch.randn((2048, 5120), generator=g).to(torch.float16).to(cuda)
    y = ops.inner_gemm(xh, tr, 4, 0)
    w = ops.decode_full(tr, 4, 0)
    np.testing.assert_array_equal(w.cpu().numpy().view(np.uint16),
                                  oracle.decode_trellis(tr_np, 4, 0).view(np.uint16))
    ref = xh.float() @ w.float()
    err = (y.float() - ref).norm() / ref.norm()
    assert float(err) < 5e-4


@pytest.mark.parametrize("rows", [40, 100, 300])
def test_split_tiles_match_oracle_and_unsplit(cuda, oracle, rows):
    """Few tiles and a deep reduction: every tile is cut into reduction ranges
    whose fp32 partial tiles a second kernel adds. Checked against the oracle,
    against the same call without a workspace (no split) and for run-to-run
    determinism."""
    import ctypes

    from ponyexl3_amd import _lib, ops

    rng = np.random.default_rng(43 + rows)
    tr_np = rng.integers(0, 65536, size=(128, 64, 64), dtype=np.uint16)  # 2048 -> 1024, K = 4
    tr = ops.as_trellis_tensor(tr_np, cuda)
    xh_np = rng.standard_normal((rows, 2048)).astype(np.float16)
    xh = _t(xh_np, cuda)
    lib = _lib.load()
    assert lib.exl3_gemm_workspace_bytes(rows, 128, 64) > 0  # this shape does split
    print(f"gemm split rows={rows}", flush=True)
    y1 = ops.inner_gemm(xh, tr, 4, 0)
    y2 = ops.inner_gemm(xh, tr, 4, 0)
    assert torch.equal(y1, y2)
    ref = xh_np.astype(np.float64) @ oracle.decode_trellis(tr_np, 4, 0).astype(np.float64)
    assert rel_l2(y1.cpu().numpy(), ref) < 5e-4
    y0 = torch.empty_like(y1)
    rc = lib.exl3_gemm(
        ctypes.c_void_p(xh.data_ptr()), rows, 2048, ctypes.c_void_p(tr.data_ptr()), 128, 64, 4, 0,
        0, 64, ctypes.c_void_p(y0.data_ptr()), 1024, None, 0,
        ctypes.c_void_p(torch.cuda.current_stream().cuda_stream))
    assert rc == 0
    assert rel_l2(y0.cpu().numpy(), ref) < 5e-4
    assert rel_l2(y0.cpu().numpy(), y1.cpu().numpy()) < 5e-4


@pytest.mark.parametrize("rows,slots,n_out,k,cb", [
    (300, 5, 1024, 4, 0), (100, 5, 1024, 4, 0), (40, 7, 1024, 4, 0), (300, 7, 1152, 4, 0),
    (300, 5, 1024, 8, 2), (300, 5, 1024, 7, 1), (100, 5, 1024, 3, 0), (40, 7, 1024, 6, 1)])
def test_runs_that_cross_tile_borders(cuda, oracle, monkeypatch, rows, slots, n_out, k, cb):
    """With few workgroup slots the tiles of the last round are laid end to end and
    cut into one run per slot, so that runs cross from one tile into the next (the
    schedule of o_proj and down_proj at M = 2048, here forced on a small shape by the
    slot count): whole tiles and two-piece workgroups in one launch, for the three
    block heights, and with a half-width last column block among the split tiles
    (1152 columns), and at other K / codebooks (K = 8 with MUL1 is the instantiation
    with the most registers); the plain GEMM and the whole layer (fix-up with the
    output transform) against the oracle, twice for determinism."""
    from ponyexl3_amd import ops

    monkeypatch.setenv("EXL3_GEMM_SLOTS", str(slots))
    rng = np.random.default_rng(4700 + rows + 10 * k + cb)
    tr_np = rng.integers(0, 65536, size=(512, n_out // 16, 16 * k), dtype=np.uint16)  # 8192 -> n_out
    tr = ops.as_trellis_tensor(tr_np, cuda)
    suh = np.where(rng.random(8192) > 0.5, -1, 1).astype(np.float16)
    svh = np.where(rng.random(n_out) > 0.5, -1, 1).astype(np.float16)
    x_np = (rng.standard_normal((rows, 8192)) * 0.25).astype(np.float16)
    x = _t(x_np, cuda)
    print(f"gemm crossing runs rows={rows} slots={slots} n_out={n_out} k={k} cb={cb}", flush=True)
    y1 = ops.inner_gemm(x, tr, k, cb)
    y2 = ops.inner_gemm(x, tr, k, cb)
    assert torch.equal(y1, y2)
    w = oracle.decode_trellis(tr_np, k, cb).astype(np.float64)
    assert rel_l2(y1.cpu().numpy(), x_np.astype(np.float64) @ w) < 5e-4
    z1 = ops.linear_forward(x, tr, k, cb, _t(suh, cuda), _t(svh, cuda))
    z2 = ops.linear_forward(x, tr, k, cb, _t(suh, cuda), _t(svh, cuda))
    assert torch.equal(z1, z2)
    ref = oracle.linear_forward(tr_np, k, cb, suh, svh, x_np)
    assert rel_l2(z1.cpu().numpy(), ref) < 1e-3


@pytest.mark.parametrize("n_in,n_out", [(17408, 5120), (5120, 34816)])
def test_config3_split_shapes_against_decoded_weights(cuda, n_in, n_out):
    """M = 2048 on down_proj (160 tiles, their steps end to end in one run per CU, runs
    crossing from one tile into the next) and gate+up (1088 tiles: four full rounds
    and 64 tiles in four runs each) against the
    bit-exact decoded weights times xh in fp32."""
    from ponyexl3_amd import ops

    g = torch.Generator().manual_seed(n_in)
    tr = torch.randint(-32768, 32767, (n_in // 16, n_out // 16, 64), generator=g, dtype=torch.int16).to(cuda)
    xh = (torch.randn((2048, n_in), generator=g) * 0.1).to(torch.float16).to(cuda)
    print(f"gemm config3 {n_in}->{n_out}", flush=True)
    y = ops.inner_gemm(xh, tr, 4, 0)
    w = ops.decode_full(tr, 4, 0)
    worst = 0.0
    for c0 in range(0, n_out, 8192):  # fp32 reference in column slabs
        ref = xh.float() @ w[:, c0:c0 + 8192].float()
        err = (y[:, c0:c0 + 8192].float() - ref).norm() / ref.norm()
        worst = max(worst, float(err))
    assert worst < 5e-4


def test_grouped_gemm_drops_bad_table_entries(cuda, oracle):
    """The row-block table of exl3_gemm_grouped is caller memory: entries that name a
    group outside the stack, a negative first row or an end row past the activations
    must not make the kernel read or write out of bounds. Bad entries are skipped,
    an end row past n_rows is clamped; the valid blocks come out as usual."""
    from ponyexl3_amd import ops

    rng = np.random.default_rng(77)
    n_groups, gt = 3, 16  # three groups of 256 columns each
    tr_np = rng.integers(0, 65536, size=(16, n_groups * gt, 64), dtype=np.uint16)  # in = 256
    tr = ops.as_trellis_tensor(tr_np, cuda)
    xh_np = rng.standard_normal((96, 256)).astype(np.float16)
    xh = _t(xh_np, cuda)
    table = torch.tensor([[0, 0, 40, 0],      # group 0: rows 0..39
                          [7, 40, 60, 0],     # group out of range: skipped
                          [1, -5, 20, 0],     # negative first row: skipped
                          [2, 64, 4000, 0],   # end row past the matrix: clamped to 96
                          [-1, 0, 10, 0]],    # negative group: skipped
                         dtype=torch.int32, device=cuda)
    sentinel = 12345.0
    y = torch.full((96, gt * 16), sentinel, dtype=torch.float16, device=cuda)
    from ponyexl3_amd import _lib
    rc = _lib.load().exl3_gemm_grouped(
        ctypes.c_void_p(xh.data_ptr()), 96, 256, ctypes.c_void_p(tr.data_ptr()), 16, n_groups * gt, 4, 0,
        0, gt, n_groups, ctypes.c_void_p(table.data_ptr()), table.shape[0], 64,
        ctypes.c_void_p(y.data_ptr()), gt * 16, ctypes.c_void_p(torch.cuda.current_stream().cuda_stream))
    assert rc == 0
    torch.cuda.synchronize()
    w = oracle.decode_trellis(tr_np, 4, 0).astype(np.float64)
    got = y.cpu().numpy()
    assert rel_l2(got[:40], xh_np[:40].astype(np.float64) @ w[:, :256]) < 5e-4
    assert rel_l2(got[64:96], xh_np[64:96].astype(np.float64) @ w[:, 512:768]) < 5e-4
    assert (got[40:64] == np.float16(sentinel)).all()  # rows of the dropped entries are untouched


def test_errors(cuda):
    from ponyexl3_amd import ops

    tr = torch.zeros((8, 9, 64), dtype=torch.int16, device=cuda)
    with pytest.raises(ValueError):
        ops.inner_gemm(torch.zeros((32, 128), dtype=torch.float16, device=cuda), tr, 4, 0)  # 9 tile columns
    with pytest.raises(ValueError):
        ops.inner_gemm(torch.zeros((32, 64), dtype=torch.float16, device=cuda), tr, 4, 0)
