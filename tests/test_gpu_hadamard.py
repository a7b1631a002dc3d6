"""Hadamard-128 kernels against the oracle (fp32 butterflies on the GPU, exact
double sums in the oracle: equal up to an fp16 ulp on rare elements)."""
import numpy as np
import pytest
import torch

from conftest import rel_l2

pytestmark = pytest.mark.gpu
TOL = 1e-3  # rel-L2 bar for floating-point outputs


def _t(a, device):
    return torch.from_numpy(np.ascontiguousarray(a)).to(device)


def test_pre_matches_oracle(cuda, oracle):
    from ponyexl3_amd import ops

    rng = np.random.default_rng(0)
    x = rng.standard_normal((5, 640)).astype(np.float16)
    suh = (np.where(rng.random(640) > 0.5, -1, 1) * rng.uniform(0.5, 2, 640)).astype(np.float16)
    got = ops.had128_pre(_t(x, cuda), _t(suh, cuda)).cpu().numpy()
    ref = oracle.had_r_128(x.astype(np.float32), pre_scale=suh).astype(np.float16)
    assert got.shape == ref.shape
    assert rel_l2(got, ref) < 3e-4
    assert (got.view(np.uint16) != ref.view(np.uint16)).mean() < 0.01
    plain = ops.had128_pre(_t(x, cuda), None).cpu().numpy()
    assert rel_l2(plain, oracle.had_r_128(x.astype(np.float32))) < 3e-4


def test_pre_stacked_suh(cuda, oracle):
    from ponyexl3_amd import ops

    rng = np.random.default_rng(1)
    x = rng.standard_normal((3, 256)).astype(np.float16)
    suh = np.where(rng.random((4, 256)) > 0.5, -1, 1).astype(np.float16)
    got = ops.had128_pre(_t(x, cuda), _t(suh, cuda)).cpu().numpy()
    assert got.shape == (3, 4, 256)
    for s in range(4):
        ref = oracle.had_r_128(x.astype(np.float32), pre_scale=suh[s]).astype(np.float16)
        assert rel_l2(got[:, s], ref) < 3e-4


def test_post_fp16_and_split_sum(cuda, oracle):
    from ponyexl3_amd import ops

    rng = np.random.default_rng(2)
    parts = (rng.standard_normal((3, 4, 384)) * 20).astype(np.float32)
    svh = np.where(rng.random(384) > 0.5, -1, 1).astype(np.float16)
    bias = (rng.standard_normal(384) * 0.1).astype(np.float16)
    total = ((parts[0] + parts[1]) + parts[2]).astype(np.float16)  # index order, fp32, then fp16
    ref = oracle.had_r_128(total.astype(np.float32), post_scale=svh).astype(np.float16)
    got = ops.had128_post(_t(parts, cuda), _t(svh, cuda)).cpu().numpy()
    assert rel_l2(got, ref) < 3e-4
    got16 = ops.had128_post(_t(total, cuda), _t(svh, cuda)).cpu().numpy()
    np.testing.assert_array_equal(got16.view(np.uint16), got.view(np.uint16))
    gotb = ops.had128_post(_t(total, cuda), _t(svh, cuda), _t(bias, cuda)).cpu().numpy()
    np.testing.assert_array_equal(gotb.view(np.uint16), (got16 + bias).view(np.uint16))


def test_wide_and_narrow_kernels_give_the_same_bits(cuda, oracle):
    """From 16 rows on a workgroup walks along a row with 16-byte accesses; below,
    one wave takes one block. Same butterflies in the same order: same bits."""
    from ponyexl3_amd import ops

    rng = np.random.default_rng(4)
    x = (rng.standard_normal((40, 640)) * 3).astype(np.float16)
    suh = (np.where(rng.random((3, 640)) > 0.5, -1, 1) * rng.uniform(0.5, 2, (3, 640))).astype(np.float16)
    svh = (np.where(rng.random(640) > 0.5, -1, 1) * rng.uniform(0.5, 2, 640)).astype(np.float16)
    bias = (rng.standard_normal(640) * 0.1).astype(np.float16)
    xt, st, vt, bt = _t(x, cuda), _t(suh, cuda), _t(svh, cuda), _t(bias, cuda)
    wide = ops.had128_pre(xt, st)  # 120 (row, sub) pairs: wide kernel
    narrow = torch.cat([ops.had128_pre(xt[r:r + 5].contiguous(), st) for r in range(0, 40, 5)])
    assert torch.equal(wide, narrow)
    ref = oracle.had_r_128(x.astype(np.float32), pre_scale=suh[1]).astype(np.float16)
    assert rel_l2(wide[:, 1].cpu().numpy(), ref) < 3e-4
    wide = ops.had128_post(xt, vt, bt)
    narrow = torch.cat([ops.had128_post(xt[r:r + 8].contiguous(), vt, bt) for r in range(0, 40, 8)])
    assert torch.equal(wide, narrow)
    ref = oracle.had_r_128(x.astype(np.float32), post_scale=svh).astype(np.float16)
    assert rel_l2(ops.had128_post(xt, vt).cpu().numpy(), ref) < 3e-4


def test_involution_at_scale(cuda):
    """Size-independent property at prefill size: H(H(x)) == x, norms preserved."""
    from ponyexl3_amd import ops

    g = torch.Generator(device="cpu").manual_seed(3)
    x = torch.randn((2048, 5120), generator=g).to(torch.float16).to(cuda)
    y = ops.had128_pre(x, None)
    z = ops.had128_post(y, None)
    assert rel_l2(z.float().cpu().numpy(), x.float().cpu().numpy()) < TOL
    nx = x.float().norm(dim=1)
    ny = y.float().norm(dim=1)
    assert float(((nx - ny).abs() / nx).max()) < TOL


def test_row_tables_out_of_range_are_skipped(cuda, oracle):
    """exl3_had128_rows takes its gather / scatter tables from caller memory: an entry
    outside the buffer it indexes (negative included) makes the kernel skip that row;
    the other rows come out as usual and nothing outside the buffers is touched."""
    import ctypes

    from ponyexl3_amd import _lib

    rng = np.random.default_rng(12)
    x = rng.standard_normal((6, 256)).astype(np.float16)
    scale = np.where(rng.random((3, 256)) > 0.5, -1.0, 1.0).astype(np.float16)
    in_index = np.array([0, 5, 6, -1, 2, 3], dtype=np.int32)       # 6 and -1 are out of range
    scale_index = np.array([0, 1, 2, 0, 3, 2], dtype=np.int32)     # 3 is out of range
    out_index = np.array([0, 1, 2, 3, 4, 9], dtype=np.int32)       # 9 is out of range
    xt, st = torch.from_numpy(x).to(cuda), torch.from_numpy(scale).to(cuda)
    ii, si, oi = (torch.from_numpy(a).to(cuda) for a in (in_index, scale_index, out_index))
    out = torch.full((6, 256), 777.0, dtype=torch.float16, device=cuda)
    p = lambda t: ctypes.c_void_p(t.data_ptr())
    lib = _lib.load()
    rc = lib.exl3_had128_rows(p(xt), 6, 6, 256, p(ii), p(st), 3, p(si), 256, 0, p(out), 6, p(oi),
                              ctypes.c_void_p(torch.cuda.current_stream().cuda_stream))
    assert rc == 0
    torch.cuda.synchronize()
    got = out.cpu().numpy()
    for r in (0, 1):  # the two rows whose three indices are all valid
        want = oracle.had_r_128(x[in_index[r]][None].astype(np.float32),
                                pre_scale=scale[scale_index[r]]).astype(np.float16)[0]
        np.testing.assert_array_equal(got[out_index[r]], want)
    assert (got[2:] == np.float16(777.0)).all()
    # identity maps longer than their buffers are refused on the host
    rc = lib.exl3_had128_rows(p(xt), 4, 6, 256, None, p(st), 3, p(si), 256, 0, p(out), 6, None,
                              ctypes.c_void_p(torch.cuda.current_stream().cuda_stream))
    assert rc == _lib.EXL3_E_BAD_SHAPE


def test_errors(cuda):
    from ponyexl3_amd import ops

    with pytest.raises(ValueError):
        ops.had128_pre(torch.zeros((1, 100), dtype=torch.float16, device=cuda), None)
    with pytest.raises(ValueError):
        ops.had128_pre(torch.zeros((1, 128), dtype=torch.float32, device=cuda), None)
    with pytest.raises(ValueError):
        ops.had128_post(torch.zeros((1, 128), dtype=torch.float16, device=cuda),
                        torch.zeros(64, dtype=torch.float16, device=cuda))
