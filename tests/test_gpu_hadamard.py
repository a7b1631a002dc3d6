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


def test_errors(cuda):
    from ponyexl3_amd import ops

    with pytest.raises(ValueError):
        ops.had128_pre(torch.zeros((1, 100), dtype=torch.float16, device=cuda), None)
    with pytest.raises(ValueError):
        ops.had128_pre(torch.zeros((1, 128), dtype=torch.float32, device=cuda), None)
    with pytest.raises(ValueError):
        ops.had128_post(torch.zeros((1, 128), dtype=torch.float16, device=cuda),
                        torch.zeros(64, dtype=torch.float16, device=cuda))
