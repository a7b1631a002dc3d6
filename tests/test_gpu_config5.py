"""Mixed-bitrate sweep at the 27B-class shapes: K in {2,3,5,6,8} x {3INST, MCG} x
1/2/4/8 rows on o_proj (8192 -> 5120), down_proj (17408 -> 5120), k_proj
(5120 -> 1024), q_proj (5120 -> 8192) and the sibling-fused gate+up launch
(5120 -> 2 x 17408, two rotations of x), the shape list of the reference's own kernel
sweep (tools/bench/gemv_split_bench.py:30-36). Every case goes through the one-launch
layer kernel at its real split counts and is compared with the oracle's forward
(rel-L2 <= 1e-3); one row is also compared with the three-launch chain."""
import numpy as np
import pytest
import torch

from conftest import rel_l2

pytestmark = pytest.mark.gpu
TOL = 1e-3

SHAPES = [("o_proj", 8192, 5120), ("down_proj", 17408, 5120), ("k_proj", 5120, 1024),
          ("q_proj", 5120, 8192)]


@pytest.mark.parametrize("name,n_in,n_out", SHAPES)
@pytest.mark.parametrize("cb", [0, 1])
@pytest.mark.parametrize("k", [2, 3, 5, 6, 8])
def test_config5_shapes_against_oracle(cuda, oracle, k, cb, name, n_in, n_out):
    from ponyexl3_amd import make_exl3_layer, ops

    layer = make_exl3_layer(k=k, in_features=n_in, out_features=n_out, seed=50_000 + 100 * k + cb,
                            mcg=cb == 1)
    tr = ops.as_trellis_tensor(layer.trellis, cuda)
    suh, svh = torch.from_numpy(layer.suh).to(cuda), torch.from_numpy(layer.svh).to(cuda)
    rng = np.random.default_rng(7 * k + cb)
    x = rng.standard_normal((8, n_in)).astype(np.float16)
    xt = torch.from_numpy(x).to(cuda)
    ref = oracle.linear_forward(layer.trellis, k, cb, layer.suh, layer.svh, x)
    for rows in (1, 2, 4, 8):
        print(f"config5 {name} k={k} cb={cb} rows={rows}", flush=True)
        y = ops.linear_forward(xt[:rows].contiguous(), tr, k, cb, suh, svh, fused=True).cpu().numpy()
        assert y.shape == (rows, n_out)
        assert rel_l2(y, ref[:rows]) <= TOL, f"rows={rows}"
    chain = ops.linear_forward(xt[:1].contiguous(), tr, k, cb, suh, svh, fused=False).cpu().numpy()
    assert rel_l2(chain, ref[:1]) <= TOL
    assert int(ops.sync_counters(cuda, 1).abs().sum()) == 0


@pytest.mark.parametrize("cb", [0, 1])
@pytest.mark.parametrize("k", [2, 3, 5, 6, 8])
def test_config5_fused_gate_up_against_oracle(cuda, oracle, k, cb):
    """gate and up (5120 -> 17408 each) as one sibling-fused launch: 2176 tile columns,
    two sign vectors, the launch that takes the eight-wave / two-block plans. Each
    member is compared with the oracle's forward of that member alone."""
    from ponyexl3_amd import FusedEXL3Group, make_exl3_layer

    n_in, n_out = 5120, 17408
    members = [make_exl3_layer(k=k, in_features=n_in, out_features=n_out,
                               seed=51_000 + 100 * k + 10 * cb + i, mcg=cb == 1, key=f"m{i}")
               for i in range(2)]
    group = FusedEXL3Group(members, cuda)
    rng = np.random.default_rng(11 * k + cb)
    x = rng.standard_normal((8, n_in)).astype(np.float16)
    xt = torch.from_numpy(x).to(cuda)
    refs = [oracle.linear_forward(m.trellis, k, cb, m.suh, m.svh, x) for m in members]
    for rows in (1, 4, 8):
        print(f"config5 gate+up k={k} cb={cb} rows={rows}", flush=True)
        outs = group.forward_all(xt[:rows].contiguous())
        for o, ref in zip(outs, refs):
            assert tuple(o.shape) == (rows, n_out)
            assert rel_l2(o.cpu().numpy(), ref[:rows]) <= TOL, f"rows={rows}"
    from ponyexl3_amd import ops

    assert int(ops.sync_counters(cuda, 1).abs().sum()) == 0


def test_config5_lm_head_k6(cuda, oracle):
    """The reference's sweep also lists the K=6 lm_head shape, 320 x 9472 tiles
    (5120 -> 151552, tools/bench/gemv_split_bench.py:35); one row."""
    from ponyexl3_amd import make_exl3_layer, ops

    n_in, n_out = 5120, 9472 * 16
    layer = make_exl3_layer(k=6, in_features=n_in, out_features=n_out, seed=56_000, mcg=True)
    tr = ops.as_trellis_tensor(layer.trellis, cuda)
    suh, svh = torch.from_numpy(layer.suh).to(cuda), torch.from_numpy(layer.svh).to(cuda)
    x = np.random.default_rng(6).standard_normal((1, n_in)).astype(np.float16)
    y = ops.linear_forward(torch.from_numpy(x).to(cuda), tr, 6, 1, suh, svh, fused=True).cpu().numpy()
    ref = oracle.linear_forward_bs1(layer.trellis, 6, 1, layer.suh, layer.svh, x[0])
    assert rel_l2(y[0], ref) <= TOL
