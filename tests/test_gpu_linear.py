"""EXL3Linear / FusedEXL3Group against the oracle's layer forward
(rel-L2 <= 1e-3, fp32 accumulation)."""
import os

import numpy as np
import pytest
import torch

from conftest import golden, rel_l2

pytestmark = pytest.mark.gpu
TOL = 1e-3


def _x(rng, shape, device):
    x = rng.standard_normal(shape).astype(np.float16)
    return x, torch.from_numpy(x).to(device)


def _oracle_forward(oracle, layer, x):
    return oracle.linear_forward(layer.trellis, layer.k, layer.codebook_mode, layer.suh, layer.svh, x,
                                 bias=layer.bias)


def _golden_cases():
    g = golden("forwards.npz")
    return sorted({n[:-2] for n in g.files if n.endswith("_y")})


@pytest.mark.parametrize("tag", _golden_cases())
def test_golden_forward_outputs(cuda, tag):
    """Outputs written by the reference's linear_forward_reconstruct."""
    from ponyexl3_amd import EXL3Layer, EXL3Linear

    g = golden("forwards.npz")
    k = int(tag[1])
    cb = int(tag.split("_")[1][2])
    suh, svh = g[tag + "_suh"], g[tag + "_svh"]
    if not tag.endswith("_bf"):
        suh, svh = suh.view(np.float16), svh.view(np.float16)
    bias = g[tag + "_bias"].view(np.float16) if tag + "_bias" in g.files else None
    layer = EXL3Layer(tag, 128, 256, k, g[tag + "_trellis"], suh, svh, bias, mcg=cb == 1, mul1=cb == 2)
    x = torch.from_numpy(g[tag + "_x"].view(np.float16)).to(cuda)
    y = EXL3Linear(layer)(x).cpu().numpy()
    assert rel_l2(y, g[tag + "_y"].view(np.float16)) <= TOL


@pytest.mark.parametrize("rows", [1, 4, 8, 16, 19, 300])
@pytest.mark.parametrize("k,mcg", [(2, True), (4, True), (4, False), (6, False)])
def test_module_matches_oracle(cuda, oracle, rows, k, mcg):
    from ponyexl3_amd import EXL3Linear, make_exl3_layer

    layer = make_exl3_layer(k=k, in_features=256, out_features=384, seed=11 + k, mcg=mcg, bias=True)
    rng = np.random.default_rng(rows)
    x, xt = _x(rng, (rows, 256), cuda)
    print(f"linear rows={rows} k={k} mcg={mcg}", flush=True)
    y = EXL3Linear(layer)(xt).cpu().numpy()
    assert y.dtype == np.float16 and y.shape == (rows, 384)
    assert rel_l2(y, _oracle_forward(oracle, layer, x)) <= TOL


@pytest.mark.parametrize("k", [1, 2, 3, 4, 5, 6, 7, 8])
@pytest.mark.parametrize("cb", [0, 1, 2])
def test_every_k_codebook_and_row_count(cuda, oracle, k, cb):
    """Every bit width, codebook and small-batch row count (each row count up to 8
    is its own instruction schedule in the one-launch kernel), row counts of the
    medium-batch kernel (9..32 rows; 70 rows are prefill), both launch
    plans, against the oracle."""
    from ponyexl3_amd import make_exl3_layer, ops

    layer = make_exl3_layer(k=k, in_features=256, out_features=256, seed=300 + 10 * k + cb,
                            mcg=cb == 1, mul1=cb == 2, bias=True)
    tr = ops.as_trellis_tensor(layer.trellis, cuda)
    suh, svh = torch.from_numpy(layer.suh).to(cuda), torch.from_numpy(layer.svh).to(cuda)
    bias = torch.from_numpy(layer.bias).to(cuda)
    rng = np.random.default_rng(k * 3 + cb)
    for rows in (1, 2, 3, 4, 5, 6, 7, 8, 9, 12, 16, 17, 31, 70):
        x, xt = _x(rng, (rows, 256), cuda)
        ref = _oracle_forward(oracle, layer, x)
        print(f"k={k} cb={cb} rows={rows}", flush=True)
        y = ops.linear_forward(xt, tr, k, cb, suh, svh, bias, fused=True).cpu().numpy()
        assert rel_l2(y, ref) <= TOL, f"one-launch rows={rows}"
        # the launch chain (up to 8 rows) / the prefill GEMM (from 9 rows on)
        y = ops.linear_forward(xt, tr, k, cb, suh, svh, bias, fused=False).cpu().numpy()
        assert rel_l2(y, ref) <= TOL, f"chain rows={rows}"


def test_general_scales_not_only_signs(cuda, oracle):
    from ponyexl3_amd import EXL3Linear, make_exl3_layer

    rng = np.random.default_rng(21)
    suh = (np.where(rng.random(256) > 0.5, -1, 1) * rng.uniform(0.25, 1.5, 256)).astype(np.float16)
    svh = (np.where(rng.random(128) > 0.5, -1, 1) * rng.uniform(0.0, 2.0, 128)).astype(np.float16)
    svh[:5] = 0  # dead columns
    layer = make_exl3_layer(k=4, in_features=256, out_features=128, seed=3, suh=suh, svh=svh, mcg=True)
    x, xt = _x(rng, (2, 256), cuda)
    y = EXL3Linear(layer)(xt).cpu().numpy()
    assert rel_l2(y, _oracle_forward(oracle, layer, x)) <= TOL
    assert (y[:, :5] == 0).all()


def test_module_keeps_leading_shape_and_has_no_parameters(cuda):
    from ponyexl3_amd import EXL3Linear, make_exl3_layer

    mod = EXL3Linear(make_exl3_layer(k=4, in_features=128, out_features=128, seed=3))
    x = torch.zeros((2, 3, 128), dtype=torch.float16, device=cuda)
    assert tuple(mod(x).shape) == (2, 3, 128)
    assert list(mod.parameters()) == [] and list(mod.buffers()) == []
    assert mod.state_dict() == {}
    assert mod.in_features == 128 and mod.out_features == 128
    mod.warm().release_source()
    assert tuple(mod(x).shape) == (2, 3, 128)
    with pytest.raises(ValueError):
        mod(torch.zeros((1, 64), dtype=torch.float16, device=cuda))


def test_config1_layer(cuda, oracle):
    """4096 -> 4096, K=4, 3INST, x [1, 4096] ~ N(0, 1)."""
    from ponyexl3_amd import EXL3Linear, make_exl3_layer

    layer = make_exl3_layer(k=4, in_features=4096, out_features=4096, seed=10_004)
    rng = np.random.default_rng(1)
    x, xt = _x(rng, (1, 4096), cuda)
    y = EXL3Linear(layer)(xt).cpu().numpy()
    assert rel_l2(y, _oracle_forward(oracle, layer, x)) <= TOL


@pytest.mark.parametrize("name,n_in,n_out", [("q_proj", 5120, 8192), ("k_proj", 5120, 1024),
                                             ("o_proj", 8192, 5120), ("down_proj", 17408, 5120)])
def test_config2_shapes_bs1(cuda, oracle, name, n_in, n_out):
    from ponyexl3_amd import EXL3Linear, make_exl3_layer

    layer = make_exl3_layer(k=4, in_features=n_in, out_features=n_out, seed=20_004)
    rng = np.random.default_rng(2)
    x, xt = _x(rng, (1, n_in), cuda)
    print(f"config2 {name}", flush=True)
    y = EXL3Linear(layer)(xt).cpu().numpy()
    ref = oracle.linear_forward_bs1(layer.trellis, 4, 0, layer.suh, layer.svh, x[0])
    assert rel_l2(y[0], ref) <= TOL


@pytest.mark.parametrize("name,n_in,n_out", [("k_proj", 5120, 1024), ("o_proj", 8192, 5120)])
def test_config2_shapes_medium_batch(cuda, name, n_in, n_out):
    """Config-2 shapes at 16 and 32 rows (batched decode): the medium-batch kernel
    with its real split counts against the prefill GEMM on the same input (both
    oracle-checked at small sizes; same fp32 products, other cut points) and, row by
    row, against the one-row kernel (linearity of the layer in its batch rows)."""
    from ponyexl3_amd import make_exl3_layer, ops

    layer = make_exl3_layer(k=4, in_features=n_in, out_features=n_out, seed=20_016)
    tr = ops.as_trellis_tensor(layer.trellis, cuda)
    suh, svh = torch.from_numpy(layer.suh).to(cuda), torch.from_numpy(layer.svh).to(cuda)
    rng = np.random.default_rng(16)
    for rows in (16, 32):
        _, xt = _x(rng, (rows, n_in), cuda)
        print(f"config2 {name} rows={rows}", flush=True)
        a = ops.linear_forward(xt, tr, 4, 0, suh, svh, fused=True)
        b = ops.linear_forward(xt, tr, 4, 0, suh, svh, fused=False)
        scale = float(b.float().abs().max())
        assert float((a.float() - b.float()).abs().max()) <= 2e-3 * scale
        for r in (0, rows - 1):
            one = ops.linear_forward(xt[r : r + 1].contiguous(), tr, 4, 0, suh, svh, fused=True)
            assert float((a[r : r + 1].float() - one.float()).abs().max()) <= 2e-3 * scale
    assert int(ops.sync_counters(cuda, 1).abs().sum()) == 0


@pytest.mark.parametrize("rows", [1, 8, 11, 16, 19])
def test_fused_group_matches_members(cuda, oracle, rows):
    from ponyexl3_amd import EXL3Linear, FusedEXL3Group, make_exl3_layer

    layers = [make_exl3_layer(k=4, in_features=256, out_features=o, seed=70 + i, mcg=True, key=f"f{i}")
              for i, o in enumerate((384, 256, 128))]
    group = FusedEXL3Group(layers)
    rng = np.random.default_rng(rows)
    x, xt = _x(rng, (rows, 256), cuda)
    outs = group.forward_all(xt)
    for o, l in zip(outs, layers):
        assert tuple(o.shape) == (rows, l.out_features)
        assert rel_l2(o.cpu().numpy(), _oracle_forward(oracle, l, x)) <= TOL
        member = EXL3Linear(l)(xt)  # tests/test_exl3_fused.py:32-48: max-rel < 5e-3
        got, ref = o.float().cpu().numpy(), member.float().cpu().numpy()
        assert np.abs(got - ref).max() / (np.abs(ref).max() + 1e-9) < 5e-3


def test_fused_gate_up_config2(cuda, oracle):
    """gate/up 5120 -> 17408 sibling-fused at batch 1."""
    from ponyexl3_amd import FusedEXL3Group, make_exl3_layer

    gate = make_exl3_layer(k=4, in_features=5120, out_features=17408, seed=20_104, key="gate")
    up = make_exl3_layer(k=4, in_features=5120, out_features=17408, seed=20_204, key="up")
    group = FusedEXL3Group([gate, up])
    rng = np.random.default_rng(3)
    x, xt = _x(rng, (1, 5120), cuda)
    g_out, u_out = group.forward_all(xt)
    for o, l in ((g_out, gate), (u_out, up)):
        ref = oracle.linear_forward_bs1(l.trellis, 4, 0, l.suh, l.svh, x[0])
        assert rel_l2(o.cpu().numpy()[0], ref) <= TOL


def test_single_slot_cache_computes_once(cuda):
    from ponyexl3_amd import FusedEXL3Group, make_exl3_layer

    layers = [make_exl3_layer(k=4, in_features=256, out_features=128, seed=80 + i, key=f"c{i}") for i in range(2)]
    group = FusedEXL3Group(layers)
    s0, s1 = group.sibling(0), group.sibling(1)
    calls = {"n": 0}
    orig = group.forward_all

    def counting(x):
        calls["n"] += 1
        return orig(x)

    group.forward_all = counting
    x = torch.zeros((1, 256), dtype=torch.float16, device=cuda)
    s0(x)
    s1(x)
    assert calls["n"] == 1
    s0(torch.zeros((1, 256), dtype=torch.float16, device=cuda))
    assert calls["n"] == 2
    assert s0.out_features == 128 and s0.in_features == 256


def test_sibling_cache_sees_in_place_updates(cuda):
    """A static input buffer refilled in place between two decode steps must not be
    served the previous step's outputs, and the cache holds nothing once every
    member has read it."""
    from ponyexl3_amd import EXL3Linear, FusedEXL3Group, make_exl3_layer

    layers = [make_exl3_layer(k=4, in_features=256, out_features=128, seed=90 + i, key=f"v{i}") for i in range(2)]
    group = FusedEXL3Group(layers)
    s0, s1 = group.sibling(0), group.sibling(1)
    x = torch.randn((1, 256), device=cuda).half()
    a0 = s0(x).clone()
    x.copy_(torch.randn((1, 256), device=cuda).half())  # same tensor object, new values
    b1 = s1(x)
    assert torch.equal(b1, EXL3Linear(layers[1])(x))
    b0 = s0(x)
    assert torch.equal(b0, EXL3Linear(layers[0])(x)) and not torch.equal(a0, b0)
    assert group._cache_out is None and group._cache_key is None  # both members served


def test_bounded_wait_gives_up_visibly(cuda, monkeypatch):
    """The finishing workgroup of the accumulator reduction waits a bounded number of
    polls for the other workgroups' adds. With an accumulator pre-seeded so that its
    count can never come out right and the bound lowered through EXL3_SPIN_LIMIT, every
    kernel still exits, the affected 128-column group is NaN, the other groups are
    untouched, exl3_counters_status reports it, and after zeroing the array the next
    call is right again."""
    from ponyexl3_amd import make_exl3_layer, ops

    if os.environ.get("EXL3_EXACT_WEIGHTS") == "1":
        pytest.skip("the multi-launch chains this knob selects have no accumulator reduction")
    layer = make_exl3_layer(k=4, in_features=1024, out_features=384, seed=97)
    tr = ops.as_trellis_tensor(layer.trellis, cuda)
    suh, svh = torch.from_numpy(layer.suh).to(cuda), torch.from_numpy(layer.svh).to(cuda)
    xt = torch.randn((2, 1024), device=cuda).half()
    good = ops.linear_forward(xt, tr, 4, 0, suh, svh, fused=True)
    ops.check_counters(cuda)
    cnt = ops.sync_counters(cuda, 1)
    try:
        # accumulator of (row 0, column 128 + 5): a count of 255 before anybody has added
        cnt.view(torch.int64)[128 + 5] = -(1 << 56)
        monkeypatch.setenv("EXL3_SPIN_LIMIT", "4")
        print("linear bounded wait", flush=True)
        bad = ops.linear_forward(xt, tr, 4, 0, suh, svh, fused=True)
        torch.cuda.synchronize()
        assert torch.isnan(bad[:, 128:256].float()).all()
        assert torch.equal(bad[:, :128], good[:, :128]) and torch.equal(bad[:, 256:], good[:, 256:])
        with pytest.raises(RuntimeError):
            ops.check_counters(cuda)
        monkeypatch.delenv("EXL3_SPIN_LIMIT")
        assert torch.equal(ops.linear_forward(xt, tr, 4, 0, suh, svh, fused=True), good)
        ops.check_counters(cuda)
    finally:
        torch.cuda.synchronize()
        cnt.zero_()  # whatever happened above, the shared array is clean for the next test


def test_sibling_cache_under_inference_mode(cuda):
    """Tensors made under torch.inference_mode() have no version counter; the sibling
    cache must still work there, and a buffer refilled in place between two steps
    must not be served the previous step's outputs."""
    from ponyexl3_amd import EXL3Linear, FusedEXL3Group, make_exl3_layer

    layers = [make_exl3_layer(k=4, in_features=256, out_features=128, seed=95 + i, key=f"i{i}") for i in range(2)]
    group = FusedEXL3Group(layers)
    s0, s1 = group.sibling(0), group.sibling(1)
    with torch.inference_mode():
        x = torch.randn((1, 256), device=cuda).half()
        assert x.is_inference()
        a0, a1 = s0(x).clone(), s1(x).clone()
        assert torch.equal(a0, EXL3Linear(layers[0])(x)) and torch.equal(a1, EXL3Linear(layers[1])(x))
        x.copy_(torch.randn((1, 256), device=cuda).half())  # same tensor object, new values
        b0, b1 = s0(x), s1(x)
        assert torch.equal(b0, EXL3Linear(layers[0])(x)) and not torch.equal(a0, b0)
        assert torch.equal(b1, EXL3Linear(layers[1])(x))
        # a step that asks only one member: the next step's request for it recomputes
        c0 = s0(x).clone()
        x.copy_(torch.randn((1, 256), device=cuda).half())
        d0 = s0(x)
        assert torch.equal(d0, EXL3Linear(layers[0])(x)) and not torch.equal(c0, d0)


CONFIG3_LAUNCHES = [
    ("qkv", 5120, (8192, 1024, 1024)),
    ("o_proj", 8192, (5120,)),
    ("gate_up", 5120, (17408, 17408)),
    ("down_proj", 17408, (5120,)),
]


@pytest.mark.parametrize("name,n_in,outs", CONFIG3_LAUNCHES)
def test_config3_whole_layer_against_oracle(cuda, oracle, name, n_in, outs):
    """M = 2048 through the path a caller uses (ponyexl3/mlx/exl3_linear.py:137-161):
    rotation, the prefill GEMM (sibling groups as one launch with a per-block member
    table, split tiles and their completion), output Hadamard and svh, on the four
    launches of a 27B-class decoder layer. 24 rows spread over the row blocks are
    compared with the oracle's forward of each member (rel-L2 <= 1e-3)."""
    from ponyexl3_amd import EXL3Linear, FusedEXL3Group, make_exl3_layer

    members = [make_exl3_layer(k=4, in_features=n_in, out_features=o, seed=30_000 + 10 * i + len(name),
                               key=f"{name}{i}") for i, o in enumerate(outs)]
    rng = np.random.default_rng(len(name))
    x = rng.standard_normal((2048, n_in)).astype(np.float16)
    xt = torch.from_numpy(x).to(cuda)
    print(f"config3 layer {name}", flush=True)
    if len(members) > 1:
        ys = FusedEXL3Group(members, cuda).forward_all(xt)
    else:
        ys = (EXL3Linear(members[0], cuda)(xt),)
    sample = np.unique(np.concatenate([np.arange(0, 2048, 128), np.arange(2047, 0, -293)]))
    assert len(sample) >= 16
    for y, m in zip(ys, members):
        assert tuple(y.shape) == (2048, m.out_features)
        ref = oracle.linear_forward(m.trellis, 4, 0, m.suh, m.svh, x[sample])
        got = y.cpu().numpy()[sample]
        assert rel_l2(got, ref) <= TOL
        worst_row = max(rel_l2(got[i], ref[i]) for i in range(len(sample)))
        assert worst_row <= 2e-3


@pytest.mark.parametrize("rows", [1, 3, 8, 13, 16])
@pytest.mark.parametrize("k,n_in,n_out", [(4, 512, 384), (3, 1024, 256), (6, 2176, 640), (4, 5120, 1024)])
def test_one_launch_layer_equals_three_launch_chain(cuda, rows, k, n_in, n_out):
    """The fused kernel (rotation + GEMV + last-wave reduction + output transform;
    from 9 rows on the medium-batch kernel behind a rotation launch) against the
    chained kernels (from 9 rows on the prefill GEMM). Both add the same fp32 products, but cut the
    reduction dimension at different tile rows, so the sums can differ in the last
    fp32 bit and, rarely, flip an fp16 rounding before the output Hadamard: they
    must agree to a few fp16 ulps of the largest output. The fused kernel must be
    bit-identical call after call (fixed sum order; its group counters have to
    come back to zero every time)."""
    from ponyexl3_amd import make_exl3_layer, ops

    layer = make_exl3_layer(k=k, in_features=n_in, out_features=n_out, seed=k + n_in, bias=True)
    tr = ops.as_trellis_tensor(layer.trellis, cuda)
    suh = torch.from_numpy(layer.suh).to(cuda)
    svh = torch.from_numpy(layer.svh).to(cuda)
    bias = torch.from_numpy(layer.bias).to(cuda)
    rng = np.random.default_rng(rows)
    for rep in range(3):
        x = torch.from_numpy(rng.standard_normal((rows, n_in)).astype(np.float16)).to(cuda)
        a = ops.linear_forward(x, tr, k, 0, suh, svh, bias, fused=True)
        a2 = ops.linear_forward(x, tr, k, 0, suh, svh, bias, fused=True)
        b = ops.linear_forward(x, tr, k, 0, suh, svh, bias, fused=False)
        assert torch.equal(a, a2), f"rep {rep}"
        diff = float((a.float() - b.float()).abs().max())
        assert diff <= 2e-3 * float(b.float().abs().max()), f"rep {rep}: {diff}"
    assert int(ops.sync_counters(cuda, 1).abs().sum()) == 0


@pytest.mark.parametrize("seed", range(14))
def test_random_shapes_all_paths_agree(cuda, oracle, seed):
    """Random layers (1..40 Hadamard blocks in, 1..24 out, K = 1..8, three codebooks, with
    and without bias) at random row counts up to 40: whatever kernel the library picks
    with counters (accumulator or partial-row reduction, half-block or two-block splits,
    eight-wave workgroups, medium-batch kernel, prefill GEMM) against the chained kernels
    without counters and against the oracle; bit-identical call after call."""
    from ponyexl3_amd import make_exl3_layer, ops

    rng = np.random.default_rng(7000 + seed)
    n_in, n_out = 128 * int(rng.integers(1, 41)), 128 * int(rng.integers(1, 25))
    k, cb = int(rng.integers(1, 9)), int(rng.integers(0, 3))
    rows = int(rng.choice([1, 1, 2, 3, 5, 8, 9, 16, 27, 40]))
    has_bias = bool(rng.integers(0, 2))
    layer = make_exl3_layer(k=k, in_features=n_in, out_features=n_out, seed=seed, mcg=cb == 1, mul1=cb == 2,
                            bias=has_bias)
    tr = ops.as_trellis_tensor(layer.trellis, cuda)
    suh, svh = torch.from_numpy(layer.suh).to(cuda), torch.from_numpy(layer.svh).to(cuda)
    bias = torch.from_numpy(layer.bias).to(cuda) if has_bias else None
    xn = rng.standard_normal((rows, n_in)).astype(np.float16)
    x = torch.from_numpy(xn).to(cuda)
    print(f"linear random seed={seed} {n_in}x{n_out} k={k} cb={cb} rows={rows} bias={has_bias}", flush=True)
    a = ops.linear_forward(x, tr, k, cb, suh, svh, bias, fused=True)
    assert torch.equal(a, ops.linear_forward(x, tr, k, cb, suh, svh, bias, fused=True))
    assert int(ops.sync_counters(cuda, 1).abs().sum()) == 0
    b = ops.linear_forward(x, tr, k, cb, suh, svh, bias, fused=False)
    want = oracle.linear_forward(layer.trellis, k, cb, layer.suh, layer.svh, xn,
                                 bias=layer.bias if has_bias else None)
    assert rel_l2(a.cpu().numpy(), want) <= 1e-3
    assert rel_l2(b.cpu().numpy(), want) <= 1e-3


@pytest.mark.parametrize("rows", [9, 13, 16, 17, 25, 32])
@pytest.mark.parametrize("k,cb,n_in,n_out", [(4, 0, 2176, 640), (3, 1, 4096, 384), (5, 0, 1024, 1280),
                                             (8, 2, 1152, 256), (7, 0, 640, 128), (6, 1, 2048, 256),
                                             (2, 0, 1536, 384), (1, 0, 1024, 256), (4, 1, 128, 128)])
def test_medium_batch_kernel(cuda, oracle, rows, k, cb, n_in, n_out):
    """9..32 rows with counters: rotation launch, then the kernel whose lanes own the
    tensor-core fragments of the trellis format and feed them to 16x16x32 MFMA from
    registers; the reduction is cut into splits of unequal length that meet through
    partial rows and the group counters. Against the oracle, against
    the prefill GEMM on the same input (same fp32 products, other cut points), and
    bit-identical twice in a row with the counters back at zero."""
    from ponyexl3_amd import make_exl3_layer, ops

    assert ops.linear_small_max_rows() >= 32
    layer = make_exl3_layer(k=k, in_features=n_in, out_features=n_out, seed=40 * k + cb + rows,
                            mcg=cb == 1, mul1=cb == 2, bias=True)
    tr = ops.as_trellis_tensor(layer.trellis, cuda)
    suh, svh = torch.from_numpy(layer.suh).to(cuda), torch.from_numpy(layer.svh).to(cuda)
    bias = torch.from_numpy(layer.bias).to(cuda)
    rng = np.random.default_rng(rows + k)
    x, xt = _x(rng, (rows, n_in), cuda)
    print(f"medium batch rows={rows} k={k} cb={cb} {n_in}->{n_out}", flush=True)
    a = ops.linear_forward(xt, tr, k, cb, suh, svh, bias, fused=True)
    a2 = ops.linear_forward(xt, tr, k, cb, suh, svh, bias, fused=True)
    assert torch.equal(a, a2)
    assert int(ops.sync_counters(cuda, 1).abs().sum()) == 0
    assert rel_l2(a.cpu().numpy(), _oracle_forward(oracle, layer, x)) <= TOL
    b = ops.linear_forward(xt, tr, k, cb, suh, svh, bias, fused=False)
    diff = float((a.float() - b.float()).abs().max())
    assert diff <= 2e-3 * float(b.float().abs().max())


@pytest.mark.parametrize("rows", [12, 20, 32])
def test_medium_batch_kernel_sibling_group(cuda, oracle, rows):
    """Stacked siblings (each 128-column group reads its member's rotation) through
    the medium-batch kernel, members of 384, 256 and 128 columns."""
    from ponyexl3_amd import FusedEXL3Group, make_exl3_layer

    layers = [make_exl3_layer(k=4, in_features=1280, out_features=o, seed=270 + i, key=f"m{i}")
              for i, o in enumerate((384, 256, 128))]
    group = FusedEXL3Group(layers)
    rng = np.random.default_rng(rows)
    x, xt = _x(rng, (rows, 1280), cuda)
    print(f"medium batch siblings rows={rows}", flush=True)
    for o, l in zip(group.forward_all(xt), layers):
        assert tuple(o.shape) == (rows, l.out_features)
        assert rel_l2(o.cpu().numpy(), _oracle_forward(oracle, l, x)) <= TOL


@pytest.mark.parametrize("rows", [17, 33, 64, 100, 130])
@pytest.mark.parametrize("k,n_in,n_out", [(4, 2176, 640), (3, 4096, 384), (5, 1024, 1280)])
def test_prefill_rows_with_every_tile_split(cuda, oracle, rows, k, n_in, n_out):
    """Few rows and few column blocks: every GEMM tile is split along the reduction
    dimension and the pass that adds the partial tiles also applies the output
    Hadamard, svh and bias. 640 and 384 columns end in a half-width block. Checked
    against the oracle and against the separate GEMM + output-transform launches."""
    from ponyexl3_amd import make_exl3_layer, ops

    layer = make_exl3_layer(k=k, in_features=n_in, out_features=n_out, seed=3 * k + rows, mcg=True, bias=True)
    cb = int(layer.codebook_mode)
    tr = ops.as_trellis_tensor(layer.trellis, cuda)
    suh, svh = torch.from_numpy(layer.suh).to(cuda), torch.from_numpy(layer.svh).to(cuda)
    bias = torch.from_numpy(layer.bias).to(cuda)
    rng = np.random.default_rng(rows + n_in)
    x, xt = _x(rng, (rows, n_in), cuda)
    print(f"split prefill rows={rows} k={k} {n_in}->{n_out}", flush=True)
    y = ops.linear_forward(xt, tr, k, cb, suh, svh, bias, fused=False)
    assert rel_l2(y.cpu().numpy(), _oracle_forward(oracle, layer, x)) <= TOL
    parts = ops.had128_post(ops.inner_gemm(ops.had128_pre(xt, suh), tr, k, cb), svh, bias)
    assert torch.equal(y, parts)


@pytest.mark.parametrize("rows", [17, 40, 300])
def test_sibling_prefill_in_one_gemm_launch(cuda, oracle, rows):
    """Members that end on 256-column blocks go through one GEMM launch in which
    every block reads its own member's rotation; same result as member by member
    (the path for members that do not end on block boundaries) and as the oracle."""
    from ponyexl3_amd import FusedEXL3Group, make_exl3_layer, ops

    layers = [make_exl3_layer(k=4, in_features=1024, out_features=o, seed=170 + i, mcg=True, key=f"s{i}")
              for i, o in enumerate((512, 256, 256))]
    group = FusedEXL3Group(layers)
    assert group._block_sub is not None
    rng = np.random.default_rng(rows)
    x, xt = _x(rng, (rows, 1024), cuda)
    print(f"sibling prefill rows={rows}", flush=True)
    outs = group.forward_all(xt)
    # fused=False keeps the prefill GEMM also at row counts that the medium-batch
    # kernel would otherwise take
    y_gemm = ops.linear_forward(xt, group._trellis, group._k, group._cb, group._suh_stack, group._svh_cat,
                                None, group._group_sub, fused=False, member_out=group._out_features,
                                block_sub=group._block_sub)
    outs_gemm = torch.split(y_gemm, group._out_features, dim=-1)
    xh = ops.had128_pre(xt, group._suh_stack)
    for i, (o, l) in enumerate(zip(outs, layers)):
        assert rel_l2(o.cpu().numpy(), _oracle_forward(oracle, l, x)) <= TOL
        assert rel_l2(outs_gemm[i].cpu().numpy(), _oracle_forward(oracle, l, x)) <= TOL
        o = outs_gemm[i]
        member = ops.had128_post(ops.inner_gemm(xh[:, i].contiguous(), ops.as_trellis_tensor(l.trellis, cuda),
                                                4, int(l.codebook_mode)),
                                 torch.from_numpy(l.svh).to(cuda))
        assert torch.equal(o, member)
    # 384 columns: not a whole number of blocks -> member-by-member launches
    odd_layers = [make_exl3_layer(k=4, in_features=512, out_features=o, seed=180 + i, key=f"o{i}")
                  for i, o in enumerate((384, 128))]
    odd = FusedEXL3Group(odd_layers)
    assert odd._block_sub is None
    x2, xt2 = _x(rng, (rows, 512), cuda)
    for o, l in zip(odd.forward_all(xt2), odd_layers):
        assert rel_l2(o.cpu().numpy(), _oracle_forward(oracle, l, x2)) <= TOL


def test_two_streams_do_not_share_scratch(cuda):
    """Layers running on two streams of one device at the same time: partial rows and
    group counters are per (device, stream), so both streams get the results they get
    when run alone."""
    from ponyexl3_amd import make_exl3_layer, ops

    la = make_exl3_layer(k=4, in_features=2176, out_features=640, seed=501)
    lb = make_exl3_layer(k=3, in_features=4096, out_features=384, seed=502)
    dev_t = lambda l: (ops.as_trellis_tensor(l.trellis, cuda), torch.from_numpy(l.suh).to(cuda),
                       torch.from_numpy(l.svh).to(cuda))
    ta, tb = dev_t(la), dev_t(lb)
    xa = torch.randn((2, 2176), device=cuda).half()
    xb = torch.randn((1, 4096), device=cuda).half()
    ref_a = ops.linear_forward(xa, ta[0], 4, 0, ta[1], ta[2])
    ref_b = ops.linear_forward(xb, tb[0], 3, 0, tb[1], tb[2])
    torch.cuda.synchronize()
    s1, s2 = torch.cuda.Stream(), torch.cuda.Stream()
    outs_a, outs_b = [], []
    with torch.cuda.stream(s1):
        ws1 = ops.workspace(cuda, 1).data_ptr()
        for _ in range(50):
            outs_a.append(ops.linear_forward(xa, ta[0], 4, 0, ta[1], ta[2]))
    with torch.cuda.stream(s2):
        ws2 = ops.workspace(cuda, 1).data_ptr()
        for _ in range(50):
            outs_b.append(ops.linear_forward(xb, tb[0], 3, 0, tb[1], tb[2]))
    torch.cuda.synchronize()
    assert ws1 != ws2
    assert all(torch.equal(o, ref_a) for o in outs_a)
    assert all(torch.equal(o, ref_b) for o in outs_b)
