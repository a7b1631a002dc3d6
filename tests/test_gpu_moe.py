"""Routed MoE expert chain against the oracle's unfused per-expert chain."""
import os

import numpy as np
import pytest
import torch

from conftest import rel_l2

pytestmark = pytest.mark.gpu
TOL = 1e-3


def _experts(E, D, H, k, mcg, seed):
    from ponyexl3_amd import make_exl3_layer

    mk = lambda i, n_in, n_out, tag: make_exl3_layer(k=k, in_features=n_in, out_features=n_out,
                                                     seed=seed + i, mcg=mcg, key=f"e{i}.{tag}")
    gate = [mk(3 * e, D, H, "gate") for e in range(E)]
    up = [mk(3 * e + 1, D, H, "up") for e in range(E)]
    down = [mk(3 * e + 2, H, D, "down") for e in range(E)]
    return gate, up, down


def _oracle_chain(oracle, gate, up, down, x, idx, act):
    experts = [{"gate": (g.trellis, g.suh, g.svh), "up": (u.trellis, u.suh, u.svh),
                "down": (d.trellis, d.suh, d.svh)} for g, u, d in zip(gate, up, down)]
    return oracle.moe_experts_forward(experts, x, idx, gate[0].k, gate[0].codebook_mode, act)


@pytest.mark.parametrize("tokens", [1, 3, 8])
@pytest.mark.parametrize("k,mcg,act", [(4, False, "silu"), (3, True, "silu"), (4, True, "gelu")])
def test_moe_matches_oracle(cuda, oracle, tokens, k, mcg, act):
    from ponyexl3_amd import EXL3SwitchGLU

    E, D, H, kk = 6, 256, 128, 2
    gate, up, down = _experts(E, D, H, k, mcg, 500)
    moe = EXL3SwitchGLU.from_layers(gate, up, down, activation=act)
    rng = np.random.default_rng(tokens + k)
    x = (rng.standard_normal((tokens, D)) * 0.5).astype(np.float16)
    idx = np.stack([rng.permutation(E)[:kk] for _ in range(tokens)]).astype(np.int32)
    print(f"moe tokens={tokens} k={k} act={act}", flush=True)
    y = moe(torch.from_numpy(x).to(cuda).reshape(1, tokens, D),
            torch.from_numpy(idx).to(cuda).reshape(1, tokens, kk)).cpu().numpy()
    assert y.shape == (1, tokens, kk, D)
    ref = _oracle_chain(oracle, gate, up, down, x, idx, act)
    assert rel_l2(y[0], ref) <= TOL


@pytest.mark.parametrize("tokens", [1, 8, 48])
def test_two_launch_and_five_launch_chains(cuda, oracle, tokens):
    """D and H of five Hadamard blocks each: both kernels of the two-launch chain
    run two workgroups per column block (one of them with a single active wave)
    and meet through the counters. 1 and 8 tokens take the eight-wave workgroups
    on half blocks, 48 tokens (96 slots) the four-wave ones on whole blocks.
    Checked against the oracle, against the five-launch chain, and twice in a row
    (the counters must be left at zero)."""
    from ponyexl3_amd import EXL3SwitchGLU, ops

    E, D, H, kk, k = 5, 640, 640, 2, 4
    gate, up, down = _experts(E, D, H, k, False, 700)
    moe = EXL3SwitchGLU.from_layers(gate, up, down)
    rng = np.random.default_rng(70 + tokens)
    x = (rng.standard_normal((tokens, D)) * 0.5).astype(np.float16)
    idx = np.stack([rng.permutation(E)[:kk] for _ in range(tokens)]).astype(np.int32)
    xt, it = torch.from_numpy(x).to(cuda), torch.from_numpy(idx).to(cuda)
    args = (xt, it, moe._gu_trellis, moe._gu_suh, moe._gu_svh, moe._dn_trellis, moe._dn_suh, moe._dn_svh,
            k, moe._cb)
    print(f"moe two-launch tokens={tokens}", flush=True)
    y1 = ops.moe_forward(*args, fused=True)
    y2 = ops.moe_forward(*args, fused=True)
    y5 = ops.moe_forward(*args, fused=False)
    assert torch.equal(y1, y2)
    assert int(ops.sync_counters(cuda, 1).abs().sum()) == 0
    ref = _oracle_chain(oracle, gate, up, down, x, idx, "silu")
    assert rel_l2(y1.cpu().numpy(), ref) <= TOL
    assert rel_l2(y5.cpu().numpy(), ref) <= TOL
    assert rel_l2(y1.cpu().numpy(), y5.cpu().numpy()) <= TOL


@pytest.mark.parametrize("tokens,top_k,E", [(2, 2, 2), (5, 2, 3), (9, 3, 4), (32, 2, 40), (256, 2, 3)])
def test_slots_grouped_by_expert_equal_ungrouped(cuda, tokens, top_k, E):
    """With several tokens the slots of one expert share a pass over its weights, four
    rows at a time (here up to 171 slots per expert, i.e. many leaders per expert, and
    the routing table scanned in up to eight chunks). The arithmetic per row is that of
    the per-slot kernels, so the result is bit-identical to runs that do not group: one
    token at a time (a token's experts are distinct), and, for the 512-slot case, whose
    waves take whole Hadamard blocks where a single token's take half blocks, the same
    tokens inside a 514-slot call, which is past the grouped kernels' routing table."""
    from ponyexl3_amd import EXL3SwitchGLU, ops

    D, H, k = 384, 256, 4
    gate, up, down = _experts(E, D, H, k, False, 1300)
    moe = EXL3SwitchGLU.from_layers(gate, up, down)
    rng = np.random.default_rng(tokens * 7 + E)
    x = (rng.standard_normal((tokens + 1, D)) * 0.5).astype(np.float16)
    idx = np.stack([rng.permutation(E)[:top_k] for _ in range(tokens + 1)]).astype(np.int32)
    xt, it = torch.from_numpy(x).to(cuda), torch.from_numpy(idx).to(cuda)
    args = (moe._gu_trellis, moe._gu_suh, moe._gu_svh, moe._dn_trellis, moe._dn_suh, moe._dn_svh, k, moe._cb)
    print(f"moe grouped tokens={tokens} top_k={top_k} E={E}", flush=True)
    y = ops.moe_forward(xt[:tokens], it[:tokens], *args)
    y_again = ops.moe_forward(xt[:tokens], it[:tokens], *args)
    assert torch.equal(y, y_again)
    assert int(ops.sync_counters(cuda, 1).abs().sum()) == 0
    # the runs that do not group reduce through partial rows like the grouped kernels
    # (accumulators=False); the accumulator reduction rounds the sum differently
    if tokens * top_k == 512:
        wide = ops.moe_forward(xt, it, *args, accumulators=False)
        assert torch.equal(y, wide[:tokens])
    step = max(1, tokens // 16)
    for t in list(range(0, tokens, step)) + [tokens - 1]:
        one = ops.moe_forward(xt[t:t + 1], it[t:t + 1], *args, accumulators=False)
        if tokens * top_k == 512:
            assert rel_l2(y[t].float().cpu().numpy(), one[0].float().cpu().numpy()) <= TOL
        else:
            assert torch.equal(y[t], one[0]), f"token {t}"


@pytest.mark.parametrize("tokens,top_k,E,D,H,act", [(1, 2, 4, 640, 640, 0), (1, 8, 64, 2048, 512, 0),
                                                     (3, 2, 64, 384, 256, 1), (8, 8, 256, 512, 256, 0)])
def test_accumulator_reduction_of_gate_up(cuda, oracle, tokens, top_k, E, D, H, act):
    """Every slot on its own: gate and up of a k-chunk run in one workgroup and meet the
    other chunks in 64-bit accumulators (D of five blocks: three chunks of two blocks, the
    last half empty; 16 blocks: eight chunks). Against the partial-row reduction of the
    same call (an fp16 ulp at most: same products, the sum rounded once instead of per
    row), twice in a row bit for bit, with the accumulators back at zero."""
    from ponyexl3_amd import EXL3SwitchGLU, ops

    k = 4
    rng = np.random.default_rng(tokens * 31 + E)
    if E <= 8:
        gate, up, down = _experts(E, D, H, k, False, 1500)
        moe = EXL3SwitchGLU.from_layers(gate, up, down, activation="silu" if act == 0 else "gelu")
    else:  # random stacks: many experts without building them one by one
        rnd = lambda *s: torch.from_numpy(rng.integers(-32768, 32768, size=s, dtype=np.int16)).to(cuda)
        sgn = lambda *s: torch.from_numpy(np.where(rng.random(s) > 0.5, -1.0, 1.0).astype(np.float16)).to(cuda)
        moe = EXL3SwitchGLU(gu_trellis=rnd(D // 16, E * 2 * H // 16, 16 * k), gu_suh=sgn(E, 2, D),
                            gu_svh=sgn(E, 2 * H), dn_trellis=rnd(H // 16, E * D // 16, 16 * k),
                            dn_suh=sgn(E, H), dn_svh=sgn(E, D), k=k, cb=0)
    x = torch.from_numpy((rng.standard_normal((tokens, D)) * 0.25).astype(np.float16)).to(cuda)
    idx = torch.from_numpy(np.stack([rng.permutation(E)[:top_k] for _ in range(tokens)]).astype(np.int32)).to(cuda)
    args = (x, idx, moe._gu_trellis, moe._gu_suh, moe._gu_svh, moe._dn_trellis, moe._dn_suh, moe._dn_svh, k,
            moe._cb, act)
    print(f"moe accumulators tokens={tokens} top_k={top_k} E={E} D={D} H={H}", flush=True)
    ya = ops.moe_forward(*args)
    ya2 = ops.moe_forward(*args)
    yp = ops.moe_forward(*args, accumulators=False)
    assert torch.equal(ya, ya2)
    assert int(ops.sync_counters(cuda, 1).abs().sum()) == 0
    assert rel_l2(ya.float().cpu().numpy(), yp.float().cpu().numpy()) <= 5e-4  # fp16 ulps over three casts
    if E <= 8:
        ref = _oracle_chain(oracle, gate, up, down, x.cpu().numpy(), idx.cpu().numpy(), "silu" if act == 0 else "gelu")
        assert rel_l2(ya.cpu().numpy(), ref) <= TOL


@pytest.mark.parametrize("seed", range(10))
def test_random_shapes_three_reductions_agree(cuda, seed):
    """Random small shapes (D and H from one to six Hadamard blocks, K from 2 to 8, both
    codebooks, 1..40 tokens, top-k up to 6, few or many experts, indices outside the
    expert range included: they are clamped): the two-launch chain with whatever kernels
    the library picks (accumulators / grouped slots / per-slot partial rows), the same
    with partial rows only, and the five-launch chain must agree to fp16 ulps."""
    from ponyexl3_amd import EXL3SwitchGLU, ops

    rng = np.random.default_rng(9000 + seed)
    D, H = 128 * int(rng.integers(1, 7)), 128 * int(rng.integers(1, 7))
    k = int(rng.integers(2, 9))
    cb = int(rng.integers(0, 2))
    E = int(rng.choice([2, 5, 16, 70]))
    top_k = int(rng.integers(1, min(E, 6) + 1))
    tokens = int(rng.choice([1, 2, 3, 7, 16, 40]))
    act = int(rng.integers(0, 2))
    rnd = lambda *s: torch.from_numpy(rng.integers(-32768, 32768, size=s, dtype=np.int16)).to(cuda)
    sgn = lambda *s: torch.from_numpy(np.where(rng.random(s) > 0.5, -1.0, 1.0).astype(np.float16)).to(cuda)
    gu, dn = rnd(D // 16, E * 2 * H // 16, 16 * k), rnd(H // 16, E * D // 16, 16 * k)
    gu_suh, gu_svh, dn_suh, dn_svh = sgn(E, 2, D), sgn(E, 2 * H), sgn(E, H), sgn(E, D)
    x = torch.from_numpy((rng.standard_normal((tokens, D)) * 0.25).astype(np.float16)).to(cuda)
    idx = np.stack([rng.permutation(E)[:top_k] for _ in range(tokens)]).astype(np.int32)
    if tokens > 1:
        idx[0, 0], idx[-1, -1] = -3, E + 5  # clamped to expert 0 and E - 1
    it = torch.from_numpy(idx).to(cuda)
    args = (x, it, gu, gu_suh, gu_svh, dn, dn_suh, dn_svh, k, cb, act)
    print(f"moe random seed={seed} D={D} H={H} k={k} cb={cb} E={E} top_k={top_k} tokens={tokens}", flush=True)
    y = ops.moe_forward(*args)
    y_rows = ops.moe_forward(*args, accumulators=False)
    y_five = ops.moe_forward(*args, fused=False)
    assert torch.equal(y, ops.moe_forward(*args))
    assert int(ops.sync_counters(cuda, 1).abs().sum()) == 0
    assert torch.isfinite(y.float()).all()
    ref = y_five.float().cpu().numpy()
    assert rel_l2(y.float().cpu().numpy(), ref) <= TOL
    assert rel_l2(y_rows.float().cpu().numpy(), ref) <= TOL


@pytest.mark.parametrize("tokens,act", [(40, "silu"), (200, "gelu")])
def test_prefill_path_matches_oracle_and_slot_kernels(cuda, oracle, tokens, act):
    """From 24 tokens on the pairs are sorted by expert and go through the segmented
    GEMM. Experts with no token, one token and many tokens occur; checked against
    the oracle chain and against the per-slot kernels on the same input."""
    from ponyexl3_amd import EXL3SwitchGLU, ops

    E, D, H, kk, k = 7, 256, 128, 2, 4
    gate, up, down = _experts(E, D, H, k, False, 800)
    moe = EXL3SwitchGLU.from_layers(gate, up, down, activation=act)
    rng = np.random.default_rng(80 + tokens)
    x = (rng.standard_normal((tokens, D)) * 0.5).astype(np.float16)
    # skewed routing: expert 5 never chosen, expert 6 exactly once, the rest unevenly
    p = np.array([0.45, 0.25, 0.15, 0.1, 0.05])
    idx = np.stack([rng.choice(5, size=kk, replace=False, p=p) for _ in range(tokens)]).astype(np.int32)
    idx[3, 1] = 6
    xt, it = torch.from_numpy(x).to(cuda), torch.from_numpy(idx).to(cuda)
    print(f"moe prefill tokens={tokens} act={act}", flush=True)
    y = moe(xt.reshape(1, tokens, D), it.reshape(1, tokens, kk))[0]
    assert tuple(y.shape) == (tokens, kk, D)
    ref = _oracle_chain(oracle, gate, up, down, x, idx, act)
    assert rel_l2(y.cpu().numpy(), ref) <= TOL
    slots = torch.cat([ops.moe_forward(xt[r:r + 8], it[r:r + 8], moe._gu_trellis, moe._gu_suh, moe._gu_svh,
                                       moe._dn_trellis, moe._dn_suh, moe._dn_svh, k, moe._cb,
                                       0 if act == "silu" else 1) for r in range(0, tokens, 8)])
    assert rel_l2(y.cpu().numpy(), slots.cpu().numpy()) <= TOL


def test_moe_equals_linear_modules(cuda):
    """The stacked chain equals the same experts run as individual EXL3Linear
    modules (fused-vs-unfused, ponyexl3/tests/test_moe_activation.py:44-65)."""
    from ponyexl3_amd import EXL3Linear, EXL3SwitchGLU

    E, D, H, kk = 4, 512, 256, 3
    gate, up, down = _experts(E, D, H, 4, False, 900)
    moe = EXL3SwitchGLU.from_layers(gate, up, down)
    g = torch.Generator().manual_seed(1)
    x = (torch.randn((2, D), generator=g) * 0.5).to(torch.float16).to(cuda)
    idx = torch.tensor([[0, 2, 3], [1, 0, 2]], dtype=torch.int32, device=cuda)
    y = moe(x.reshape(1, 2, D), idx.reshape(1, 2, kk))[0]
    for t in range(2):
        for s in range(kk):
            e = int(idx[t, s])
            gv = EXL3Linear(gate[e])(x[t : t + 1]).float()
            uv = EXL3Linear(up[e])(x[t : t + 1]).float()
            h = (torch.nn.functional.silu(gv) * uv).to(torch.float16)
            ref = EXL3Linear(down[e])(h).float()
            got = y[t, s].float()
            assert float((got - ref[0]).abs().max() / (ref.abs().max() + 1e-9)) < 5e-3


def test_bounded_wait_gives_up_visibly(cuda, monkeypatch):
    """A counters array that is not zero on entry breaks the accumulator reduction of
    gate/up: the finishing workgroup's wait for complete counts is bounded (lowered here
    through EXL3_SPIN_LIMIT so that it runs out at once), every kernel still exits, the
    slot's output is NaN, the other slots are untouched and the status word is set."""
    from ponyexl3_amd import EXL3SwitchGLU, ops

    if os.environ.get("EXL3_EXACT_WEIGHTS") == "1":
        pytest.skip("the multi-launch chains this knob selects have no accumulator reduction")
    E, D, H, kk, k = 4, 640, 256, 2, 4
    gate, up, down = _experts(E, D, H, k, False, 900)
    moe = EXL3SwitchGLU.from_layers(gate, up, down)
    rng = np.random.default_rng(9)
    xt = torch.from_numpy((rng.standard_normal((1, D)) * 0.5).astype(np.float16)).to(cuda)
    it = torch.tensor([[2, 1]], dtype=torch.int32, device=cuda)
    args = (xt, it, moe._gu_trellis, moe._gu_suh, moe._gu_svh, moe._dn_trellis, moe._dn_suh, moe._dn_svh,
            k, moe._cb)
    good = ops.moe_forward(*args, fused=True)
    ops.check_counters(cuda)
    cnt = ops.sync_counters(cuda, 1)
    try:
        # accumulator of (slot 0, gate, column 5): a count of 255 that can never come out right
        cnt.view(torch.int64)[5] = -(1 << 56)
        monkeypatch.setenv("EXL3_SPIN_LIMIT", "4")
        print("moe bounded wait", flush=True)
        bad = ops.moe_forward(*args, fused=True)
        torch.cuda.synchronize()
        assert torch.isnan(bad[0, 0].float()).all()
        assert torch.equal(bad[0, 1], good[0, 1])
        with pytest.raises(RuntimeError):
            ops.check_counters(cuda)
        monkeypatch.delenv("EXL3_SPIN_LIMIT")
        assert torch.equal(ops.moe_forward(*args, fused=True), good)  # check_counters zeroed the array
        ops.check_counters(cuda)
    finally:
        torch.cuda.synchronize()
        cnt.zero_()  # whatever happened above, the shared array is clean for the next test


def test_config4_a3b_shapes(cuda, oracle):
    """hidden 2048, 256 experts of 2048->512 / 512->2048, top-8 routing from a
    softmax over seeded router logits, at 1 and 8 tokens. Every (token, expert) slot
    is checked against the oracle's unfused expert chain
    (ponyexl3/mlx/exl3_moe.py:648-682) at rel-L2 <= 1e-3, two slots also against
    per-expert EXL3Linear chains, and the slot order against permutation
    equivariance."""
    from ponyexl3_amd import EXL3Layer, EXL3Linear, EXL3SwitchGLU, ops
    from ponyexl3_amd.moe import combine_experts, route_topk

    E, D, H, kk, k = 256, 2048, 512, 8, 4
    rng = np.random.default_rng(40_004)
    gu = rng.integers(0, 65536, size=(D // 16, E * 2 * H // 16, 16 * k), dtype=np.uint16)
    dn = rng.integers(0, 65536, size=(H // 16, E * D // 16, 16 * k), dtype=np.uint16)
    sgn = lambda shape: np.where(rng.random(shape) > 0.5, -1.0, 1.0).astype(np.float16)
    gu_suh, gu_svh, dn_suh, dn_svh = sgn((E, 2, D)), sgn((E, 2 * H)), sgn((E, H)), sgn((E, D))
    dev = lambda a: torch.from_numpy(a).to(cuda)
    moe = EXL3SwitchGLU(gu_trellis=ops.as_trellis_tensor(gu, cuda), gu_suh=dev(gu_suh), gu_svh=dev(gu_svh),
                        dn_trellis=ops.as_trellis_tensor(dn, cuda), dn_suh=dev(dn_suh), dn_svh=dev(dn_svh),
                        k=k, cb=0)
    for T in (1, 8):
        x = (rng.standard_normal((T, D)) * 0.25).astype(np.float16)
        logits = torch.from_numpy(rng.standard_normal((T, E)).astype(np.float32)).to(cuda)
        inds, scores = route_topk(logits, kk)
        assert torch.allclose(scores.sum(-1), torch.ones(T, device=cuda), atol=1e-5)
        xt = dev(x)
        print(f"config4 T={T}", flush=True)
        y = moe(xt.reshape(1, T, D), inds.reshape(1, T, kk))
        assert tuple(y.shape) == (1, T, kk, D)
        out = combine_experts(y, scores.reshape(1, T, kk))
        assert tuple(out.shape) == (1, T, D) and torch.isfinite(out.float()).all()
        # slot-order permutation equivariance
        perm = torch.randperm(kk, generator=torch.Generator().manual_seed(T)).to(cuda)
        y2 = moe(xt.reshape(1, T, D), inds[:, perm].reshape(1, T, kk))
        assert torch.equal(y2, y[:, :, perm])
        # all T * 8 slots against the oracle's chain over the selected experts
        gt = H // 16
        cut = lambda a: np.ascontiguousarray(a)
        experts = {}
        for e in sorted(set(int(v) for v in inds.cpu().numpy().ravel())):
            experts[e] = {
                "gate": (cut(gu[:, e * gt : (e + 1) * gt]), gu_suh[e, 0], gu_svh[e, :H]),
                "up": (cut(gu[:, (E + e) * gt : (E + e + 1) * gt]), gu_suh[e, 1], gu_svh[e, H:]),
                "down": (cut(dn[:, e * (D // 16) : (e + 1) * (D // 16)]), dn_suh[e], dn_svh[e]),
            }
        ref_all = oracle.moe_experts_forward(experts, x, inds.cpu().numpy(), k, 0)
        got_all = y[0].cpu().numpy()
        worst = max(float(np.linalg.norm(got_all[t, s].astype(np.float64) - ref_all[t, s].astype(np.float64))
                          / np.linalg.norm(ref_all[t, s].astype(np.float64)))
                    for t in range(T) for s in range(kk))
        print(f"config4 T={T}: worst slot rel-L2 vs oracle {worst:.2e}", flush=True)
        assert worst <= 1e-3
        # two sampled slots against stand-alone layers cut out of the stacks
        for (t, s) in [(0, 0), (T - 1, kk - 1)]:
            e = int(inds[t, s])
            mk = lambda tr, suh, svh, n_in, n_out: EXL3Linear(
                EXL3Layer(f"e{e}", n_in, n_out, k, np.ascontiguousarray(tr), suh, svh))
            gl = mk(gu[:, e * gt : (e + 1) * gt], gu_suh[e, 0], gu_svh[e, :H], D, H)
            ul = mk(gu[:, (E + e) * gt : (E + e + 1) * gt], gu_suh[e, 1], gu_svh[e, H:], D, H)
            dl = mk(dn[:, e * (D // 16) : (e + 1) * (D // 16)], dn_suh[e], dn_svh[e], H, D)
            h = (torch.nn.functional.silu(gl(xt[t : t + 1]).float()) * ul(xt[t : t + 1]).float()).to(torch.float16)
            ref = dl(h).float()[0]
            got = y[0, t, s].float()
            assert float((got - ref).norm() / ref.norm()) <= 5e-3


def test_errors(cuda):
    from ponyexl3_amd import EXL3SwitchGLU

    z = lambda *s: torch.zeros(s, dtype=torch.float16, device=cuda)
    zi = lambda *s: torch.zeros(s, dtype=torch.int16, device=cuda)
    with pytest.raises(ValueError):
        EXL3SwitchGLU(gu_trellis=zi(8, 16, 64), gu_suh=z(1, 2, 128), gu_svh=z(1, 256), dn_trellis=zi(8, 8, 64),
                      dn_suh=z(1, 128), dn_svh=z(1, 128), k=4, cb=0, activation="relu")
    with pytest.raises(ValueError):
        EXL3SwitchGLU(gu_trellis=zi(8, 8, 64), gu_suh=z(1, 2, 128), gu_svh=z(1, 256), dn_trellis=zi(8, 8, 64),
                      dn_suh=z(1, 128), dn_svh=z(1, 128), k=4, cb=0)


def test_moe_block_with_shared_expert(cuda, oracle):
    """Router (softmax, top-k, renormalise), the shared expert stacked last with a
    sigmoid gate, weighted sum: against the same composition over the oracle chain
    (ponyexl3/mlx/exl3_moe.py:790-839)."""
    from ponyexl3_amd import EXL3MoEBlock, EXL3SwitchGLU

    E, D, H, kk = 5, 256, 128, 2  # 4 routed experts + the shared one
    gate, up, down = _experts(E, D, H, 4, True, 950)
    switch = EXL3SwitchGLU.from_layers(gate, up, down)
    g = torch.Generator().manual_seed(2)
    router = torch.nn.Linear(D, E - 1, bias=False)
    shared_gate = torch.nn.Linear(D, 1, bias=False)
    with torch.no_grad():
        router.weight.copy_(torch.randn((E - 1, D), generator=g) * 0.2)
        shared_gate.weight.copy_(torch.randn((1, D), generator=g) * 0.2)
    block = EXL3MoEBlock(router.half().to(cuda), shared_gate.half().to(cuda), switch, kk).to(cuda)
    x = (torch.randn((3, D), generator=g) * 0.5).to(torch.float16)
    with torch.no_grad():
        y = block(x.to(cuda)).float().cpu().numpy()
        inds, scores = block.route(x.to(cuda).reshape(1, 3, D))
    assert y.shape == (3, D)
    inds, scores = inds[0].cpu().numpy(), scores[0].float().cpu().numpy()
    assert inds.shape == (3, kk + 1) and (inds[:, -1] == E - 1).all() and (inds[:, :kk] < E - 1).all()
    np.testing.assert_allclose(scores[:, :kk].sum(axis=1), 1.0, atol=2e-3)
    per_expert = _oracle_chain(oracle, gate, up, down, x.numpy(), inds.astype(np.int32), "silu")
    ref = (per_expert.astype(np.float32) * scores[..., None]).sum(axis=1)
    assert rel_l2(y, ref) <= 2 * TOL  # fp16 products and sum over three experts on top of the chain


@pytest.mark.parametrize("tokens,top_k,E,block_rows", [(40, 2, 7, 64), (513, 8, 256, 64), (3000, 4, 1024, 64),
                                                        (2100, 8, 16, 256), (1, 1, 1, 64)])
def test_pair_sort_kernel_equals_stable_argsort(cuda, tokens, top_k, E, block_rows):
    """Integer work, bit-exact: order / tok / sidx against torch's stable argsort, the
    row-block table against the table built from device-side torch ops (same worst-case
    length, same empty entries). Includes out-of-range ids (clamped), experts with no
    pair and more pairs than one 1024-pair scatter round."""
    from ponyexl3_amd import ops

    rng = np.random.default_rng(tokens + E)
    idx = rng.integers(0, E, size=(tokens, top_k)).astype(np.int32)
    if E > 4:
        idx[idx == 3] = 2  # expert 3 gets nothing
        idx[0, 0] = E + 5  # clamps to E - 1
        if tokens > 1:
            idx[1, 0] = -4  # clamps to 0
    it = torch.from_numpy(idx).to(cuda)
    order, tok, sidx, table = ops.moe_sort(it, E, block_rows)
    flat = it.reshape(-1).long().clamp(0, E - 1)
    ref_order = torch.argsort(flat, stable=True)
    assert torch.equal(order.long(), ref_order)
    assert torch.equal(sidx.long(), flat[ref_order])
    assert torch.equal(tok.long(), ref_order // top_k)
    ref_table = ops.segment_table(flat[ref_order], E, block_rows)
    assert tuple(table.shape) == tuple(ref_table.shape)
    assert torch.equal(table, ref_table)
    o2, t2, s2, tab2 = ops.moe_sort(it, E, block_rows)  # same answer every call
    assert torch.equal(o2, order) and torch.equal(tab2, table)


@pytest.mark.parametrize("act", [0, 1])
def test_glu_rows_kernel_equals_separate_launches(cuda, act):
    """Finish gate/up + GLU + down rotation in one launch against the per-row
    Hadamard launches around torch's GLU (same casts: fp16 after every stage)."""
    from ponyexl3_amd import ops

    rng = np.random.default_rng(17 + act)
    N, H, E = 300, 384, 9
    g = torch.from_numpy((rng.standard_normal((N, H)) * 2).astype(np.float16)).to(cuda)
    u = torch.from_numpy((rng.standard_normal((N, H)) * 2).astype(np.float16)).to(cuda)
    sidx = torch.from_numpy(np.sort(rng.integers(0, E, size=N)).astype(np.int32)).to(cuda)
    sgn = lambda *s: torch.from_numpy(np.where(rng.random(s) > 0.5, -1, 1).astype(np.float16)).to(cuda)
    gu_svh, dn_suh = sgn(E, 2 * H), sgn(E, H)
    got = ops.moe_glu_rows(g, u, sidx, gu_svh, dn_suh, act)
    gf = ops.had128_rows(g, gu_svh[:, :H], True, scale_index=sidx).float()
    uf = ops.had128_rows(u, gu_svh[:, H:], True, scale_index=sidx).float()
    a = torch.nn.functional.gelu(gf, approximate="tanh") if act else torch.nn.functional.silu(gf)
    ref = ops.had128_rows((a * uf).to(torch.float16), dn_suh, False, scale_index=sidx)
    diff = (got.float() - ref.float()).abs().max()
    # expf / tanhf of the kernel vs torch's: an fp16 ulp of h here and there
    assert float(diff) <= 4e-3 * float(ref.float().abs().max())
    with pytest.raises(ValueError):
        ops.moe_glu_rows(g, u[:, :256], sidx, gu_svh, dn_suh, act)
