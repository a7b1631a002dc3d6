"""HIP-graph replays of the layer, MoE and prefill paths give the eager results.

A decoder captures its token step once and replays it; the kernels keep state
between launches (group counters that must return to zero, per-device workspaces),
so every replay -- several, with eager launches and synchronisations between them
and fresh inputs each time -- is checked bit for bit against the eager call."""
import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu


def _replay_matches_eager(cuda, make_inputs, run, n_replays=4):
    static_in = make_inputs(0)
    run(*static_in)  # warm-up outside the capture: workspaces and counters get allocated here
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        static_out = run(*static_in)
    outs = static_out if isinstance(static_out, (tuple, list)) else (static_out,)
    for rep in range(1, n_replays + 1):
        fresh = make_inputs(rep)
        for dst, src in zip(static_in, fresh):
            dst.copy_(src)
        graph.replay()
        torch.cuda.synchronize()
        got = [o.clone() for o in outs]
        eager = run(*fresh)  # eager work between the replays, on the same workspaces
        eager = eager if isinstance(eager, (tuple, list)) else (eager,)
        torch.cuda.synchronize()
        for g, e in zip(got, eager):
            assert torch.equal(g, e), f"replay {rep} differs from the eager launch"


@pytest.mark.parametrize("rows", [1, 4, 8, 12, 40])
def test_layer_step_replays(cuda, rows):
    """One decoder layer's linears (sibling-fused qkv-like group, a plain layer with
    bias) at small-batch, medium-batch (9..32 rows) and prefill row counts."""
    from ponyexl3_amd import EXL3Linear, FusedEXL3Group, make_exl3_layer

    group = FusedEXL3Group([make_exl3_layer(k=4, in_features=512, out_features=o, seed=40 + i, key=f"g{i}")
                            for i, o in enumerate((384, 128, 128))])
    lin = EXL3Linear(make_exl3_layer(k=3, in_features=640, out_features=512, seed=50, mcg=True, bias=True))

    def make_inputs(seed):
        g = torch.Generator().manual_seed(100 * rows + seed)
        return (torch.randn((rows, 512), generator=g).half().to(cuda),)

    def run(x):
        q, k, v = group.forward_all(x)
        return q, k, v, lin(torch.cat([q, k, v], dim=-1))

    print(f"graph layer rows={rows}", flush=True)
    _replay_matches_eager(cuda, make_inputs, run)


@pytest.mark.parametrize("tokens", [1, 8, 64])
def test_moe_replays(cuda, tokens):
    """Two-launch expert chain (1 and 8 tokens) and the sorted prefill path (64
    tokens: pair sort, segmented GEMM, fused GLU) with routing that changes from
    replay to replay."""
    from ponyexl3_amd import EXL3SwitchGLU, make_exl3_layer

    E, D, H, kk = 8, 256, 128, 2
    mk = lambda n_in, n_out, s: make_exl3_layer(k=4, in_features=n_in, out_features=n_out, seed=s)
    moe = EXL3SwitchGLU.from_layers([mk(D, H, 600 + e) for e in range(E)], [mk(D, H, 700 + e) for e in range(E)],
                                    [mk(H, D, 800 + e) for e in range(E)])

    def make_inputs(seed):
        rng = np.random.default_rng(1000 * tokens + seed)
        x = torch.from_numpy((rng.standard_normal((1, tokens, D)) * 0.5).astype(np.float16)).to(cuda)
        idx = np.stack([rng.permutation(E)[:kk] for _ in range(tokens)]).astype(np.int32)
        return x, torch.from_numpy(idx).reshape(1, tokens, kk).to(cuda)

    print(f"graph moe tokens={tokens}", flush=True)
    _replay_matches_eager(cuda, make_inputs, lambda x, idx: moe(x, idx))
