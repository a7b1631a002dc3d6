"""Checkpoint directory -> EXL3 modules on the GPU: module swap, sibling fusion
and expert stacking (ponyexl3/mlx/model.py:77-127, 357-432, 625-650)."""
import numpy as np
import pytest
import torch

from conftest import rel_l2
from test_loader import _write_checkpoint

pytestmark = pytest.mark.gpu
TOL = 1e-3


class _Mlp(torch.nn.Module):
    def __init__(self, d, h):
        super().__init__()
        self.gate_proj = torch.nn.Linear(d, h, bias=False)
        self.up_proj = torch.nn.Linear(d, h, bias=False)
        self.down_proj = torch.nn.Linear(h, d, bias=False)

    def forward(self, x):
        g, u = self.gate_proj(x), self.up_proj(x)
        return self.down_proj((torch.nn.functional.silu(g.float()) * u.float()).to(torch.float16))


class _Block(torch.nn.Module):
    def __init__(self, d, h):
        super().__init__()
        self.mlp = _Mlp(d, h)


class _Model(torch.nn.Module):
    def __init__(self, d, h):
        super().__init__()
        self.layers = torch.nn.ModuleList([_Block(d, h)])
        self.lm_head = torch.nn.Linear(d, 2 * d, bias=False)  # stays a plain Linear: not in the checkpoint


def test_swap_and_fuse_from_checkpoint(cuda, oracle, tmp_path):
    from ponyexl3_amd import EXL3Linear, FusedEXL3Sibling, loader, make_exl3_layer

    d, h = 256, 384
    src = [
        make_exl3_layer(k=4, in_features=d, out_features=h, seed=11, key="layers.0.mlp.gate_proj", mcg=True),
        make_exl3_layer(k=4, in_features=d, out_features=h, seed=12, key="layers.0.mlp.up_proj", mcg=True),
        make_exl3_layer(k=3, in_features=h, out_features=d, seed=13, key="layers.0.mlp.down_proj", mcg=True),
    ]
    layers = loader.load_all_exl3_layers(_write_checkpoint(tmp_path, src))
    model = _Model(d, h).half().to(cuda)
    assert loader.swap_exl3_linears(model, layers, device=cuda) == 3
    mlp = model.layers[0].mlp
    assert isinstance(mlp.gate_proj, EXL3Linear) and isinstance(model.lm_head, torch.nn.Linear)
    rng = np.random.default_rng(0)
    x = (rng.standard_normal((3, d)) * 0.5).astype(np.float16)
    xt = torch.from_numpy(x).to(cuda)

    def ref_forward():
        fw = lambda l, v: oracle.linear_forward(l.trellis, l.k, l.codebook_mode, l.suh, l.svh, v)
        g, u = fw(src[0], x).astype(np.float32), fw(src[1], x).astype(np.float32)
        hmid = (g / (1.0 + np.exp(-g)) * u).astype(np.float16)
        return fw(src[2], hmid)

    ref = ref_forward()
    y_unfused = mlp(xt).cpu().numpy()
    assert rel_l2(y_unfused, ref) <= TOL
    assert loader.fuse_exl3_siblings(model) == 0  # 0.4 MB of fp16-equivalent weights: below the threshold
    assert loader.fuse_exl3_siblings(model, min_bytes=0) == 1
    assert isinstance(mlp.gate_proj, FusedEXL3Sibling) and isinstance(mlp.down_proj, EXL3Linear)
    assert loader.fuse_exl3_siblings(model, min_bytes=0) == 0  # already fused
    assert rel_l2(mlp(xt).cpu().numpy(), ref) <= TOL


def test_stack_experts_from_checkpoint(cuda, oracle, tmp_path):
    from ponyexl3_amd import loader, make_exl3_layer

    E, D, H, kk = 3, 256, 128, 2
    src = []
    for e in range(E):
        pre = f"model.layers.0.mlp.experts.{e}"
        src += [make_exl3_layer(k=4, in_features=D, out_features=H, seed=30 + 3 * e, key=f"{pre}.gate_proj"),
                make_exl3_layer(k=4, in_features=D, out_features=H, seed=31 + 3 * e, key=f"{pre}.up_proj"),
                make_exl3_layer(k=4, in_features=H, out_features=D, seed=32 + 3 * e, key=f"{pre}.down_proj")]
    layers = loader.load_all_exl3_layers(_write_checkpoint(tmp_path, src, shards=2))
    moe, consumed = loader.stack_expert_switch_glu(
        [f"model.layers.0.mlp.experts.{e}" for e in range(E)], layers, device=cuda)
    assert consumed == {l.key for l in src}
    rng = np.random.default_rng(1)
    x = (rng.standard_normal((2, D)) * 0.5).astype(np.float16)
    idx = np.array([[0, 2], [1, 0]], dtype=np.int32)
    y = moe(torch.from_numpy(x).to(cuda).reshape(1, 2, D), torch.from_numpy(idx).to(cuda).reshape(1, 2, kk))
    experts = [{"gate": (g.trellis, g.suh, g.svh), "up": (u.trellis, u.suh, u.svh),
                "down": (dn.trellis, dn.suh, dn.svh)} for g, u, dn in zip(src[0::3], src[1::3], src[2::3])]
    ref = oracle.moe_experts_forward(experts, x, idx, 4, 0, "silu")
    assert rel_l2(y[0].cpu().numpy(), ref) <= TOL
    with pytest.raises(KeyError):
        loader.stack_expert_switch_glu(["model.layers.0.mlp.experts.7"], layers, device=cuda)
