"""Folded fp16 engine: the public weight of an EXL3 layer as a plain
``torch.nn.Linear`` (``fold16``).

The EXL3 forward is linear in x, so both Hadamard transforms and both sign/scale
vectors fold into ``W_pub = diag(suh) . H . W_inner . H . diag(svh)``. As in the
reference (``ponyexl3/mlx/native.py:49-85``) W_pub is obtained by pushing an fp16
identity through the same prefill forward the exact engine uses (input Hadamard
kernel, MFMA trellis GEMM, output Hadamard kernel), one stripe of output columns
at a time, so the folded weight carries exactly the runtime's cast points.

The reference's w8a16 / w4a16 targets re-quantize W_pub with MLX's affine group
quantizer (``native.py:88-124,216-264``); that is an MLX storage format with no
counterpart here and is not provided.
"""

from __future__ import annotations

from dataclasses import dataclass

import torch

from . import ops
from .layer import EXL3Layer
from .linear import EXL3Linear, layer_runtime

# One stripe of output columns at a time (multiple of 128), native.py:45.
PUBLIC_CHUNK_COLS = 8192


def public_weight_chunks(layer: EXL3Layer, *, chunk_cols: int = PUBLIC_CHUNK_COLS, device="cuda"):
    """Yield ``W_pub[:, n0:n1]`` fp16 chunks with all transforms folded in
    (``public_weight_chunks``, ponyexl3/mlx/native.py:49-70)."""
    if chunk_cols % 128 != 0:
        raise ValueError("chunk_cols must be a multiple of 128")
    rt = layer_runtime(layer, device)
    n_in, n_out = layer.in_features, layer.out_features
    eye = torch.eye(n_in, dtype=torch.float16, device=rt.trellis.device)
    xh = ops.had128_pre(eye, rt.suh)  # rows of the scaled input Hadamard, computed once
    del eye
    for n0 in range(0, n_out, chunk_cols):
        n = min(chunk_cols, n_out - n0)
        y = ops.inner_gemm(xh, rt.trellis, rt.k, rt.cb, n0 // 16, n // 16)
        if y.dtype != torch.float16:  # small-batch kernel (in_features <= 8) returns fp32 sums
            y = y.to(torch.float16)
        svh = None if rt.svh is None else rt.svh[n0:n0 + n].contiguous()
        yield ops.had128_post(y, svh)


def public_weight(layer: EXL3Layer, *, device="cuda") -> torch.Tensor:
    """Full ``(in, out)`` fp16 public weight (``public_weight_mlx``, native.py:73-75)."""
    return torch.cat(list(public_weight_chunks(layer, device=device)), dim=1)


def folded_linear_from_exl3(layer: EXL3Layer, *, device="cuda") -> torch.nn.Linear:
    """Exact fold: ``torch.nn.Linear`` holding the fp16 public weight, no
    requantization (``folded_linear_from_exl3``, native.py:78-85)."""
    lin = torch.nn.Linear(layer.in_features, layer.out_features, bias=layer.bias is not None,
                          device=device, dtype=torch.float16)
    with torch.no_grad():
        lin.weight.copy_(public_weight(layer, device=device).T)
        if layer.bias is not None:
            lin.bias.copy_(torch.from_numpy(layer.bias).to(torch.float16))
    lin.requires_grad_(False)
    return lin


class FusedSwiGLU(torch.nn.Module):
    """gate_proj + up_proj folded into one matmul (``FusedSwiGLU``, native.py:127-139)."""

    def __init__(self, gate_up: torch.nn.Module, down: torch.nn.Module) -> None:
        super().__init__()
        self.gate_up = gate_up
        self.down = down

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        g, u = self.gate_up(x).chunk(2, dim=-1)
        return self.down(torch.nn.functional.silu(g) * u)


def _fuse_two_linears(a: torch.nn.Linear, b: torch.nn.Linear) -> torch.nn.Linear:
    out = torch.nn.Linear(a.in_features, a.out_features + b.out_features, bias=False,
                          device=a.weight.device, dtype=a.weight.dtype)
    with torch.no_grad():
        out.weight.copy_(torch.cat([a.weight, b.weight], dim=0))
    out.requires_grad_(False)
    return out


def fuse_mlps(model) -> int:
    """Replace folded bias-free gate/up/down MLPs (``model.layers[i].mlp``) by
    :class:`FusedSwiGLU` (``fuse_mlps``, native.py:166-185). Exact."""
    n = 0
    for layer in model.layers:
        mlp = getattr(layer, "mlp", None)
        gate = getattr(mlp, "gate_proj", None)
        up = getattr(mlp, "up_proj", None)
        down = getattr(mlp, "down_proj", None)
        if gate is None or up is None or down is None:
            continue
        if not (type(gate) is torch.nn.Linear and type(up) is torch.nn.Linear):
            continue
        if gate.bias is not None or up.bias is not None:
            continue
        layer.mlp = FusedSwiGLU(_fuse_two_linears(gate, up), down)
        n += 1
    return n


@dataclass
class LayerError:
    """Output-space error of a converted layer vs the exact EXL3 path (native.py:188-201)."""

    key: str
    engine: str
    rms_ref: float
    rms_err: float

    @property
    def rel(self) -> float:
        return self.rms_err / self.rms_ref if self.rms_ref else 0.0

    def __str__(self) -> str:
        return f"{self.key}: rel RMS err {self.rel:.2e} ({self.engine})"


def layer_error(layer: EXL3Layer, module: torch.nn.Module, engine: str, *, rows: int = 8,
                device="cuda") -> LayerError:
    """RMS error of ``module`` against ``EXL3Linear(layer)`` on ``rows`` seeded
    N(0, 0.5^2) activations (``layer_error``, native.py:204-214)."""
    gen = torch.Generator(device="cpu").manual_seed(0)
    x = (torch.randn((rows, layer.in_features), generator=gen) * 0.5).to(torch.float16).to(device)
    with torch.no_grad():
        y_ref = EXL3Linear(layer, device=device)(x).float()
        y_new = module(x).float()
    rms_ref = float(torch.sqrt(torch.mean(y_ref * y_ref)))
    rms_err = float(torch.sqrt(torch.mean((y_new - y_ref) ** 2)))
    return LayerError(key=layer.key, engine=engine, rms_ref=rms_ref, rms_err=rms_err)
