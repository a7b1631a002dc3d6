"""EXL3 quantized linear module on ROCm tensors.

Mirrors ``EXL3Linear`` (ponyexl3/mlx/exl3_linear.py:56-165) and the per-layer
runtime cache of ponyexl3/mlx/layer_state.py:24-37,118-167: the trellis stays
packed on the device and every batch size reads it directly (small batches
through the fused decode GEMV, larger ones through the MFMA prefill GEMM), so
there is no fp16 weight to cache and ``warm()`` has nothing to pre-decode.
"""

from __future__ import annotations

from dataclasses import dataclass
from typing import Any

import numpy as np
import torch

from . import ops
from .layer import EXL3Layer, codebook_mode_from_flags, unpack_signs_or_pass


def _layer_key(layer: EXL3Layer) -> tuple[Any, ...]:
    return (id(layer), layer.key, layer.in_features, layer.out_features, layer.k, layer.mcg,
            layer.mul1)


@dataclass(frozen=True)
class EXL3LayerRuntime:
    """Device tensors kept for one EXL3 layer."""

    key: tuple[Any, ...]
    trellis: torch.Tensor  # int16 bits of the packed uint16 trellis
    suh: torch.Tensor | None
    svh: torch.Tensor | None
    bias: torch.Tensor | None
    k: int
    cb: int

    def prepare_xh(self, x2d: torch.Tensor) -> torch.Tensor:
        return ops.had128_pre(x2d, self.suh)

    def finish_y(self, y: torch.Tensor) -> torch.Tensor:
        return ops.had128_post(y, self.svh)


_runtime_cache: dict[tuple[Any, ...], EXL3LayerRuntime] = {}


def _to_half(v, device):
    if v is None:
        return None
    return torch.from_numpy(np.ascontiguousarray(v, dtype=np.float16)).to(device)


def layer_runtime(layer: EXL3Layer, device="cuda") -> EXL3LayerRuntime:
    """Trellis + signs + bias uploaded once per layer object."""
    key = _layer_key(layer) + (str(device),)
    rt = _runtime_cache.get(key)
    if rt is None:
        if layer.trellis is None:
            raise ValueError(f"{layer.key}: host trellis was released before the first upload")
        rt = EXL3LayerRuntime(
            key=key,
            trellis=ops.as_trellis_tensor(layer.trellis, device),
            suh=_to_half(unpack_signs_or_pass(layer.suh), device),
            svh=_to_half(unpack_signs_or_pass(layer.svh), device),
            bias=_to_half(layer.bias, device),
            k=int(layer.k),
            cb=int(codebook_mode_from_flags(mcg=layer.mcg, mul1=layer.mul1)),
        )
        _runtime_cache[key] = rt
    return rt


def clear_layer_caches() -> None:
    _runtime_cache.clear()


class EXL3Linear(torch.nn.Module):
    """One EXL3-quantized linear layer; callable ``(..., in) -> (..., out)`` fp16.

    Exposes no parameters or buffers, so loading the surrounding model's
    state dict never expects a ``weight`` here."""

    def __init__(self, layer: EXL3Layer, device="cuda"):
        super().__init__()
        layer.validate()
        if layer.in_features % 128 or layer.out_features % 128:
            raise ValueError("in/out features must be multiples of 128 (Hadamard-128 blocks)")
        self._exl3 = layer
        self._rt = layer_runtime(layer, device)
        self.in_features = layer.in_features
        self.out_features = layer.out_features

    def extra_repr(self) -> str:
        return f"in={self.in_features}, out={self.out_features}, k={self._exl3.k}"

    def warm(self) -> "EXL3Linear":
        return self

    def release_source(self) -> "EXL3Linear":
        """Drop the host-side numpy trellis; the device runtime keeps the weights."""
        self._exl3.trellis = None
        return self

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        rt = self._rt
        if x.shape[-1] != self.in_features:
            raise ValueError(f"expected last dim {self.in_features}, got {x.shape[-1]}")
        x2d = x.reshape(-1, self.in_features).to(torch.float16).contiguous()
        y = ops.linear_forward(x2d, rt.trellis, rt.k, rt.cb, rt.suh, rt.svh, rt.bias)
        return y.reshape(tuple(x.shape[:-1]) + (self.out_features,))
