"""Fused sibling groups: several same-K linears that share an input run as one
launch chain over a concatenated trellis.

Mirrors ``FusedEXL3Group`` / ``FusedEXL3Sibling`` / ``fusable``
(ponyexl3/mlx/exl3_fused.py:79-228). Members are concatenated along out_tiles,
``suh`` rows are stacked so each member sees its own rotated activations, and
``svh`` is concatenated (member out_features are multiples of 128, so an output
Hadamard block never straddles two members).
"""

from __future__ import annotations

import weakref

import numpy as np
import torch

from . import ops
from .layer import EXL3Layer, codebook_mode_from_flags, unpack_signs_or_pass


def fusable(layers: list[EXL3Layer]) -> bool:
    first = layers[0]
    return (
        len(layers) >= 2
        and all(l.in_features == first.in_features for l in layers)
        and all(l.k == first.k for l in layers)
        and all((l.mcg, l.mul1) == (first.mcg, first.mul1) for l in layers)
        and all(l.out_features % 128 == 0 for l in layers)
        and all(l.suh is not None and l.svh is not None for l in layers)
        and all(l.bias is None for l in layers)
    )


class FusedEXL3Group(torch.nn.Module):
    """Owner of the concatenated trellis + stacked signs for sibling linears."""

    def __init__(self, layers: list[EXL3Layer], device="cuda"):
        super().__init__()
        if not fusable(layers):
            raise ValueError("layers not fusable: " + ", ".join(l.key for l in layers))
        for l in layers:
            l.validate()
        if layers[0].in_features % 128:
            raise ValueError("in_features must be a multiple of 128")
        self._keys = [l.key for l in layers]
        self._k = int(layers[0].k)
        self._cb = int(codebook_mode_from_flags(mcg=layers[0].mcg, mul1=layers[0].mul1))
        self.in_features = layers[0].in_features
        self._out_features = [l.out_features for l in layers]
        self._trellis = ops.as_trellis_tensor(
            np.concatenate([np.asarray(l.trellis).view(np.uint16) for l in layers], axis=1), device
        )
        suh = np.stack([unpack_signs_or_pass(l.suh) for l in layers]).astype(np.float16)
        svh = np.concatenate([unpack_signs_or_pass(l.svh) for l in layers]).astype(np.float16)
        self._suh_stack = torch.from_numpy(suh).to(device)
        self._svh_cat = torch.from_numpy(svh).to(device)
        tile_sub = np.repeat(
            np.arange(len(layers), dtype=np.uint32), [l.out_features // 16 for l in layers]
        )
        self._tile_sub = tile_sub
        self._group_sub = ops.group_sub_from_tile_sub(tile_sub).to(device)
        # member of every 256-column block, for the one-launch prefill GEMM
        self._block_sub = (self._group_sub[::2].contiguous()
                           if all(n % 256 == 0 for n in self._out_features) else None)
        self._cache_key = None
        self._cache_out = None
        self._cache_served: set = set()

    def extra_repr(self) -> str:
        return f"members={self._keys}, k={self._k}"

    def forward_all(self, x: torch.Tensor) -> tuple[torch.Tensor, ...]:
        lead = tuple(x.shape[:-1])
        x2d = x.reshape(-1, self.in_features).to(torch.float16).contiguous()
        y = ops.linear_forward(
            x2d, self._trellis, self._k, self._cb, self._suh_stack, self._svh_cat, None,
            self._group_sub, member_out=self._out_features, block_sub=self._block_sub,
        )
        outs = torch.split(y, self._out_features, dim=-1)
        return tuple(o.reshape(lead + (n,)) for o, n in zip(outs, self._out_features))

    def _same_input(self, x: torch.Tensor, idx: int | None = None) -> bool:
        """Whether x is the input the cached outputs were computed from. The reference
        compares object identity (ponyexl3/mlx/exl3_fused.py:204-208), which is enough
        for immutable mlx arrays. A torch tensor can be refilled in place (static
        decode buffers, HIP-graph inputs), so the version counter must match too; the
        tensor is held weakly (a freed tensor's address can be handed out again); and a
        result computed eagerly must not stand in for a launch that a graph capture
        has to record. Tensors made under ``torch.inference_mode()`` keep no version
        counter; for those a request is served from the cache only while it asks for a
        member that has not been served from it yet (a second request for the same
        member is a new step, whatever the tensor object is)."""
        if self._cache_out is None or self._cache_key is None:
            return False
        ref, version, capturing = self._cache_key
        if ref() is not x or version != self._version_of(x):
            return False
        if version is None and (idx is None or idx in self._cache_served):
            return False
        return capturing == (x.is_cuda and torch.cuda.is_current_stream_capturing())

    @staticmethod
    def _version_of(x: torch.Tensor):
        return None if x.is_inference() else x._version

    def cached(self, x: torch.Tensor, idx: int | None = None) -> tuple[torch.Tensor, ...]:
        """Outputs of all members for x, computed once per distinct input and dropped
        as soon as every member has been served (nothing is kept alive after that)."""
        if not self._same_input(x, idx):
            self._cache_out = self.forward_all(x)
            self._cache_key = (weakref.ref(x), self._version_of(x),
                               x.is_cuda and torch.cuda.is_current_stream_capturing())
            self._cache_served = set()
        outs = self._cache_out
        if idx is not None:
            self._cache_served.add(idx)
            if len(self._cache_served) == len(self._out_features):
                self._cache_out = None
                self._cache_key = None
        return outs

    def sibling(self, idx: int) -> "FusedEXL3Sibling":
        return FusedEXL3Sibling(self, idx)


class FusedEXL3Sibling(torch.nn.Module):
    """Drop-in replacement for one member linear; delegates to the group and
    serves from its single-slot input-identity cache."""

    def __init__(self, group: FusedEXL3Group, idx: int):
        super().__init__()
        # keep the group out of the module tree: siblings do not own it
        object.__setattr__(self, "_group", group)
        self._idx = idx
        self.in_features = group.in_features
        self.out_features = group._out_features[idx]

    def extra_repr(self) -> str:
        return f"{self._group._keys[self._idx]} (member {self._idx})"

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        return self._group.cached(x, self._idx)[self._idx]
