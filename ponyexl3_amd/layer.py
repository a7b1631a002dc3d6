"""EXL3 layer container and host-side helpers (numpy), mirroring
``ponyexl3/ref/layer.py:12-44``, ``ponyexl3/ref/codebook.py:9-12,94-99`` and
``ponyexl3/ref/signs.py:8-27``."""

from __future__ import annotations

from dataclasses import dataclass
from enum import IntEnum

import numpy as np


class CodebookMode(IntEnum):
    DEFAULT = 0  # "3INST"
    MCG = 1
    MUL1 = 2


def codebook_mode_from_flags(mcg: bool = False, mul1: bool = False) -> CodebookMode:
    if mcg:
        return CodebookMode.MCG
    if mul1:
        return CodebookMode.MUL1
    return CodebookMode.DEFAULT


def tensor_core_perm() -> np.ndarray:
    """Kernel order -> row-major position inside a 16x16 tile: ``kernel[i] =
    row_major[perm[i]]`` (``tensor_core_perm``, ponyexl3/ref/perm.py:8-25). Closed
    form: codewords 8t..8t+7 belong to the fragment lane t of an m16n8k16 B operand,
    i.e. rows 2(t%4) + {0, 1, 8, 9} of columns t//4 and t//4 + 8."""
    i = np.arange(256, dtype=np.int32)
    t, j = i >> 3, i & 7
    row = 2 * (t & 3) + (j & 1) + 8 * ((j >> 1) & 1)
    col = (t >> 2) + 8 * (j >> 2)
    return (row * 16 + col).astype(np.int32)


def tensor_core_perm_inverse() -> np.ndarray:
    """``row_major[p] = kernel[inv[p]]`` (ponyexl3/ref/perm.py:28-32)."""
    inv = np.empty(256, dtype=np.int32)
    inv[tensor_core_perm()] = np.arange(256, dtype=np.int32)
    return inv


def unpack_sign_bitfield(bitfield: np.ndarray) -> np.ndarray:
    """Packed int16 sign words (one per 16 channels, bit set = -1, least
    significant bit = first channel) -> +-1 float16."""
    bf = np.asarray(bitfield).astype(np.uint16).reshape(-1, 1)
    bits = (bf >> np.arange(16, dtype=np.uint16).reshape(1, 16)) & 1
    return np.where(bits != 0, -1.0, 1.0).astype(np.float16).reshape(-1)


def unpack_signs_or_pass(values):
    if values is None:
        return None
    values = np.asarray(values)
    if values.dtype == np.float16 or values.dtype == np.float32:
        return values.astype(np.float16, copy=False)
    return unpack_sign_bitfield(values)


@dataclass
class EXL3Layer:
    """One EXL3-quantized linear layer as stored on disk."""

    key: str
    in_features: int
    out_features: int
    k: int
    trellis: np.ndarray  # (in_tiles, out_tiles, 16*k) uint16 (int16 accepted)
    suh: np.ndarray | None = None  # float16 (in,) or packed int16 (in//16,)
    svh: np.ndarray | None = None
    bias: np.ndarray | None = None
    mcg: bool = False
    mul1: bool = False

    @property
    def codebook_mode(self) -> int:
        return int(codebook_mode_from_flags(mcg=self.mcg, mul1=self.mul1))

    @property
    def packed_tile_size(self) -> int:
        return 256 * self.k // 16

    def validate(self) -> None:
        if not 1 <= int(self.k) <= 8:
            raise ValueError(f"K must be in [1, 8], got {self.k}")
        if self.in_features % 16 != 0 or self.out_features % 16 != 0:
            raise ValueError("in/out features must be multiples of 16")
        expected = (self.in_features // 16, self.out_features // 16, self.packed_tile_size)
        if self.trellis is None or tuple(self.trellis.shape) != expected:
            got = None if self.trellis is None else tuple(self.trellis.shape)
            raise ValueError(f"trellis shape {got} != expected {expected}")


def make_exl3_layer(
    *,
    k: int = 4,
    in_features: int = 128,
    out_features: int = 128,
    seed: int = 0,
    suh="random",
    svh="random",
    mcg: bool = False,
    mul1: bool = False,
    bias: bool = False,
    key: str = "synthetic.layer",
) -> EXL3Layer:
    """Seeded synthetic layer. Every uint16 fill is a legal bitstream, so the
    trellis is raw random words (``numpy.random.default_rng(seed)``); signs are
    ``where(rng.random(n) > 0.5, -1, 1)`` drawn after the trellis, suh first."""
    rng = np.random.default_rng(seed)
    trellis = rng.integers(
        0, 65536, size=(in_features // 16, out_features // 16, 16 * k), dtype=np.uint16
    )

    def _signs(n):
        return np.where(rng.random(n) > 0.5, -1.0, 1.0).astype(np.float16)

    suh_arr = _signs(in_features) if isinstance(suh, str) else suh
    svh_arr = _signs(out_features) if isinstance(svh, str) else svh
    bias_arr = (rng.standard_normal(out_features) * 0.01).astype(np.float16) if bias else None
    return EXL3Layer(
        key=key, in_features=in_features, out_features=out_features, k=k, trellis=trellis,
        suh=suh_arr, svh=svh_arr, bias=bias_arr, mcg=mcg, mul1=mul1,
    )
