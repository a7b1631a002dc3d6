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


def pack_trellis_tiles(symbols: np.ndarray, k: int) -> np.ndarray:
    """K-bit symbols (..., 256) -> packed tiles (..., 16*K) uint16, the bit order of
    ``pack_trellis_tile`` (ponyexl3/ref/trellis.py:13-49): symbol c fills stream bits
    [c*K, (c+1)*K) most significant bit first, and stream bit b is bit 31 - b % 32 of
    little-endian 32-bit word b // 32 of the tile."""
    sym = np.asarray(symbols).astype(np.uint32) & ((1 << k) - 1)
    lead = sym.shape[:-1]
    shifts = np.arange(k - 1, -1, -1, dtype=np.uint32)
    bits = ((sym[..., None] >> shifts) & 1).reshape(lead + (8 * k, 32))  # stream order, 32 per word
    weights = (np.uint32(1) << np.arange(31, -1, -1, dtype=np.uint32))
    words = (bits * weights).sum(axis=-1, dtype=np.uint64).astype("<u4")
    return np.ascontiguousarray(words).view("<u2").reshape(lead + (16 * k,)).astype(np.uint16)


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
    ref_compatible: bool = False,
) -> EXL3Layer:
    """Seeded synthetic layer. Every uint16 fill is a legal bitstream, so by default
    the trellis is raw random words (``numpy.random.default_rng(seed)``); signs are
    ``where(rng.random(n) > 0.5, -1, 1)`` drawn after the trellis, suh first.

    ``ref_compatible=True`` reproduces ``ponyexl3.ref.synthetic.make_exl3_layer``
    (ponyexl3/ref/synthetic.py:13-82) bit for bit: tile (i, j) packs 256 symbols
    ``integers(0, 2**16, 256, uint32) & (2**K - 1)`` drawn from its own generator
    seeded ``seed*1000 + i*10 + j``; signs and bias come from a separate
    ``default_rng(seed)``, suh first, then svh, then ``standard_normal(out)`` cast to
    fp16 and scaled by 0.01 in fp16. One generator per tile makes it slow for large
    layers (65 536 tiles at 4096 x 4096), which is why it is not the default."""
    rng = np.random.default_rng(seed)
    in_tiles, out_tiles = in_features // 16, out_features // 16
    if ref_compatible:
        sym = np.empty((in_tiles, out_tiles, 256), dtype=np.uint32)
        for i in range(in_tiles):
            for j in range(out_tiles):
                sym[i, j] = np.random.default_rng(seed * 1000 + i * 10 + j).integers(
                    0, 2**16, size=256, dtype=np.uint32)
        trellis = pack_trellis_tiles(sym, k)
    else:
        trellis = rng.integers(0, 65536, size=(in_tiles, out_tiles, 16 * k), dtype=np.uint16)

    def _signs(n):
        return np.where(rng.random(n) > 0.5, -1.0, 1.0).astype(np.float16)

    suh_arr = _signs(in_features) if isinstance(suh, str) else suh
    svh_arr = _signs(out_features) if isinstance(svh, str) else svh
    if not bias:
        bias_arr = None
    elif ref_compatible:
        bias_arr = rng.standard_normal(out_features).astype(np.float16) * np.float16(0.01)
    else:
        bias_arr = (rng.standard_normal(out_features) * 0.01).astype(np.float16)
    return EXL3Layer(
        key="test.layer" if ref_compatible and key == "synthetic.layer" else key,
        in_features=in_features, out_features=out_features, k=k, trellis=trellis,
        suh=suh_arr, svh=svh_arr, bias=bias_arr, mcg=mcg, mul1=mul1,
    )
