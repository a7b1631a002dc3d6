"""Encoder side of the trellis on the GPU: tail-biting Viterbi search for batches
of 16x16 tiles and the K-bit symbol packer.

Host-side mirror of ``ponyexl3/convert/metal_search.py:254-315``
(``quantize_tiles_mlx`` / ``quantize_tiles_mlx_np``: same arguments, same
``ValueError`` cases, same ``max_scratch_bytes`` bound on the backpointer scratch)
and ``ponyexl3/convert/mlx_trellis.py:66-84`` (``pack_trellis_mlx``). The
converter around them (Hessian capture, LDL feedback, bit allocation) is not part
of this package.
"""

from __future__ import annotations

import numpy as np
import torch

from . import _lib
from .ops import _check_cuda, _ptr, _stream

# Bound on the backpointer scratch of one launch. The reference's default is
# 256 MiB; here the default is what keeps every CU of the device busy (about
# 2 GiB at K = 4), because a launch walks over any number of tiles with the slots
# it has.
DEFAULT_MAX_SCRATCH_BYTES = 4 << 30


def scratch_bytes_per_tile(k: int) -> int:
    """Backpointer bytes one resident tile needs (``_scratch_bytes_per_tile``,
    metal_search.py:206-210; the two cost rows live in LDS here)."""
    return int(_lib.load().exl3_quantize_slot_bytes(int(k)))


def quantize_tiles(tiles, k: int, cb: int = 0, *, max_scratch_bytes: int = DEFAULT_MAX_SCRATCH_BYTES,
                   device="cuda"):
    """Quantize kernel-order tiles ``(N, 256)`` fp32 with the trellis search.

    Returns ``(quantized_tiles, indices)`` device tensors shaped like the input:
    fp32 decoded values and full 16-bit codewords (int16 storage of the uint16
    bits); pass ``indices & ((1 << k) - 1)`` to :func:`pack_trellis`."""
    if not 2 <= int(k) <= 8:
        raise ValueError("trellis search currently supports K in [2, 8]")
    if int(cb) not in (0, 1, 2):
        raise ValueError(f"unknown codebook {cb}")
    arr = torch.as_tensor(tiles, dtype=torch.float32, device=device)
    if arr.dim() == 1:
        arr = arr.reshape(1, 256)
    if arr.dim() != 2 or arr.shape[1] != 256:
        raise ValueError(f"expected tiles shape (N, 256), got {tuple(arr.shape)}")
    n_tiles = arr.shape[0]
    if n_tiles == 0:
        raise ValueError("expected at least one tile")
    if max_scratch_bytes <= 0:
        raise ValueError("max_scratch_bytes must be positive")
    arr = arr.contiguous()
    _check_cuda(arr, "tiles")
    lib = _lib.load()
    slot = scratch_bytes_per_tile(k)
    want = int(lib.exl3_quantize_workspace_bytes(n_tiles, int(k)))
    nbytes = max(slot, min(want, (max_scratch_bytes // slot) * slot))
    ws = torch.empty(nbytes, dtype=torch.uint8, device=arr.device)
    q = torch.empty_like(arr)
    idx = torch.empty((n_tiles, 256), dtype=torch.int16, device=arr.device)
    rc = lib.exl3_quantize_tiles(_ptr(arr), n_tiles, int(k), int(cb), _ptr(q), _ptr(idx), _ptr(ws),
                                 nbytes, _stream())
    _lib.check(rc, "exl3_quantize_tiles")
    return q, idx


def quantize_tiles_np(tiles: np.ndarray, k: int, cb: int = 0, *,
                      max_scratch_bytes: int = DEFAULT_MAX_SCRATCH_BYTES, device="cuda"):
    """NumPy wrapper (``quantize_tiles_mlx_np``, metal_search.py:306-315):
    ``(q_tiles fp32, indices uint16)``."""
    q, idx = quantize_tiles(np.asarray(tiles, dtype=np.float32), k, cb,
                            max_scratch_bytes=max_scratch_bytes, device=device)
    return q.cpu().numpy(), idx.cpu().numpy().view(np.uint16)


def pack_trellis(encoded, k: int, *, device="cuda") -> torch.Tensor:
    """Pack the low K bits of ``encoded (..., 256)`` into ``(..., 16*K)`` trellis
    words (int16 storage of the uint16 bits), matching ``ponyexl3.ref.trellis.
    pack_trellis`` bit for bit (``pack_trellis_mlx``, mlx_trellis.py:66-84)."""
    if not 1 <= int(k) <= 8:
        raise ValueError(f"K must be in [1, 8], got {k}")
    if isinstance(encoded, np.ndarray):
        encoded = torch.from_numpy(np.ascontiguousarray(encoded).astype(np.uint16).view(np.int16))
    arr = encoded.to(device)
    if arr.dtype not in (torch.int16, torch.uint16):
        arr = arr.to(torch.int16)
    if arr.dim() < 1 or arr.shape[-1] != 256:
        raise ValueError(f"expected encoded last dim 256, got {tuple(arr.shape)}")
    arr = arr.contiguous()
    _check_cuda(arr, "encoded")
    out = torch.empty(tuple(arr.shape[:-1]) + (16 * int(k),), dtype=torch.int16, device=arr.device)
    n_tiles = arr.numel() // 256
    if n_tiles:
        rc = _lib.load().exl3_pack_trellis(_ptr(arr), n_tiles, int(k), _ptr(out), _stream())
        _lib.check(rc, "exl3_pack_trellis")
    return out
