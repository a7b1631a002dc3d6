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
from .layer import tensor_core_perm, tensor_core_perm_inverse
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


def unpack_trellis(packed, k: int, *, device="cuda") -> torch.Tensor:
    """Packed ``(..., 16*K)`` trellis words -> ``(..., 256)`` 16-bit codewords in
    kernel order (int16 storage of the uint16 bits); ``unpack_trellis``,
    ponyexl3/ref/trellis.py:153-214. The low K bits are what :func:`pack_trellis`
    takes."""
    if not 1 <= int(k) <= 8:
        raise ValueError(f"K must be in [1, 8], got {k}")
    if isinstance(packed, np.ndarray):
        packed = torch.from_numpy(np.ascontiguousarray(packed).astype(np.uint16).view(np.int16))
    arr = packed.to(device)
    if arr.dtype == torch.uint16:
        arr = arr.view(torch.int16)
    if arr.dtype != torch.int16 or arr.dim() < 1 or arr.shape[-1] != 16 * int(k):
        raise ValueError(f"expected 16-bit words with last dim {16 * int(k)}, got {arr.dtype} {tuple(arr.shape)}")
    arr = arr.contiguous()
    _check_cuda(arr, "packed")
    out = torch.empty(tuple(arr.shape[:-1]) + (256,), dtype=torch.int16, device=arr.device)
    n_tiles = out.numel() // 256
    if n_tiles:
        rc = _lib.load().exl3_unpack_trellis(_ptr(arr), n_tiles, int(k), _ptr(out), _stream())
        _lib.check(rc, "exl3_unpack_trellis")
    return out


_perm_cache: dict = {}


def _perm_tensors(device):
    key = str(device)
    if key not in _perm_cache:
        _perm_cache[key] = (torch.from_numpy(tensor_core_perm().astype(np.int64)).to(device),
                            torch.from_numpy(tensor_core_perm_inverse().astype(np.int64)).to(device))
    return _perm_cache[key]


def inner_to_kernel_tiles(inner: torch.Tensor) -> torch.Tensor:
    """(in, out) matrix -> (in/16 * out/16, 256) fp32 tiles in kernel order, tiles
    enumerated row-major over (tile row, tile column) (``_inner_to_kernel_tiles``,
    ponyexl3/convert/direct.py:409-419)."""
    if inner.dim() != 2 or inner.shape[0] % 16 or inner.shape[1] % 16:
        raise ValueError(f"expected 2D matrix with 16-multiple dims, got {tuple(inner.shape)}")
    tk, tn = inner.shape[0] // 16, inner.shape[1] // 16
    perm, _ = _perm_tensors(inner.device)
    row_major = inner.reshape(tk, 16, tn, 16).permute(0, 2, 1, 3).reshape(tk * tn, 256)
    return row_major[:, perm].to(torch.float32).contiguous()


def kernel_tiles_to_inner(tiles: torch.Tensor, rows: int, cols: int) -> torch.Tensor:
    """Inverse of :func:`inner_to_kernel_tiles` (``_kernel_tiles_to_inner``,
    ponyexl3/convert/direct.py:422-433)."""
    tk, tn = rows // 16, cols // 16
    if tuple(tiles.shape) != (tk * tn, 256):
        raise ValueError(f"decoded tile shape {tuple(tiles.shape)} does not match {(rows, cols)}")
    _, inv = _perm_tensors(tiles.device)
    return tiles[:, inv].reshape(tk, tn, 16, 16).permute(0, 2, 1, 3).reshape(rows, cols).contiguous()


def quantize_inner_matrix_direct(inner, *, k: int, cb: int = 0, return_states: bool = False,
                                 verify_roundtrip: bool = False,
                                 max_scratch_bytes: int = DEFAULT_MAX_SCRATCH_BYTES, device="cuda"):
    """Quantize an inner-domain matrix tile by tile, without LDL error feedback:
    ``(packed trellis (in/16, out/16, 16K) int16, states or None, reconstructed (in,
    out) fp32)``, all on the device (``quantize_inner_matrix_direct[_mlx]``,
    ponyexl3/convert/direct.py:469-556). The packed trellis is what
    ``exl3_decode_full`` and the forward kernels read."""
    w = torch.as_tensor(inner, dtype=torch.float32, device=device)
    tiles = inner_to_kernel_tiles(w)
    q, idx = quantize_tiles(tiles, k, cb, max_scratch_bytes=max_scratch_bytes, device=w.device)
    tk, tn = w.shape[0] // 16, w.shape[1] // 16
    states = idx.reshape(tk, tn, 256)
    packed = pack_trellis(states & ((1 << int(k)) - 1), k, device=w.device)
    if verify_roundtrip and not torch.equal(unpack_trellis(packed, k, device=w.device), states):
        raise AssertionError("direct quantization produced non-round-trippable trellis")
    recon = kernel_tiles_to_inner(q, w.shape[0], w.shape[1])
    return packed, (states if return_states else None), recon
