"""numpy front end of the CPU oracle (``exl3_oracle.c``).

TEST INFRASTRUCTURE ONLY: imported by tests/, by the smoke check and by the
cpu_baseline leg of bench.py, never by the shipped package.

Every function here forwards to the C restatement of ``ponyexl3/ref`` (the
citations live beside the C functions). The MoE chain has no CPU twin in the
reference; ``moe_experts_forward`` composes the pinned linear forward with the
activation of ``ponyexl3/mlx/exl3_moe.py:62-75`` and the unfused chain of
``ponyexl3/mlx/exl3_moe.py:648-682``.
"""

from __future__ import annotations

import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "_build", "libexl3_oracle.so")

_u16p = ctypes.POINTER(ctypes.c_uint16)
_f32p = ctypes.POINTER(ctypes.c_float)
_f64p = ctypes.POINTER(ctypes.c_double)
_i32p = ctypes.POINTER(ctypes.c_int32)


def build(force: bool = False) -> str:
    """Compile the oracle with gcc (``make -C oracle``)."""
    if force or not os.path.exists(_LIB_PATH):
        args = ["make", "-C", _HERE] + (["-B"] if force else [])
        subprocess.run(args, check=True, stdout=subprocess.DEVNULL)
    return _LIB_PATH


_lib = None


def lib() -> ctypes.CDLL:
    global _lib
    if _lib is None:
        build()
        L = ctypes.CDLL(_LIB_PATH)
        L.exl3o_decode_cw.restype = ctypes.c_uint16
        L.exl3o_decode_cw.argtypes = [ctypes.c_uint32, ctypes.c_int]
        L.exl3o_decode_table.argtypes = [ctypes.c_int, _u16p]
        L.exl3o_unpack_tile.argtypes = [_u16p, ctypes.c_int, _u16p]
        L.exl3o_pack_tile.argtypes = [_u16p, ctypes.c_int, _u16p]
        L.exl3o_perm.argtypes = [_i32p]
        L.exl3o_decode_tile.argtypes = [_u16p, ctypes.c_int, ctypes.c_int, _u16p]
        L.exl3o_decode_trellis.argtypes = [_u16p] + [ctypes.c_int] * 6 + [_u16p]
        L.exl3o_hadamard128.argtypes = [_f32p, ctypes.c_int, ctypes.c_int, _u16p, _u16p, _f32p]
        L.exl3o_linear_forward.argtypes = (
            [_u16p] + [ctypes.c_int] * 4 + [_u16p] * 5 + [ctypes.c_int] + [_u16p] * 3
        )
        L.exl3o_linear_forward_bs1.argtypes = [_u16p] + [ctypes.c_int] * 4 + [_u16p] * 4
        L.exl3o_half_to_float.argtypes = [_u16p, _f32p, ctypes.c_size_t]
        L.exl3o_float_to_half.argtypes = [_f32p, _u16p, ctypes.c_size_t]
        L.exl3o_double_to_half.argtypes = [_f64p, _u16p, ctypes.c_size_t]
        L.exl3o_quantize_tile_exact.argtypes = [_f32p] + [ctypes.c_int] * 4 + [_u16p, _f32p]
        L.exl3o_quantize_tiles_search.argtypes = [_f32p] + [ctypes.c_int] * 3 + [_f32p, _u16p]
        L.exl3o_num_threads.restype = ctypes.c_int
        L.exl3o_set_num_threads.argtypes = [ctypes.c_int]
        _lib = L
    return _lib


def _p16(a):
    return None if a is None else a.ctypes.data_as(_u16p)


def _as_u16(a, name="array"):
    """fp16 / int16 / uint16 array -> contiguous uint16 view of the same bits."""
    if a is None:
        return None
    a = np.ascontiguousarray(a)
    if a.dtype == np.float16 or a.dtype == np.int16:
        return a.view(np.uint16)
    if a.dtype == np.uint16:
        return a
    raise TypeError(f"{name}: expected a 16-bit array, got {a.dtype}")


def _fp16_scale(v):
    """suh/svh as fp16 bits. Packed int16 bitfields expand as ref/signs.py:8-27
    (bit set means -1, least significant bit is the first channel)."""
    if v is None:
        return None
    v = np.asarray(v)
    if v.dtype in (np.float16, np.float32):
        return np.ascontiguousarray(v.astype(np.float16)).view(np.uint16)
    bits = (v.astype(np.uint16).reshape(-1, 1) >> np.arange(16, dtype=np.uint16)) & 1
    return np.where(bits != 0, -1.0, 1.0).astype(np.float16).reshape(-1).view(np.uint16)


def unpack_signs_or_pass(v):
    s = _fp16_scale(v)
    return None if s is None else s.view(np.float16)


def decode_cw(cw: int, cb: int) -> np.float16:
    bits = np.array([lib().exl3o_decode_cw(int(cw) & 0xFFFF, int(cb))], dtype=np.uint16)
    return bits.view(np.float16)[0]


def decode_table(cb: int) -> np.ndarray:
    out = np.empty(65536, dtype=np.uint16)
    lib().exl3o_decode_table(int(cb), _p16(out))
    return out.view(np.float16)


def unpack_tile(packed: np.ndarray, k: int) -> np.ndarray:
    packed = _as_u16(packed)
    if packed.shape != (16 * k,):
        raise ValueError(f"expected packed shape ({16 * k},), got {packed.shape}")
    out = np.empty(256, dtype=np.uint16)
    if lib().exl3o_unpack_tile(_p16(packed), k, _p16(out)):
        raise ValueError(f"K must be in [1, 8], got {k}")
    return out


def pack_tile(encoded: np.ndarray, k: int) -> np.ndarray:
    encoded = np.ascontiguousarray(encoded, dtype=np.uint16)
    if encoded.shape != (256,):
        raise ValueError(f"expected encoded shape (256,), got {encoded.shape}")
    out = np.empty(16 * k, dtype=np.uint16)
    if lib().exl3o_pack_tile(_p16(encoded), k, _p16(out)):
        raise ValueError(f"K must be in [1, 8], got {k}")
    return out


def pack_trellis(encoded: np.ndarray, k: int) -> np.ndarray:
    """(tiles_k, tiles_n, 256) K-bit values -> (tiles_k, tiles_n, 16K) uint16."""
    tk, tn, n = encoded.shape
    if n != 256:
        raise ValueError("expected last dim 256")
    out = np.empty((tk, tn, 16 * k), dtype=np.uint16)
    for i in range(tk):
        for j in range(tn):
            out[i, j] = pack_tile(encoded[i, j], k)
    return out


def unpack_trellis(packed: np.ndarray, k: int) -> np.ndarray:
    packed = _as_u16(packed)
    tk, tn, _ = packed.shape
    out = np.empty((tk, tn, 256), dtype=np.uint16)
    for i in range(tk):
        for j in range(tn):
            out[i, j] = unpack_tile(packed[i, j], k)
    return out


def tensor_core_perm() -> np.ndarray:
    out = np.empty(256, dtype=np.int32)
    lib().exl3o_perm(out.ctypes.data_as(_i32p))
    return out


def decode_tile(packed: np.ndarray, k: int, cb: int) -> np.ndarray:
    packed = _as_u16(packed)
    out = np.empty(256, dtype=np.uint16)
    if lib().exl3o_decode_tile(_p16(packed), k, int(cb), _p16(out)):
        raise ValueError("bad K")
    return out.view(np.float16).reshape(16, 16)


def decode_trellis(trellis, k, cb, tn_offset=0, tn_count=None) -> np.ndarray:
    trellis = _as_u16(trellis, "trellis")
    if trellis.ndim != 3:
        raise ValueError("trellis must be 3D")
    in_tiles, out_tiles, ps = trellis.shape
    if ps != 16 * k:
        raise ValueError(f"packed size {ps} != expected {16 * k} for K={k}")
    if tn_count is None:
        tn_count = out_tiles - tn_offset
    out = np.empty((in_tiles * 16, tn_count * 16), dtype=np.uint16)
    rc = lib().exl3o_decode_trellis(
        _p16(trellis), in_tiles, out_tiles, k, int(cb), tn_offset, tn_count, _p16(out)
    )
    if rc:
        raise ValueError(f"decode_trellis failed ({rc})")
    return out.view(np.float16)


def had_r_128(x, pre_scale=None, post_scale=None) -> np.ndarray:
    x = np.ascontiguousarray(x, dtype=np.float32)
    if x.ndim != 2:
        raise ValueError("had_r_128 expects 2D input (rows, features)")
    rows, n = x.shape
    out = np.empty_like(x)
    rc = lib().exl3o_hadamard128(
        x.ctypes.data_as(_f32p), rows, n, _p16(_fp16_scale(pre_scale)),
        _p16(_fp16_scale(post_scale)), out.ctypes.data_as(_f32p),
    )
    if rc:
        raise ValueError(f"feature dim {n} not divisible by 128")
    return out


def linear_forward(trellis, k, cb, suh, svh, x, bias=None, w_inner=None, taps=False):
    """fp16 forward of one EXL3 linear; x (..., in) fp16 -> (..., out) fp16."""
    trellis = _as_u16(trellis, "trellis")
    in_tiles, out_tiles, ps = trellis.shape
    if ps != 16 * k:
        raise ValueError("trellis last dim does not match K")
    x = np.asarray(x, dtype=np.float16)
    lead = x.shape[:-1]
    x2 = np.ascontiguousarray(x.reshape(-1, in_tiles * 16))
    rows = x2.shape[0]
    y = np.empty((rows, out_tiles * 16), dtype=np.uint16)
    xh = np.empty((rows, in_tiles * 16), dtype=np.uint16) if taps else None
    yraw = np.empty((rows, out_tiles * 16), dtype=np.uint16) if taps else None
    wi = None if w_inner is None else _as_u16(np.asarray(w_inner, dtype=np.float16))
    b = None if bias is None else _as_u16(np.asarray(bias, dtype=np.float16))
    rc = lib().exl3o_linear_forward(
        _p16(trellis), in_tiles, out_tiles, k, int(cb), _p16(_fp16_scale(suh)),
        _p16(_fp16_scale(svh)), _p16(b), _p16(wi), _p16(x2.view(np.uint16)), rows,
        _p16(y), _p16(xh), _p16(yraw),
    )
    if rc:
        raise ValueError(f"linear_forward failed ({rc})")
    yv = y.view(np.float16).reshape(lead + (out_tiles * 16,))
    if taps:
        return yv, xh.view(np.float16), yraw.view(np.float16)
    return yv


def linear_forward_bs1(trellis, k, cb, suh, svh, x):
    trellis = _as_u16(trellis, "trellis")
    in_tiles, out_tiles, _ = trellis.shape
    x = np.ascontiguousarray(np.asarray(x, dtype=np.float16).reshape(-1))
    y = np.empty(out_tiles * 16, dtype=np.uint16)
    rc = lib().exl3o_linear_forward_bs1(
        _p16(trellis), in_tiles, out_tiles, k, int(cb), _p16(_fp16_scale(suh)),
        _p16(_fp16_scale(svh)), _p16(x.view(np.uint16)), _p16(y),
    )
    if rc:
        raise ValueError(f"linear_forward_bs1 failed ({rc})")
    return y.view(np.float16)


def reconstruct_public_weights(trellis, suh, svh, k, cb) -> np.ndarray:
    """diag(suh) H W H diag(svh) in fp32, cast to fp16 (ref/reconstruct.py:26-49)."""
    w = decode_trellis(trellis, k, cb).astype(np.float32)
    if suh is not None:
        # preapply_had_left: H @ W per 128-row block == (W^T H)^T
        w = had_r_128(np.ascontiguousarray(w.T)).T.copy()
        w *= unpack_signs_or_pass(suh).astype(np.float32).reshape(-1, 1)
    if svh is not None:
        w = had_r_128(np.ascontiguousarray(w))
        w *= unpack_signs_or_pass(svh).astype(np.float32).reshape(1, -1)
    return w.astype(np.float16)


def glu(g: np.ndarray, u: np.ndarray, activation: str = "silu") -> np.ndarray:
    """fp16 gate activation, evaluated in fp32 and rounded once
    (ponyexl3/mlx/exl3_moe.py:62-75)."""
    g = g.astype(np.float32)
    u = u.astype(np.float32)
    if activation == "silu":
        h = (g / (np.float32(1.0) + np.exp(-g))) * u
    elif activation == "gelu":
        t = np.float32(0.797884560803) * (g + np.float32(0.044715) * g * g * g)
        h = np.float32(0.5) * g * (np.float32(1.0) + np.tanh(t)) * u
    else:
        raise ValueError(f"unsupported MoE activation {activation!r}")
    return h.astype(np.float16)


def moe_experts_forward(experts, x, indices, k, cb, activation="silu"):
    """Unfused expert chain (ponyexl3/mlx/exl3_moe.py:648-682).

    experts: list of dicts with gate/up/down = (trellis, suh, svh).
    x (T, D) fp16, indices (T, kk) int -> (T, kk, D) fp16.
    """
    x = np.asarray(x, dtype=np.float16)
    T, D = x.shape
    kk = indices.shape[1]
    out = np.empty((T, kk, D), dtype=np.float16)
    for t in range(T):
        for s in range(kk):
            e = experts[int(indices[t, s])]
            g = linear_forward(*e["gate"][:1], k, cb, e["gate"][1], e["gate"][2], x[t : t + 1])
            u = linear_forward(*e["up"][:1], k, cb, e["up"][1], e["up"][2], x[t : t + 1])
            h = glu(g, u, activation)
            out[t, s] = linear_forward(*e["down"][:1], k, cb, e["down"][1], e["down"][2], h)[0]
    return out


def quantize_tile_exact(w: np.ndarray, k: int, cb: int, max_pins: int = 4):
    """Exact Viterbi, float64 path costs (``quantize_tile_reference``,
    ponyexl3/convert/reference_search.py:59-87). w: (n,) fp32 in kernel order, n = 256
    for a tile (shorter trellises are for brute-force checks). Returns (states u16,
    decoded fp32)."""
    w = np.ascontiguousarray(w, dtype=np.float32).reshape(-1)
    states = np.empty(w.size, dtype=np.uint16)
    decoded = np.empty(w.size, dtype=np.float32)
    rc = lib().exl3o_quantize_tile_exact(w.ctypes.data_as(_f32p), w.size, int(k), int(cb), int(max_pins),
                                         _p16(states), decoded.ctypes.data_as(_f32p))
    if rc:
        raise ValueError(f"bad arguments (K={k}, cb={cb})")
    return states, decoded


def quantize_tiles_search(tiles: np.ndarray, k: int, cb: int):
    """The production search's arithmetic (``quantize_tiles_mlx``,
    ponyexl3/convert/metal_search.py:63-196, 254-303). tiles: (N, 256) fp32 in kernel
    order. Returns (q_tiles fp32 (N, 256), full 16-bit codewords u16 (N, 256))."""
    if not 2 <= int(k) <= 8:
        raise ValueError("trellis search supports K in [2, 8]")
    tiles = np.ascontiguousarray(tiles, dtype=np.float32)
    if tiles.ndim == 1:
        tiles = tiles.reshape(1, 256)
    if tiles.ndim != 2 or tiles.shape[1] != 256:
        raise ValueError(f"expected tiles shape (N, 256), got {tiles.shape}")
    q = np.empty_like(tiles)
    idx = np.empty(tiles.shape, dtype=np.uint16)
    rc = lib().exl3o_quantize_tiles_search(tiles.ctypes.data_as(_f32p), tiles.shape[0], int(k), int(cb),
                                           q.ctypes.data_as(_f32p), _p16(idx))
    if rc:
        raise ValueError(f"bad arguments (K={k}, cb={cb})")
    return q, idx


def num_threads() -> int:
    return int(lib().exl3o_num_threads())


def set_num_threads(n: int) -> None:
    lib().exl3o_set_num_threads(int(n))
