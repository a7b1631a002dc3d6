"""Inner operators on torch (ROCm) tensors, thin wrappers over the C ABI.

These mirror the reference's inner operator API
(``ponyexl3/mlx/gemv_metal.py:717-743,1481-1515`` and
``ponyexl3/mlx/layer_state.py:133-141``): same names, argument meaning and
ValueError-before-launch behaviour; arrays are torch tensors on the GPU and
all launches go to torch's current HIP stream. PyTorch only provides device
memory and streams here; every result is produced by libexl3_hip.so.
"""

from __future__ import annotations

import ctypes

import numpy as np
import torch

from . import _lib

_workspaces: dict = {}
# Buffers that were replaced by larger ones stay allocated: a HIP graph captured
# earlier still replays launches that point into them.
_retired: list = []


def _check_cuda(t: torch.Tensor, name: str) -> None:
    if not isinstance(t, torch.Tensor):
        raise ValueError(f"{name} must be a torch.Tensor")
    if not t.is_cuda:
        raise ValueError(f"{name} must live on the GPU (got device {t.device})")
    if not t.is_contiguous():
        raise ValueError(f"{name} must be contiguous")


def _ptr(t):
    return None if t is None else ctypes.c_void_p(t.data_ptr())


def _stream():
    return ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)


def _buffer_key(device):
    """Scratch buffers and counters belong to one (device, stream) pair: launches on
    one stream are ordered, so they can share a buffer; two streams of a device
    running EXL3 layers at the same time must not (the group counters and partial
    rows of one launch would be read by the other)."""
    index = device.index if device.index is not None else torch.cuda.current_device()
    return (device.type, index, torch.cuda.current_stream(index).cuda_stream)


def workspace(device, nbytes: int) -> torch.Tensor:
    """Scratch buffer of the current (device, stream), grown on demand."""
    key = _buffer_key(device)
    buf = _workspaces.get(key)
    if buf is None or buf.numel() < nbytes:
        if buf is not None:
            _retired.append(buf)
        buf = torch.empty(max(int(nbytes), 1 << 20), dtype=torch.uint8, device=device)
        _workspaces[key] = buf
    return buf


_gemm_workspaces: dict = {}


def gemm_workspace(device, nbytes: int):
    """Scratch of the current (device, stream) for the prefill GEMM's fp32 partial
    tiles (kept apart from ``workspace``, which holds the GEMM's operands during a
    layer forward)."""
    if nbytes <= 0:
        return None
    key = _buffer_key(device)
    buf = _gemm_workspaces.get(key)
    if buf is None or buf.numel() < nbytes:
        if buf is not None:
            _retired.append(buf)
        buf = torch.empty(int(nbytes), dtype=torch.uint8, device=device)
        _gemm_workspaces[key] = buf
    return buf


_counters: dict = {}


def sync_counters(device, n: int) -> torch.Tensor:
    """int32 array of group counters / accumulators of the current (device, stream) for
    the one-launch layer kernel and the MoE chain, at least ``n + 2`` ints. Zeroed when
    created; the kernels leave it zero, so it is reused as is. Its last int is the
    status word the library sets when a split reduction gives up
    (``check_counters`` reads it)."""
    key = _buffer_key(device)
    buf = _counters.get(key)
    if buf is None or buf.numel() < n + 2:
        if buf is not None:
            _retired.append(buf)
        buf = torch.zeros(max(int(n) + 2, 4096), dtype=torch.int32, device=device)
        _counters[key] = buf
    return buf


def check_counters(device) -> None:
    """Waits for the current stream and raises RuntimeError if a split reduction on its
    counters gave up (``exl3_counters_status``: the array was not zero on entry, or two
    calls overlapped on it; the affected outputs are NaN) or if the array is not all zero
    as every finished launch leaves it. Either way the array is zeroed again, so the
    next call starts clean. A synchronisation: for tests and debugging, not the hot path."""
    buf = _counters.get(_buffer_key(device))
    if buf is None:
        return
    rc = _lib.load().exl3_counters_status(_ptr(buf), buf.numel(), _stream())
    dirty = int(buf.ne(0).sum())
    if rc != _lib.EXL3_OK or dirty:
        buf.zero_()
        torch.cuda.current_stream().synchronize()
        if rc != _lib.EXL3_OK:
            _lib.check(rc, "exl3_counters_status")
        raise RuntimeError(f"{dirty} words of the split-reduction counters were left non-zero")


def as_trellis_tensor(trellis, device=None) -> torch.Tensor:
    """numpy/torch uint16|int16 (in_tiles, out_tiles, 16K) -> int16 GPU tensor
    holding the same bits."""
    if isinstance(trellis, np.ndarray):
        if trellis.dtype not in (np.uint16, np.int16):
            raise ValueError(f"trellis must be uint16/int16, got {trellis.dtype}")
        t = torch.from_numpy(np.ascontiguousarray(trellis).view(np.int16))
    else:
        t = trellis
        if t.dtype == torch.uint16:
            t = t.view(torch.int16)
        if t.dtype != torch.int16:
            raise ValueError(f"trellis must be uint16/int16, got {t.dtype}")
    if device is not None:
        t = t.to(device)
    return t.contiguous()


def _trellis_dims(trellis: torch.Tensor, k: int):
    _check_cuda(trellis, "trellis")
    if trellis.dtype not in (torch.int16, torch.uint16):
        raise ValueError(f"trellis must be a 16-bit integer tensor, got {trellis.dtype}")
    if trellis.dim() != 3:
        raise ValueError("trellis must be 3D (in_tiles, out_tiles, 16*K)")
    if not 1 <= int(k) <= 8:
        raise ValueError(f"K must be in [1, 8], got {k}")
    in_tiles, out_tiles, ps = trellis.shape
    if ps != 16 * k:
        raise ValueError(f"packed size {ps} != expected {16 * k} for K={k}")
    return int(in_tiles), int(out_tiles)


def _half(t: torch.Tensor, name: str) -> torch.Tensor:
    _check_cuda(t, name)
    if t.dtype != torch.float16:
        raise ValueError(f"{name} must be float16, got {t.dtype}")
    return t


def decode_full(trellis, k: int, cb: int, tn_offset: int = 0, tn_count: int | None = None):
    """Trellis -> fp16 W (in, 16*tn_count) (``decode_full_mlx``,
    ponyexl3/mlx/gemv_metal.py:717-743)."""
    in_tiles, out_tiles = _trellis_dims(trellis, k)
    if tn_count is None:
        tn_count = out_tiles - tn_offset
    if tn_offset < 0 or tn_count < 0 or tn_offset + tn_count > out_tiles:
        raise ValueError("slice exceeds output features")
    w = torch.empty((in_tiles * 16, tn_count * 16), dtype=torch.float16, device=trellis.device)
    if w.numel() == 0:
        return w
    rc = _lib.load().exl3_decode_full(
        _ptr(trellis), in_tiles, out_tiles, int(k), int(cb), int(tn_offset), int(tn_count),
        _ptr(w), _stream(),
    )
    _lib.check(rc, "exl3_decode_full")
    return w


def decode_full_eg(trellis, k: int, cb: int, *, tiles_per_e: int):
    """Stacked-expert trellis -> contiguous (E, in, 16*tiles_per_e) fp16
    (``decode_full_eg_mlx``, ponyexl3/mlx/gemv_metal.py:746-774)."""
    in_tiles, out_tiles = _trellis_dims(trellis, k)
    if tiles_per_e < 1 or out_tiles % tiles_per_e != 0:
        raise ValueError("out_tiles not divisible by tiles_per_e")
    w = torch.empty((out_tiles // tiles_per_e, in_tiles * 16, tiles_per_e * 16), dtype=torch.float16,
                    device=trellis.device)
    if w.numel() == 0:
        return w
    rc = _lib.load().exl3_decode_full_eg(
        _ptr(trellis), in_tiles, out_tiles, int(k), int(cb), int(tiles_per_e), _ptr(w), _stream())
    _lib.check(rc, "exl3_decode_full_eg")
    return w


def decode_full_t(trellis, k: int, cb: int, tn_offset: int = 0, tn_count: int | None = None):
    """Trellis -> fp16 W^T (16*tn_count, in) (``decode_full_t_mlx``,
    ponyexl3/mlx/gemv_metal.py:841-866)."""
    in_tiles, out_tiles = _trellis_dims(trellis, k)
    if tn_count is None:
        tn_count = out_tiles - tn_offset
    if tn_offset < 0 or tn_count < 0 or tn_offset + tn_count > out_tiles:
        raise ValueError("slice exceeds output features")
    w = torch.empty((tn_count * 16, in_tiles * 16), dtype=torch.float16, device=trellis.device)
    if w.numel() == 0:
        return w
    rc = _lib.load().exl3_decode_full_t(
        _ptr(trellis), in_tiles, out_tiles, int(k), int(cb), int(tn_offset), int(tn_count),
        _ptr(w), _stream())
    _lib.check(rc, "exl3_decode_full_t")
    return w


def reconstruct_inner(trellis, k: int, cb: int, n_offset: int = 0, n_count: int | None = None):
    """Inner weight W (in, n_count) fp16 for a 128-aligned column range
    (``reconstruct_inner``, ponyexl3/ref/reconstruct.py:13-23; the reference
    rejects unaligned offsets the same way, ref/decode.py:46-51)."""
    _, out_tiles = _trellis_dims(trellis, k)
    if n_count is None:
        n_count = out_tiles * 16 - n_offset
    if n_offset % 128 or n_count % 16 or n_offset < 0 or n_count < 0:
        raise ValueError("column slice must start on a multiple of 128 and cover whole tiles")
    return decode_full(trellis, k, cb, n_offset // 16, n_count // 16)


def _hadamard128_matrix(device) -> torch.Tensor:
    h = torch.ones((1, 1), dtype=torch.float32, device=device)
    while h.shape[0] < 128:
        h = torch.cat([torch.cat([h, h], dim=1), torch.cat([h, -h], dim=1)], dim=0)
    return h * (128.0 ** -0.5)


def reconstruct_public_weights(trellis, suh, svh, k: int, cb: int):
    """Public weight diag(suh) . H . W . H . diag(svh), fp32 arithmetic, one cast to
    fp16 (``reconstruct_public_weights``, ponyexl3/ref/reconstruct.py:26-49). The
    decode runs in the HIP kernel; the two blockwise Hadamard products are plain
    torch matmuls, this is a checking and export utility, not a forward path."""
    w = decode_full(trellis, k, cb).float()
    n_in, n_out = w.shape
    h = _hadamard128_matrix(w.device)
    if suh is not None:
        if n_in % 128:
            raise ValueError(f"in_features {n_in} not divisible by 128")
        w = torch.matmul(h, w.reshape(n_in // 128, 128, n_out)).reshape(n_in, n_out)
        w = w * suh.to(w.device).float().reshape(-1, 1)
    if svh is not None:
        if n_out % 128:
            raise ValueError(f"out_features {n_out} not divisible by 128")
        w = torch.matmul(w.reshape(n_in, n_out // 128, 128), h).reshape(n_in, n_out)
        w = w * svh.to(w.device).float().reshape(1, -1)
    return w.to(torch.float16)


def had128_pre(x2d: torch.Tensor, suh: torch.Tensor | None):
    """xh = fp16(had128(x * suh)); suh (in,) or stacked (n_sub, in) -> xh
    (rows, in) or (rows, n_sub, in). ``EXL3LayerRuntime.prepare_xh`` /
    ``_fused_prep`` (ponyexl3/mlx/layer_state.py:133-136, exl3_fused.py:44-60)."""
    _half(x2d, "x")
    if x2d.dim() != 2:
        raise ValueError("had128_pre expects 2D input (rows, features)")
    rows, n = x2d.shape
    if n % 128 != 0:
        raise ValueError(f"feature dim {n} not divisible by 128")
    n_sub = 1
    stacked = False
    if suh is not None:
        _half(suh, "suh")
        stacked = suh.dim() == 2
        n_sub = suh.shape[0] if stacked else 1
        if suh.shape[-1] != n:
            raise ValueError("suh length does not match the feature dim")
    shape = (rows, n_sub, n) if stacked else (rows, n)
    xh = torch.empty(shape, dtype=torch.float16, device=x2d.device)
    rc = _lib.load().exl3_had128_pre(_ptr(x2d), rows, n, _ptr(suh), n_sub, _ptr(xh), _stream())
    _lib.check(rc, "exl3_had128_pre")
    return xh


def had128_post(y: torch.Tensor, svh: torch.Tensor | None, bias: torch.Tensor | None = None):
    """out = fp16(had128(fp16(sum of y slices)) * svh) (+ bias).

    y: fp16 (rows, n), fp32 (rows, n) or fp32 (n_sum, rows, n) split-K partials.
    ``EXL3LayerRuntime.finish_y`` (ponyexl3/mlx/layer_state.py:138-141)."""
    _check_cuda(y, "y")
    if y.dtype == torch.float16:
        if y.dim() != 2:
            raise ValueError("fp16 y must be 2D (rows, features)")
        n_sum, (rows, n), is32 = 1, y.shape, 0
    elif y.dtype == torch.float32:
        if y.dim() == 2:
            n_sum, (rows, n) = 1, y.shape
        elif y.dim() == 3:
            n_sum, rows, n = y.shape
        else:
            raise ValueError("fp32 y must be (rows, n) or (n_sum, rows, n)")
        is32 = 1
    else:
        raise ValueError(f"y must be float16 or float32, got {y.dtype}")
    if n % 128 != 0:
        raise ValueError(f"feature dim {n} not divisible by 128")
    for name, v in (("svh", svh), ("bias", bias)):
        if v is not None:
            _half(v, name)
            if v.numel() != n:
                raise ValueError(f"{name} length does not match the feature dim")
    out = torch.empty((rows, n), dtype=torch.float16, device=y.device)
    rc = _lib.load().exl3_had128_post(
        _ptr(y), is32, int(n_sum), rows * n, int(rows), int(n), _ptr(svh), _ptr(bias), _ptr(out),
        _stream(),
    )
    _lib.check(rc, "exl3_had128_post")
    return out


def gemv_max_rows() -> int:
    return int(_lib.load().exl3_gemv_max_rows())


def linear_small_max_rows() -> int:
    """Rows up to which ``linear_forward(fused=True)`` uses the small- and
    medium-batch kernels (stacked ``suh`` included); above it the prefill GEMM runs."""
    return int(_lib.load().exl3_linear_small_max_rows())


def group_sub_from_tile_sub(tile_sub) -> torch.Tensor:
    """tile_sub (out_tiles,) -> per-128-column table; every run of 8 tiles must
    share one member (members have out_features % 128 == 0)."""
    ts = np.asarray(tile_sub.cpu() if isinstance(tile_sub, torch.Tensor) else tile_sub)
    ts = ts.astype(np.int64).reshape(-1)
    if ts.size % 8 != 0:
        raise ValueError("tile_sub length must be a multiple of 8")
    g = ts.reshape(-1, 8)
    if not (g == g[:, :1]).all():
        raise ValueError("tile_sub must be constant inside each 128-column group")
    return torch.from_numpy(g[:, 0].astype(np.int32).copy())


def inner_gem_fused(xh, trellis, k: int, cb: int, group_sub=None, group_tile=None, n_groups=None):
    """y (rows, 128*n_groups) fp32 = xh[:, sub(g), :] @ W for rows <= gemv_max_rows().

    xh (rows, n_sub, in) fp16. ``inner_gem_fused_mlx`` /
    ``_mapped_gemv`` (ponyexl3/mlx/gemv_metal.py:1481-1492, exl3_moe.py:139-171)
    with tile tables at 128-column granularity."""
    in_tiles, out_tiles = _trellis_dims(trellis, k)
    _half(xh, "xh")
    if xh.dim() != 3:
        raise ValueError("xh must be (rows, n_sub, in)")
    rows, n_sub, n_in = xh.shape
    if n_in != in_tiles * 16:
        raise ValueError(f"xh features {n_in} != trellis in_features {in_tiles * 16}")
    if n_in % 128 or out_tiles % 8:
        raise ValueError("in/out features must be multiples of 128")
    if not 1 <= rows <= gemv_max_rows():
        raise ValueError(f"rows must be in [1, {gemv_max_rows()}], got {rows}")
    if n_groups is None:
        n_groups = out_tiles // 8 if group_tile is None else int(group_tile.numel())
    for name, v, need in (("group_sub", group_sub, n_sub > 1), ("group_tile", group_tile, False)):
        if v is None:
            if need:
                raise ValueError(f"{name} is required when n_sub > 1")
            continue
        _check_cuda(v, name)
        if v.dtype != torch.int32 or v.numel() != n_groups:
            raise ValueError(f"{name} must be int32 with {n_groups} entries")
    lib = _lib.load()
    ws_bytes = int(lib.exl3_gemv_workspace_bytes(rows, in_tiles, n_groups))
    ws = workspace(xh.device, ws_bytes)
    y = torch.empty((rows, n_groups * 128), dtype=torch.float32, device=xh.device)
    rc = lib.exl3_gemv(
        _ptr(xh), rows, n_sub, _ptr(trellis), in_tiles, out_tiles, int(k), int(cb),
        _ptr(group_sub), _ptr(group_tile), int(n_groups), _ptr(y), _ptr(ws), ws.numel(), _stream(),
    )
    _lib.check(rc, "exl3_gemv")
    return y


def gemv_plan(rows: int, in_tiles: int, n_groups: int) -> tuple[int, int]:
    """(n_splits, tile rows per split) the small-batch kernel uses for a shape."""
    a, b = ctypes.c_int(0), ctypes.c_int(0)
    rc = _lib.load().exl3_gemv_plan(int(rows), int(in_tiles), int(n_groups), ctypes.byref(a),
                                    ctypes.byref(b))
    _lib.check(rc, "exl3_gemv_plan")
    return a.value, b.value


def inner_gemv_partials(xh, trellis, k: int, cb: int, group_sub=None, out=None):
    """Decode-GEMV kernel alone: (n_splits, rows, out) fp32 partial sums
    (``_run_inner_gem`` before its final sum, gemv_metal.py:1431-1457)."""
    in_tiles, out_tiles = _trellis_dims(trellis, k)
    _half(xh, "xh")
    if xh.dim() != 3 or xh.shape[2] != in_tiles * 16:
        raise ValueError("xh must be (rows, n_sub, in)")
    rows, n_sub, _ = xh.shape
    if (in_tiles * 16) % 128 or out_tiles % 8:
        raise ValueError("in/out features must be multiples of 128")
    if not 1 <= rows <= gemv_max_rows():
        raise ValueError(f"rows must be in [1, {gemv_max_rows()}], got {rows}")
    n_groups = out_tiles // 8
    n_splits, _ = gemv_plan(rows, in_tiles, n_groups)
    if out is None:
        out = torch.empty((n_splits, rows, out_tiles * 16), dtype=torch.float32, device=xh.device)
    elif out.dtype != torch.float32 or out.numel() < n_splits * rows * out_tiles * 16:
        raise ValueError("out must be fp32 with n_splits*rows*out elements")
    rc = _lib.load().exl3_gemv_partials(
        _ptr(xh), rows, n_sub, _ptr(trellis), in_tiles, out_tiles, int(k), int(cb),
        _ptr(group_sub), None, n_groups, _ptr(out), out.numel() * 4, _stream(),
    )
    _lib.check(rc, "exl3_gemv_partials")
    return out


def inner_gemv(xh, trellis, k: int, cb: int):
    """(in,) fp16 -> (out,) fp32 (``inner_gemv_mlx``, gemv_metal.py:1495-1505)."""
    if xh.dim() != 1:
        raise ValueError("inner_gemv expects a 1D activation vector")
    return inner_gem_fused(xh.reshape(1, 1, -1), trellis, k, cb).reshape(-1)


def inner_gemm(xh, trellis, k: int, cb: int, tn_offset: int = 0, tn_count: int | None = None):
    """(M, in) fp16 -> (M, out) : fp32 from the small-batch kernel for
    M <= gemv_max_rows(), fp16 (the oracle's cast of the fp32 accumulator) from
    the MFMA prefill kernel above that (``inner_gemm_mlx``,
    gemv_metal.py:1508-1515; exl3_linear.py:137-161)."""
    in_tiles, out_tiles = _trellis_dims(trellis, k)
    _half(xh, "xh")
    if xh.dim() != 2:
        raise ValueError("inner_gemm expects (M, in)")
    rows, n_in = xh.shape
    if n_in != in_tiles * 16:
        raise ValueError(f"xh features {n_in} != trellis in_features {in_tiles * 16}")
    if tn_count is None:
        tn_count = out_tiles - tn_offset
    if rows <= gemv_max_rows() and tn_offset == 0 and tn_count == out_tiles:
        return inner_gem_fused(xh.reshape(rows, 1, n_in), trellis, k, cb)
    if n_in % 64 or tn_count % 8 or tn_offset < 0 or tn_offset + tn_count > out_tiles:
        raise ValueError("prefill GEMM needs in % 64 == 0 and a 128-column aligned slice")
    y = torch.empty((rows, tn_count * 16), dtype=torch.float16, device=xh.device)
    gemm_into(xh.data_ptr(), rows, n_in, trellis, k, cb, tn_offset, tn_count, y.data_ptr(),
              tn_count * 16, xh.device)
    return y


def gemm_into(xh_ptr: int, rows: int, ldx: int, trellis, k: int, cb: int, tn_offset: int,
              tn_count: int, y_ptr: int, ldy: int, device) -> None:
    """``exl3_gemm`` on raw device addresses (strided activations / output slices),
    with the split-tile scratch taken from the per-device GEMM workspace."""
    lib = _lib.load()
    in_tiles, out_tiles = _trellis_dims(trellis, k)
    nbytes = lib.exl3_gemm_workspace_bytes(int(rows), in_tiles, int(tn_count))
    ws = gemm_workspace(device, nbytes)
    rc = lib.exl3_gemm(
        ctypes.c_void_p(xh_ptr), int(rows), int(ldx), _ptr(trellis), in_tiles, out_tiles, int(k),
        int(cb), int(tn_offset), int(tn_count), ctypes.c_void_p(y_ptr), int(ldy),
        _ptr(ws) if ws is not None else None, int(nbytes), _stream(),
    )
    _lib.check(rc, "exl3_gemm")


def had128_rows(x2d: torch.Tensor, scale: torch.Tensor, post: bool, *, rows: int | None = None,
                in_index=None, scale_index=None, out_index=None) -> torch.Tensor:
    """Hadamard-128 with one scale vector per row: ``fp16(had(x * s))`` (``post``
    False, ``_rows_prep``) or ``fp16(had(x) * s)`` (``post`` True, ``_rows_finish``;
    ponyexl3/mlx/exl3_moe.py:105-136). Output row r is computed from input row
    ``in_index[r]`` and scale row ``scale_index[r]`` and stored at ``out_index[r]``
    (int32 device tensors; None = identity). ``scale`` is a 2D view whose rows may
    be strided (e.g. ``gu_suh[:, 0]``)."""
    _half(x2d, "x")
    if not isinstance(scale, torch.Tensor) or not scale.is_cuda or scale.dtype != torch.float16:
        raise ValueError("scale must be an fp16 tensor on the GPU")
    if x2d.dim() != 2 or scale.dim() != 2 or scale.shape[1] != x2d.shape[1] or scale.stride(1) != 1:
        raise ValueError("x and scale must be (rows, n) with unit inner stride")
    n = x2d.shape[1]
    if rows is None:
        rows = x2d.shape[0] if in_index is None else in_index.numel()
    for name, t in (("in_index", in_index), ("scale_index", scale_index), ("out_index", out_index)):
        if t is not None:
            _check_cuda(t, name)
            if t.dtype != torch.int32 or t.numel() != rows:
                raise ValueError(f"{name} must be int32 with one entry per row")
    if n % 128:
        raise ValueError(f"feature dim {n} not divisible by 128")
    out = torch.empty((rows, n), dtype=torch.float16, device=x2d.device)
    rc = _lib.load().exl3_had128_rows(
        _ptr(x2d), x2d.shape[0], rows, n, _ptr(in_index), _ptr(scale), scale.shape[0],
        _ptr(scale_index), scale.stride(0), int(bool(post)), _ptr(out), rows, _ptr(out_index),
        _stream())
    _lib.check(rc, "exl3_had128_rows")
    return out


def segment_table(sorted_groups: torch.Tensor, n_groups: int, block_rows: int) -> torch.Tensor:
    """Row-block table for ``gemm_grouped``: rows are sorted by group id; every block
    of at most ``block_rows`` rows lies inside one group. Built with device-side
    torch ops only (no host sync), sized for the worst case ``N // block_rows +
    n_groups`` with unused entries marked empty, like the reference's table
    (ponyexl3/mlx/exl3_moe.py:79-98). Returns int32 (n_blocks, 4) = {group, first
    row, end row, 0}."""
    n = sorted_groups.numel()
    dev = sorted_groups.device
    nb_max = n // block_rows + n_groups
    cnt = torch.bincount(sorted_groups, minlength=n_groups)[:n_groups]
    seg_end = torch.cumsum(cnt, 0)
    seg_start = seg_end - cnt
    nblk = (cnt + block_rows - 1) // block_rows
    blk_end = torch.cumsum(nblk, 0)
    blk_start = blk_end - nblk
    b = torch.arange(nb_max, device=dev)
    e = torch.searchsorted(blk_end, b, right=True).clamp_(max=n_groups - 1)
    row0 = seg_start[e] + (b - blk_start[e]) * block_rows
    end = seg_end[e]
    row0 = torch.where(b < blk_end[-1], row0, end)
    return torch.stack([e, row0, end, torch.zeros_like(e)], dim=1).to(torch.int32).contiguous()


MOE_SORT_MAX_EXPERTS = 1024


def moe_sort(indices: torch.Tensor, n_experts: int, block_rows: int):
    """Stable sort of the (token, slot) pairs of ``indices`` (T, top_k) int32 by
    expert, with the row-block table of :func:`gemm_grouped`, in one launch
    (``exl3_moe_sort``; the argsort + ``_seg_table`` of ponyexl3/mlx/exl3_moe.py:
    79-98, 700-716). Returns int32 tensors (order, tok, sidx, table (n_blocks, 4))."""
    _check_cuda(indices, "indices")
    if indices.dtype != torch.int32 or indices.dim() != 2 or not indices.is_contiguous():
        raise ValueError("indices must be a contiguous int32 (tokens, top_k) tensor")
    if n_experts > MOE_SORT_MAX_EXPERTS:
        raise ValueError(f"moe_sort handles at most {MOE_SORT_MAX_EXPERTS} experts")
    tokens, top_k = indices.shape
    n = tokens * top_k
    dev = indices.device
    out = torch.empty((3, n), dtype=torch.int32, device=dev)
    table = torch.empty((n // block_rows + n_experts, 4), dtype=torch.int32, device=dev)
    rc = _lib.load().exl3_moe_sort(_ptr(indices), n, top_k, int(n_experts), int(block_rows),
                                   _ptr(out[0]), _ptr(out[1]), _ptr(out[2]), _ptr(table),
                                   table.shape[0], _stream())
    _lib.check(rc, "exl3_moe_sort")
    return out[0], out[1], out[2], table


def moe_glu_rows(g, u, sidx, gu_svh, dn_suh, activation: int = 0):
    """Per sorted row: finish gate and up (output Hadamard, per-expert svh), GLU,
    rotate for the down projection (``exl3_moe_glu_rows``). g, u: (N, H) fp16."""
    _half(g, "g")
    _half(u, "u")
    _half(gu_svh, "gu_svh")
    _half(dn_suh, "dn_suh")
    _check_cuda(sidx, "sidx")
    n, h = g.shape
    n_experts = dn_suh.shape[0]
    if (u.shape != g.shape or not g.is_contiguous() or not u.is_contiguous() or h % 128
            or sidx.dtype != torch.int32 or sidx.numel() != n
            or tuple(gu_svh.shape) != (n_experts, 2 * h) or tuple(dn_suh.shape) != (n_experts, h)
            or not gu_svh.is_contiguous() or not dn_suh.is_contiguous()):
        raise ValueError("moe_glu_rows: inconsistent shapes")
    out = torch.empty_like(g)
    rc = _lib.load().exl3_moe_glu_rows(_ptr(g), _ptr(u), n, h, _ptr(sidx), _ptr(gu_svh), _ptr(dn_suh),
                                       n_experts, int(activation), _ptr(out), _stream())
    _lib.check(rc, "exl3_moe_glu_rows")
    return out


def gemm_grouped(xh, trellis, k: int, cb: int, tn_base: int, group_tiles: int, n_groups: int,
                 table: torch.Tensor, block_rows: int):
    """Segmented prefill GEMM: rows of ``xh`` (N, in) are sorted into groups, group g
    multiplies tile columns ``tn_base + g*group_tiles ..`` (``inner_mm_seg_mlx``,
    ponyexl3/mlx/gemv_metal.py:1685-1741). Returns (N, 16*group_tiles) fp16."""
    in_tiles, out_tiles = _trellis_dims(trellis, k)
    _half(xh, "xh")
    if xh.dim() != 2 or xh.shape[1] != in_tiles * 16:
        raise ValueError(f"xh must be (rows, {in_tiles * 16})")
    if table.dtype != torch.int32 or table.dim() != 2 or table.shape[1] != 4:
        raise ValueError("table must be int32 (n_blocks, 4)")
    n = xh.shape[0]
    y = torch.empty((n, group_tiles * 16), dtype=torch.float16, device=xh.device)
    if n == 0:
        return y
    rc = _lib.load().exl3_gemm_grouped(
        _ptr(xh), n, in_tiles * 16, _ptr(trellis), in_tiles, out_tiles, int(k), int(cb), int(tn_base),
        int(group_tiles), int(n_groups), _ptr(table), table.shape[0], int(block_rows), _ptr(y),
        group_tiles * 16, _stream(),
    )
    _lib.check(rc, "exl3_gemm_grouped")
    return y


def linear_forward(x2d, trellis, k, cb, suh=None, svh=None, bias=None, group_sub=None,
                   fused: bool = True, member_out=None, block_sub=None):
    """Whole-layer forward on (rows, in) fp16 (``exl3_linear_forward``).
    ``fused=False`` selects the three-launch chain for small batches.
    ``member_out`` (out_features of each sibling, in order) is needed for a
    sibling-fused group above ``linear_small_max_rows()`` rows: the prefill GEMM runs once
    per member over its tile columns, each on its own rotated activations
    (``FusedEXL3Group.forward_all``, ponyexl3/mlx/exl3_fused.py:136-202), or once
    over all members when each has ``out_features % 256 == 0`` (``block_sub``: the
    member index of every 256-column block, derived from ``group_sub`` if absent)."""
    in_tiles, out_tiles = _trellis_dims(trellis, k)
    _half(x2d, "x")
    if x2d.dim() != 2 or x2d.shape[1] != in_tiles * 16:
        raise ValueError(f"x must be (rows, {in_tiles * 16})")
    rows = x2d.shape[0]
    n_in, n_out = in_tiles * 16, out_tiles * 16
    if n_in % 128 or n_out % 128:
        raise ValueError("in/out features must be multiples of 128 for the Hadamard transform")
    n_sub = 1
    if suh is not None:
        _half(suh, "suh")
        n_sub = suh.shape[0] if suh.dim() == 2 else 1
        if suh.shape[-1] != n_in:
            raise ValueError("suh length does not match in_features")
    for name, v in (("svh", svh), ("bias", bias)):
        if v is not None:
            _half(v, name)
            if v.numel() != n_out:
                raise ValueError(f"{name} length does not match out_features")
    if group_sub is not None:
        _check_cuda(group_sub, "group_sub")
        if group_sub.dtype != torch.int32 or group_sub.numel() != n_out // 128:
            raise ValueError("group_sub must be int32 with out_features/128 entries")
    elif n_sub > 1:
        raise ValueError("group_sub is required with stacked suh")
    y = torch.empty((rows, n_out), dtype=torch.float16, device=x2d.device)
    if rows == 0:
        return y
    if n_sub > 1 and rows > (linear_small_max_rows() if fused else gemv_max_rows()):
        if member_out is None or len(member_out) != n_sub or sum(member_out) != n_out:
            raise ValueError("member_out must list the out_features of the stacked members")
        xh = had128_pre(x2d, suh)  # (rows, n_sub, in)
        if all(n % 256 == 0 for n in member_out):
            # members end on 256-column blocks: one GEMM launch over all of them, each
            # block reading its member's rotation, then the output transform
            if block_sub is None:
                block_sub = group_sub[::2].contiguous()
            lib = _lib.load()
            ws_bytes = int(lib.exl3_linear_prefill_workspace_bytes(rows, n_in, n_out))
            ws = workspace(x2d.device, ws_bytes)
            rc = lib.exl3_linear_prefill(
                _ptr(xh), rows, n_sub, _ptr(trellis), in_tiles, out_tiles, int(k), int(cb),
                _ptr(block_sub), _ptr(svh), _ptr(bias), _ptr(y), _ptr(ws), ws.numel(), _stream())
            _lib.check(rc, "exl3_linear_prefill")
            return y
        tn0 = 0
        for i, n in enumerate(member_out):
            if n % 128:
                raise ValueError("member out_features must be multiples of 128")
            gemm_into(xh.data_ptr() + 2 * i * n_in, rows, n_sub * n_in, trellis, k, cb, tn0, n // 16,
                      y.data_ptr() + 2 * 16 * tn0, n_out, x2d.device)
            tn0 += n // 16
        return had128_post(y, svh, bias)
    lib = _lib.load()
    ws_bytes = int(lib.exl3_linear_workspace_bytes(rows, n_in, n_out, n_sub))
    ws = workspace(x2d.device, ws_bytes)
    # one-launch kernel: a 64-bit accumulator per (row, output column) = two ints each;
    # medium-batch kernel: one counter per 128-column group
    n_cnt = 2 * rows * n_out if rows <= gemv_max_rows() else n_out // 128
    cnt = sync_counters(x2d.device, n_cnt) if fused else None
    rc = lib.exl3_linear_forward(
        _ptr(x2d), rows, _ptr(trellis), in_tiles, out_tiles, int(k), int(cb), _ptr(suh), n_sub,
        _ptr(group_sub), _ptr(svh), _ptr(bias), _ptr(y), _ptr(ws), ws.numel(), _ptr(cnt),
        0 if cnt is None else cnt.numel(), _stream(),
    )
    _lib.check(rc, "exl3_linear_forward")
    return y


def moe_forward(x2d, indices, gu_trellis, gu_suh, gu_svh, dn_trellis, dn_suh, dn_svh, k, cb,
                activation: int = 0, fused: bool = True, accumulators: bool = True):
    """(T, D) fp16, (T, top_k) int32 -> (T, top_k, D) fp16 (``exl3_moe_forward``).
    ``fused`` selects the two-launch chain (needs the per-stream counters);
    otherwise the five-launch chain runs. ``accumulators`` hands the library enough
    counter memory for the gate/up reduction through 64-bit accumulators (it then
    chooses per call); without, the reduction goes through partial rows."""
    _half(x2d, "x")
    _check_cuda(indices, "indices")
    if indices.dtype != torch.int32 or indices.dim() != 2:
        raise ValueError("indices must be int32 (tokens, top_k)")
    T, D = x2d.shape
    top_k = indices.shape[1]
    E = gu_suh.shape[0]
    H = dn_suh.shape[1]
    y = torch.empty((T, top_k, D), dtype=torch.float16, device=x2d.device)
    lib = _lib.load()
    ws_bytes = int(lib.exl3_moe_workspace_bytes(T, top_k, D, H))
    if ws_bytes == 0:
        raise ValueError("MoE dims must be positive multiples of 128")
    ws = workspace(x2d.device, ws_bytes)
    n_cnt = T * top_k * ((4 * H if accumulators else H // 128) + D // 128)
    cnt = sync_counters(x2d.device, n_cnt) if fused else None
    rc = lib.exl3_moe_forward(
        _ptr(x2d), T, _ptr(indices), top_k, _ptr(gu_trellis), _ptr(gu_suh), _ptr(gu_svh),
        _ptr(dn_trellis), _ptr(dn_suh), _ptr(dn_svh), E, D, H, int(k), int(cb), int(activation),
        _ptr(y), _ptr(ws), ws.numel(), _ptr(cnt) if cnt is not None else None,
        # the length asked for (it selects the reduction), not the buffer's, plus the two
        # ints that make the last one the status word
        n_cnt + 2 if cnt is not None else 0, _stream(),
    )
    _lib.check(rc, "exl3_moe_forward")
    return y
