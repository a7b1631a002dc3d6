"""The diagnostic entry points (libexl3_diag.so, include/exl3_diag.h) behind bench.py's measured ceilings: argument
checks, and that a launch over a small buffer runs to completion and writes only
inside the output the header describes."""
import ctypes

import pytest
import torch

pytestmark = pytest.mark.gpu


def _args(cuda):
    from ponyexl3_amd import _lib

    lib = _lib.load_diag()
    buf = torch.randint(-2**31, 2**31 - 1, (1 << 20,), dtype=torch.int32, device=cuda)  # 4 MiB
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    return _lib, lib, buf, stream


def test_stream_read(cuda):
    _lib, lib, buf, stream = _args(cuda)
    out = torch.zeros(4, dtype=torch.int32, device=cuda)
    p = lambda t: ctypes.c_void_p(t.data_ptr())
    print("diag stream read", flush=True)
    assert lib.exl3_diag_stream_read(p(buf), buf.numel() * 4, p(out), stream) == 0
    assert lib.exl3_diag_stream_read(p(buf), 4096 + 48, p(out), stream) == 0  # ragged tail
    torch.cuda.synchronize()
    assert lib.exl3_diag_stream_read(None, 4096, p(out), stream) == _lib.EXL3_E_NULL_POINTER
    assert lib.exl3_diag_stream_read(p(buf), 8, p(out), stream) == _lib.EXL3_E_BAD_SHAPE
    assert lib.exl3_diag_stream_read(ctypes.c_void_p(buf.data_ptr() + 4), 4096, p(out), stream) == _lib.EXL3_E_BAD_SHAPE


@pytest.mark.parametrize("k,cb", [(2, 0), (4, 0), (4, 1), (8, 0)])
def test_decode_loop(cuda, k, cb):
    _lib, lib, buf, stream = _args(cuda)
    n_wg, steps = 8, 8
    out = torch.full((n_wg * 16 * 64 + 64,), 7.0, dtype=torch.float32, device=cuda)
    p = lambda t: ctypes.c_void_p(t.data_ptr())
    print(f"diag decode loop k={k} cb={cb}", flush=True)
    rc = lib.exl3_diag_decode_loop(p(buf), buf.numel() * 4, k, cb, n_wg, steps, p(out), stream)
    assert rc == 0
    torch.cuda.synchronize()
    assert torch.isfinite(out[: n_wg * 16 * 64]).all()
    assert (out[n_wg * 16 * 64:] == 7.0).all()  # one value per lane of every wave, nothing past them
    bad = lambda **kw: lib.exl3_diag_decode_loop(
        p(buf), kw.get("nbytes", buf.numel() * 4), kw.get("k", k), kw.get("cb", cb), kw.get("n_wg", n_wg),
        kw.get("steps", steps), p(out), stream)
    assert bad(steps=6) == _lib.EXL3_E_BAD_SHAPE
    assert bad(n_wg=0) == _lib.EXL3_E_BAD_SHAPE
    assert bad(nbytes=16) == _lib.EXL3_E_BAD_SHAPE
    assert bad(cb=2) == _lib.EXL3_E_UNSUPPORTED
    assert bad(k=9) != 0


def test_launch_phase_probes(cuda):
    _lib, lib, buf, stream = _args(cuda)
    out = torch.zeros(4, dtype=torch.int32, device=cuda)
    p = lambda t: ctypes.c_void_p(t.data_ptr())
    print("diag launch phases", flush=True)
    assert lib.exl3_diag_empty_launch(40, 16, 256, stream) == 0
    assert lib.exl3_diag_empty_launch(272, 5, 512, stream) == 0
    for k in (2, 4, 5, 8):
        assert lib.exl3_diag_first_rows(p(buf), buf.numel() * 4, k, 40, 16, 256, 12345, p(out), stream) == 0
    torch.cuda.synchronize()
    assert lib.exl3_diag_empty_launch(0, 1, 256, stream) == _lib.EXL3_E_BAD_SHAPE
    assert lib.exl3_diag_empty_launch(4, 1, 100, stream) == _lib.EXL3_E_BAD_SHAPE
    assert lib.exl3_diag_empty_launch(4, 1, 2048, stream) == _lib.EXL3_E_BAD_SHAPE
    assert lib.exl3_diag_first_rows(None, 4096, 4, 4, 1, 256, 0, p(out), stream) == _lib.EXL3_E_NULL_POINTER
    assert lib.exl3_diag_first_rows(p(buf), 100, 4, 4, 1, 256, 0, p(out), stream) == _lib.EXL3_E_BAD_SHAPE
    assert lib.exl3_diag_first_rows(p(buf), buf.numel() * 4, 9, 4, 1, 256, 0, p(out), stream) != 0
