"""libexl3_hip.so loads without a GPU and exports exactly what include/exl3_hip.h
declares; argument errors are reported as status codes before any launch."""
import ctypes
import os
import re

import pytest

from conftest import ROOT


def _declared(header="exl3_hip.h"):
    text = open(os.path.join(ROOT, "include", header)).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(exl3_[a-z0-9_]+)\s*\(", text)))


@pytest.fixture(scope="module")
def lib():
    from ponyexl3_amd import _lib

    assert os.path.exists(_lib.LIB_PATH), "build libexl3_hip.so first: python -m ponyexl3_amd.build"
    return _lib.load()


def test_every_declared_symbol_is_exported(lib):
    names = _declared()
    assert len(names) >= 12
    for n in names:
        assert hasattr(lib, n), f"{n} declared in include/exl3_hip.h but not exported"


def test_binding_table_matches_header(lib):
    from ponyexl3_amd import _lib

    assert sorted(_lib.PROTOTYPES) == _declared()


def test_diag_library_matches_its_header():
    """The measurement probes live in a library of their own (include/exl3_diag.h) and
    the product library exports none of them."""
    from ponyexl3_amd import _lib

    diag = _lib.load_diag()
    names = _declared("exl3_diag.h")
    assert names == sorted(_lib.DIAG_PROTOTYPES) and len(names) == 4
    for n in names:
        assert hasattr(diag, n)
        assert not hasattr(_lib.load(), n), f"{n} must not be exported by libexl3_hip.so"


def test_version_and_status_strings(lib):
    from ponyexl3_amd import _lib

    assert lib.exl3_version() >= 100
    assert _lib.status_string(0) == "ok"
    for code in range(-10, 0):
        assert _lib.status_string(code) not in ("", "unknown status")
    assert lib.exl3_gemv_max_rows() == 8


def test_argument_errors_before_launch(lib):
    from ponyexl3_amd import _lib

    p = ctypes.c_void_p(0x1000)  # never dereferenced: the checks below fail first
    assert lib.exl3_decode_full(p, 1, 1, 9, 0, 0, 1, p, None) == _lib.EXL3_E_BAD_K
    assert lib.exl3_decode_full(p, 1, 1, 4, 3, 0, 1, p, None) == _lib.EXL3_E_BAD_CODEBOOK
    assert lib.exl3_decode_full(None, 1, 1, 4, 0, 0, 1, p, None) == _lib.EXL3_E_NULL_POINTER
    assert lib.exl3_decode_full(p, 1, 1, 4, 0, 1, 1, p, None) == _lib.EXL3_E_BAD_SHAPE
    assert lib.exl3_quantize_tiles(p, 1, 1, 0, p, p, p, 1 << 30, None) == _lib.EXL3_E_BAD_K
    assert lib.exl3_quantize_tiles(p, 1, 4, 7, p, p, p, 1 << 30, None) == _lib.EXL3_E_BAD_CODEBOOK
    assert lib.exl3_quantize_tiles(p, 1, 4, 0, p, p, None, 0, None) == _lib.EXL3_E_NULL_POINTER
    assert lib.exl3_quantize_tiles(p, 1, 4, 0, p, p, p, 100, None) == _lib.EXL3_E_WORKSPACE
    assert lib.exl3_quantize_tiles(p, 0, 4, 0, p, p, p, 0, None) == _lib.EXL3_OK  # empty: no launch
    assert lib.exl3_quantize_slot_bytes(4) == 256 * 4096 * 2 and lib.exl3_quantize_slot_bytes(1) == 0
    assert lib.exl3_pack_trellis(p, 1, 0, p, None) == _lib.EXL3_E_BAD_K
    assert lib.exl3_pack_trellis(p, 1, 4, None, None) == _lib.EXL3_E_NULL_POINTER
    assert lib.exl3_pack_trellis(p, 0, 4, p, None) == _lib.EXL3_OK
    assert lib.exl3_unpack_trellis(p, 1, 9, p, None) == _lib.EXL3_E_BAD_K
    assert lib.exl3_unpack_trellis(None, 1, 4, p, None) == _lib.EXL3_E_NULL_POINTER
    assert lib.exl3_unpack_trellis(p, 0, 4, p, None) == _lib.EXL3_OK
    assert lib.exl3_linear_prefill(p, 4, 2, p, 8, 16, 4, 0, None, p, None, p, p, 1 << 30, None) == _lib.EXL3_E_BAD_INDEX
    assert lib.exl3_linear_prefill(p, 4, 1, p, 8, 16, 4, 0, None, p, None, p, p, 16, None) == _lib.EXL3_E_WORKSPACE
    assert lib.exl3_linear_prefill(p, 4, 1, p, 7, 16, 4, 0, None, p, None, p, p, 1 << 30, None) == _lib.EXL3_E_BAD_SHAPE
    assert lib.exl3_linear_prefill_workspace_bytes(4, 128, 256) >= 4 * 256 * 2
    assert lib.exl3_moe_sort(p, 8, 2, 4, 64, p, p, p, p, 3, None) == _lib.EXL3_E_BAD_SHAPE  # table too short
    assert lib.exl3_moe_sort(p, 8, 2, 2000, 64, p, p, p, p, 4000, None) == _lib.EXL3_E_UNSUPPORTED
    assert lib.exl3_moe_sort(p, 8, 2, 4, 64, p, p, None, p, 8, None) == _lib.EXL3_E_NULL_POINTER
    assert lib.exl3_moe_glu_rows(p, p, 4, 100, p, p, p, 2, 0, p, None) == _lib.EXL3_E_BAD_SHAPE
    assert lib.exl3_moe_glu_rows(p, p, 4, 128, p, p, p, 2, 5, p, None) == _lib.EXL3_E_UNSUPPORTED
    assert lib.exl3_moe_glu_rows(p, p, 0, 128, p, p, p, 2, 0, p, None) == _lib.EXL3_OK
    assert lib.exl3_decode_full_eg(p, 1, 6, 4, 0, 4, p, None) == _lib.EXL3_E_BAD_SHAPE
    assert lib.exl3_decode_full_eg(p, 1, 6, 4, 0, 0, p, None) == _lib.EXL3_E_BAD_SHAPE
    assert lib.exl3_decode_full_eg(p, 1, 6, 0, 0, 3, p, None) == _lib.EXL3_E_BAD_K
    assert lib.exl3_decode_full_t(p, 1, 1, 4, 0, 1, 1, p, None) == _lib.EXL3_E_BAD_SHAPE
    assert lib.exl3_decode_full_t(p, 1, 1, 4, 0, 0, 1, None, None) == _lib.EXL3_E_NULL_POINTER
    assert lib.exl3_decode_full_t(p, 0, 1, 4, 0, 0, 1, p, None) == _lib.EXL3_OK  # empty: no launch
    assert lib.exl3_had128_pre(p, 1, 100, None, 1, p, None) == _lib.EXL3_E_BAD_SHAPE
    assert lib.exl3_had128_post(p, 0, 2, 0, 1, 128, None, None, p, None) == _lib.EXL3_E_BAD_SHAPE
    assert lib.exl3_gemv(p, 9, 1, p, 8, 8, 4, 0, None, None, 1, p, p, 1 << 20, None) == _lib.EXL3_E_BAD_SHAPE
    assert lib.exl3_gemv(p, 1, 2, p, 8, 8, 4, 0, None, None, 1, p, p, 1 << 20, None) == _lib.EXL3_E_BAD_INDEX
    assert lib.exl3_gemm(p, 32, 100, p, 8, 8, 4, 0, 0, 8, p, 128, None, 0, None) == _lib.EXL3_E_BAD_SHAPE
    assert lib.exl3_linear_forward(p, 1, p, 8, 8, 4, 0, None, 1, None, None, None, p, p, 16, None, 0, None) == _lib.EXL3_E_WORKSPACE
    assert lib.exl3_linear_forward(p, 1, p, 7, 8, 4, 0, None, 1, None, None, None, p, p, 1 << 20, None, 0, None) == _lib.EXL3_E_BAD_SHAPE
    assert lib.exl3_linear_forward(p, 1, p, 8, 16, 4, 0, None, 1, None, None, None, p, p, 1 << 20, p, 1, None) == _lib.EXL3_E_WORKSPACE
    assert lib.exl3_moe_forward(p, 1, p, 8, p, p, p, p, p, p, 4, 256, 100, 4, 0, 0, p, p, 1 << 20, None, 0, None) == _lib.EXL3_E_BAD_SHAPE
    assert lib.exl3_moe_forward(p, 1, p, 8, p, p, p, p, p, p, 4, 256, 128, 4, 0, 7, p, p, 1 << 20, None, 0, None) == _lib.EXL3_E_UNSUPPORTED


def test_workspace_sizes(lib):
    assert lib.exl3_gemv_workspace_bytes(1, 256, 32) >= 4096 * 4
    assert lib.exl3_gemv_workspace_bytes(0, 256, 32) == 0
    assert lib.exl3_linear_workspace_bytes(1, 4096, 4096, 1) > 4096 * 2
    assert lib.exl3_linear_workspace_bytes(2048, 5120, 8192, 1) >= 2048 * (5120 + 8192) * 2
    assert lib.exl3_moe_workspace_bytes(1, 8, 2048, 512) > 0
    assert lib.exl3_moe_workspace_bytes(1, 8, 2048, 500) == 0


def test_gemm_split_plan_sizes(lib, monkeypatch):
    """The prefill GEMM's split plan (host arithmetic only): the workspace it asks for
    is whole fp32 partial tiles, at most one per run plus one per split tile, for any
    shape and any number of workgroup slots; nothing is asked for when the tiles fill
    whole rounds of the slots."""
    def tiles_of(rows, tn):
        mi = 2 if rows <= 64 else 4 if rows <= 128 else 8
        bm = 32 * mi
        return (rows + bm - 1) // bm * ((tn + 15) // 16), bm * 256 * 4

    for slots in (1, 3, 7, 64, 256, 304):
        monkeypatch.setenv("EXL3_GEMM_SLOTS", str(slots))
        for rows in (17, 64, 100, 128, 300, 2048, 5000):
            for in_tiles in (4, 8, 64, 320, 1088, 4096):
                for tn in (8, 24, 64, 320, 2176):
                    nbytes = int(lib.exl3_gemm_workspace_bytes(rows, in_tiles, tn))
                    tiles, tile_bytes = tiles_of(rows, tn)
                    rem = tiles % slots
                    assert nbytes % tile_bytes == 0
                    # runs <= max(slots, 16 * rem) (one per slot, or up to 16 per tile), + rem
                    assert nbytes // tile_bytes <= max(slots, 16 * rem) + rem
                    if rem == 0:
                        assert nbytes == 0
    monkeypatch.setenv("EXL3_GEMM_SLOTS", "256")
    # config 3: o_proj / down_proj (160 tiles: one run per CU, 415 / 416 slots reserved),
    # gate+up (64 tiles in four runs each)
    assert int(lib.exl3_gemm_workspace_bytes(2048, 512, 320)) == (256 + 160) * 256 * 256 * 4
    assert int(lib.exl3_gemm_workspace_bytes(2048, 320, 2176)) == (256 + 64) * 256 * 256 * 4


def test_status_to_exception():
    from ponyexl3_amd import _lib

    _lib.check(0, "x")
    with pytest.raises(ValueError):
        _lib.check(_lib.EXL3_E_BAD_SHAPE, "x")
    with pytest.raises(RuntimeError):
        _lib.check(_lib.EXL3_E_LAUNCH, "x")


def test_header_is_plain_c_and_cxx():
    """include/exl3_hip.h is the boundary: it has to compile on its own as C99 and as
    C++ (no HIP or torch types in any signature)."""
    import shutil
    import subprocess

    header = os.path.join(ROOT, "include", "exl3_hip.h")
    if shutil.which("gcc") is None:
        pytest.skip("gcc not available")
    subprocess.run(["gcc", "-std=c99", "-Wall", "-Werror", "-fsyntax-only", "-x", "c", header], check=True)
    subprocess.run(["g++", "-std=c++17", "-Wall", "-Werror", "-fsyntax-only", "-x", "c++", header], check=True)
