"""ctypes binding of libexl3_hip.so, the C-ABI library declared in include/exl3_hip.h.

The library is the only compute path of this package: if it has not been built
(``python -m ponyexl3_amd.build``) loading fails with an error instead of
falling back to anything else.
"""

from __future__ import annotations

import ctypes
import os

_PKG_DIR = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_PKG_DIR, "libexl3_hip.so")
DIAG_LIB_PATH = os.path.join(_PKG_DIR, "libexl3_diag.so")

EXL3_OK = 0
EXL3_E_BAD_K = -1
EXL3_E_BAD_CODEBOOK = -2
EXL3_E_BAD_SHAPE = -3
EXL3_E_NULL_POINTER = -4
EXL3_E_WORKSPACE = -5
EXL3_E_LAUNCH = -6
EXL3_E_BAD_INDEX = -7
EXL3_E_UNSUPPORTED = -8
EXL3_E_STATIC_LIMIT = -9
EXL3_E_INCOMPLETE = -10

_vp = ctypes.c_void_p
_i = ctypes.c_int
_sz = ctypes.c_size_t

# name -> (restype, argtypes); mirrors include/exl3_hip.h one to one
PROTOTYPES = {
    "exl3_version": (_i, []),
    "exl3_status_string": (ctypes.c_char_p, [_i]),
    "exl3_gemv_max_rows": (_i, []),
    "exl3_linear_small_max_rows": (_i, []),
    "exl3_decode_full": (_i, [_vp, _i, _i, _i, _i, _i, _i, _vp, _vp]),
    "exl3_linear_prefill_workspace_bytes": (_sz, [_i, _i, _i]),
    "exl3_linear_prefill": (_i, [_vp, _i, _i, _vp, _i, _i, _i, _i, _vp, _vp, _vp, _vp, _vp, _sz, _vp]),
    "exl3_moe_sort": (_i, [_vp, _i, _i, _i, _i, _vp, _vp, _vp, _vp, _i, _vp]),
    "exl3_moe_glu_rows": (_i, [_vp, _vp, _i, _i, _vp, _vp, _vp, _i, _i, _vp, _vp]),
    "exl3_quantize_slot_bytes": (_sz, [_i]),
    "exl3_quantize_workspace_bytes": (_sz, [_i, _i]),
    "exl3_quantize_tiles": (_i, [_vp, _i, _i, _i, _vp, _vp, _vp, _sz, _vp]),
    "exl3_unpack_trellis": (_i, [_vp, ctypes.c_longlong, _i, _vp, _vp]),
    "exl3_pack_trellis": (_i, [_vp, ctypes.c_longlong, _i, _vp, _vp]),
    "exl3_decode_full_eg": (_i, [_vp, _i, _i, _i, _i, _i, _vp, _vp]),
    "exl3_decode_full_t": (_i, [_vp, _i, _i, _i, _i, _i, _i, _vp, _vp]),
    "exl3_had128_pre": (_i, [_vp, _i, _i, _vp, _i, _vp, _vp]),
    "exl3_had128_post": (_i, [_vp, _i, _i, _sz, _i, _i, _vp, _vp, _vp, _vp]),
    "exl3_gemv": (_i, [_vp, _i, _i, _vp, _i, _i, _i, _i, _vp, _vp, _i, _vp, _vp, _sz, _vp]),
    "exl3_gemv_workspace_bytes": (_sz, [_i, _i, _i]),
    "exl3_gemv_plan": (_i, [_i, _i, _i, ctypes.POINTER(_i), ctypes.POINTER(_i)]),
    "exl3_gemv_partials": (_i, [_vp, _i, _i, _vp, _i, _i, _i, _i, _vp, _vp, _i, _vp, _sz, _vp]),
    "exl3_gemm": (_i, [_vp, _i, _sz, _vp, _i, _i, _i, _i, _i, _i, _vp, _sz, _vp, _sz, _vp]),
    "exl3_gemm_workspace_bytes": (_sz, [_i, _i, _i]),
    "exl3_gemm_grouped": (_i, [_vp, _i, _sz, _vp, _i, _i, _i, _i, _i, _i, _i, _vp, _i, _i, _vp, _sz, _vp]),
    "exl3_had128_rows": (_i, [_vp, _i, _i, _i, _vp, _vp, _i, _vp, _sz, _i, _vp, _i, _vp, _vp]),
    "exl3_linear_forward": (
        _i,
        [_vp, _i, _vp, _i, _i, _i, _i, _vp, _i, _vp, _vp, _vp, _vp, _vp, _sz, _vp, _sz, _vp],
    ),
    "exl3_linear_workspace_bytes": (_sz, [_i, _i, _i, _i]),
    "exl3_counters_status": (_i, [_vp, _sz, _vp]),
    "exl3_linear_plan": (_i, [_i, _i, _i, _i] + [ctypes.POINTER(_i)] * 4),
    "exl3_linear_static_scratch_bytes": (_sz, []),
    "exl3_linear_static_need_bytes": (_sz, [_i, _i, _i]),
    "exl3_linear_forward_static": (
        _i, [_vp, _i, _vp, _i, _i, _i, _i, _vp, _i, _vp, _vp, _vp, _vp, _vp],
    ),
    "exl3_moe_forward": (
        _i,
        [_vp, _i, _vp, _i, _vp, _vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _i, _i, _vp, _vp, _sz, _vp,
         _sz, _vp],
    ),
    "exl3_moe_workspace_bytes": (_sz, [_i, _i, _i, _i]),
}

# libexl3_diag.so (include/exl3_diag.h): measurement probes, not part of the product library
DIAG_PROTOTYPES = {
    "exl3_diag_stream_read": (_i, [_vp, _sz, _vp, _vp]),
    "exl3_diag_decode_loop": (_i, [_vp, _sz, _i, _i, _i, _i, _vp, _vp]),
    "exl3_diag_empty_launch": (_i, [_i, _i, _i, _vp]),
    "exl3_diag_first_rows": (_i, [_vp, _sz, _i, _i, _i, _i, ctypes.c_uint, _vp, _vp]),
}

_lib = None
_diag = None


def load() -> ctypes.CDLL:
    """Load libexl3_hip.so (after torch, so both share one HIP runtime)."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise RuntimeError(
                f"{LIB_PATH} is missing: build the HIP kernels first with "
                "`python -m ponyexl3_amd.build` (there is no fallback path)"
            )
        import torch  # noqa: F401  (loads libamdhip64 before our library resolves it)

        lib = ctypes.CDLL(LIB_PATH)
        for name, (restype, argtypes) in PROTOTYPES.items():
            fn = getattr(lib, name)
            fn.restype = restype
            fn.argtypes = argtypes
        _lib = lib
    return _lib


def load_diag() -> ctypes.CDLL:
    """Load libexl3_diag.so, the measurement probes bench.py reports its ceilings from."""
    global _diag
    if _diag is None:
        if not os.path.exists(DIAG_LIB_PATH):
            raise RuntimeError(f"{DIAG_LIB_PATH} is missing: run `python -m ponyexl3_amd.build`")
        import torch  # noqa: F401

        lib = ctypes.CDLL(DIAG_LIB_PATH)
        for name, (restype, argtypes) in DIAG_PROTOTYPES.items():
            fn = getattr(lib, name)
            fn.restype = restype
            fn.argtypes = argtypes
        _diag = lib
    return _diag


def status_string(status: int) -> str:
    return load().exl3_status_string(int(status)).decode()


def check(status: int, what: str) -> None:
    """Raise like the reference's host wrappers do: ValueError for argument
    errors found before launch, RuntimeError if a launch itself failed."""
    if status == EXL3_OK:
        return
    msg = f"{what}: {status_string(status)} (status {status})"
    if status in (EXL3_E_LAUNCH, EXL3_E_INCOMPLETE):
        raise RuntimeError(msg)
    raise ValueError(msg)
