"""MI355X-native EXL3 quantized-linear path (trellis decode GEMV/GEMM,
Hadamard-128 regularisation, routed MoE expert GEMV) behind the reference's
module API. All compute is in libexl3_hip.so (``python -m ponyexl3_amd.build``)."""

from .layer import (
    CodebookMode,
    EXL3Layer,
    codebook_mode_from_flags,
    make_exl3_layer,
    unpack_sign_bitfield,
    unpack_signs_or_pass,
)

__all__ = [
    "CodebookMode",
    "EXL3Layer",
    "codebook_mode_from_flags",
    "make_exl3_layer",
    "unpack_sign_bitfield",
    "unpack_signs_or_pass",
    "EXL3Linear",
    "FusedEXL3Group",
    "FusedEXL3Sibling",
    "EXL3SwitchGLU",
    "EXL3MoEBlock",
    "fusable",
    "reconstruct_inner",
    "reconstruct_public_weights",
]


def __getattr__(name):
    # torch-dependent modules load lazily so the host-side pieces import fast
    if name in ("EXL3Linear", "EXL3LayerRuntime", "layer_runtime", "clear_layer_caches"):
        from . import linear

        return getattr(linear, name)
    if name in ("FusedEXL3Group", "FusedEXL3Sibling", "fusable"):
        from . import fused

        return getattr(fused, name)
    if name in ("EXL3SwitchGLU", "EXL3MoEBlock", "route_topk", "combine_experts"):
        from . import moe

        return getattr(moe, name)
    if name in ("reconstruct_inner", "reconstruct_public_weights"):
        from . import ops

        return getattr(ops, name)
    raise AttributeError(name)
