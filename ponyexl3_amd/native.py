"""Folded fp16 engine: the public weight of an EXL3 layer as a plain
``torch.nn.Linear`` (``fold16``).

The EXL3 forward is linear in x, so both Hadamard transforms and both sign/scale
vectors fold into ``W_pub = diag(suh) . H . W_inner . H . diag(svh)``. As in the
reference (``ponyexl3/mlx/native.py:49-85``) W_pub is obtained by pushing an fp16
identity through the same prefill forward the exact engine uses (input Hadamard
kernel, MFMA trellis GEMM, output Hadamard kernel), one stripe of output columns
at a time, so the folded weight carries exactly the runtime's cast points.

Only the fold itself is provided: it is the fp16 materialisation of the decode path.
The reference's lossy engines around it (w8a16 / w4a16 re-quantization with MLX's
affine group quantizer, the fused SwiGLU module and the per-layer error report,
``native.py:88-264``) are alternative engines, not part of the EXL3 path.
"""

from __future__ import annotations

import torch

from . import ops
from .layer import EXL3Layer
from .linear import layer_runtime

# One stripe of output columns at a time (multiple of 128), native.py:45.
PUBLIC_CHUNK_COLS = 8192


def public_weight_chunks(layer: EXL3Layer, *, chunk_cols: int = PUBLIC_CHUNK_COLS, device="cuda"):
    """Yield ``W_pub[:, n0:n1]`` fp16 chunks with all transforms folded in
    (``public_weight_chunks``, ponyexl3/mlx/native.py:49-70)."""
    if chunk_cols % 128 != 0:
        raise ValueError("chunk_cols must be a multiple of 128")
    rt = layer_runtime(layer, device)
    n_in, n_out = layer.in_features, layer.out_features
    eye = torch.eye(n_in, dtype=torch.float16, device=rt.trellis.device)
    xh = ops.had128_pre(eye, rt.suh)  # rows of the scaled input Hadamard, computed once
    del eye
    for n0 in range(0, n_out, chunk_cols):
        n = min(chunk_cols, n_out - n0)
        y = ops.inner_gemm(xh, rt.trellis, rt.k, rt.cb, n0 // 16, n // 16)
        if y.dtype != torch.float16:  # small-batch kernel (in_features <= 8) returns fp32 sums
            y = y.to(torch.float16)
        svh = None if rt.svh is None else rt.svh[n0:n0 + n].contiguous()
        yield ops.had128_post(y, svh)


def public_weight(layer: EXL3Layer, *, device="cuda") -> torch.Tensor:
    """Full ``(in, out)`` fp16 public weight (``public_weight_mlx``, native.py:73-75)."""
    return torch.cat(list(public_weight_chunks(layer, device=device)), dim=1)


def folded_linear_from_exl3(layer: EXL3Layer, *, device="cuda") -> torch.nn.Linear:
    """Exact fold: ``torch.nn.Linear`` holding the fp16 public weight, no
    requantization (``folded_linear_from_exl3``, native.py:78-85)."""
    lin = torch.nn.Linear(layer.in_features, layer.out_features, bias=layer.bias is not None,
                          device=device, dtype=torch.float16)
    with torch.no_grad():
        lin.weight.copy_(public_weight(layer, device=device).T)
        if layer.bias is not None:
            lin.bias.copy_(torch.from_numpy(layer.bias).to(torch.float16))
    lin.requires_grad_(False)
    return lin
