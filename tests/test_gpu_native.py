"""Folded fp16 engine (public weight through the prefill kernels) against the
oracle's public-weight reconstruction and the exact EXL3 module."""
import numpy as np
import pytest
import torch

from conftest import rel_l2

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("k,mcg,mul1,n_in,n_out", [(4, False, False, 256, 384), (3, True, False, 384, 256),
                                                   (6, False, True, 128, 640)])
def test_public_weight_matches_oracle(cuda, oracle, k, mcg, mul1, n_in, n_out):
    """W_pub from identity activations vs diag(suh).H.W.H.diag(svh) in fp32
    (ponyexl3/ref/reconstruct.py:26-49). The prefill path rounds to fp16 after the
    input transform and after the GEMM, hence a tolerance, not equality."""
    from ponyexl3_amd import make_exl3_layer, native

    layer = make_exl3_layer(k=k, in_features=n_in, out_features=n_out, seed=500 + k, mcg=mcg, mul1=mul1)
    cb = int(layer.codebook_mode)
    ref = oracle.reconstruct_public_weights(layer.trellis, layer.suh, layer.svh, k, cb)
    w = native.public_weight(layer, device=cuda)
    assert w.dtype == torch.float16 and tuple(w.shape) == (n_in, n_out)
    assert rel_l2(w.cpu().numpy(), ref) < 1e-3
    # chunked = whole: stripes of 128 columns are independent
    parts = list(native.public_weight_chunks(layer, chunk_cols=128, device=cuda))
    assert len(parts) == n_out // 128
    assert torch.equal(torch.cat(parts, dim=1), w)
    with pytest.raises(ValueError):
        list(native.public_weight_chunks(layer, chunk_cols=100, device=cuda))


def test_public_weight_equals_identity_through_the_module(cuda):
    """The fold is the module applied to the identity. Both round the same fp32 sums to
    fp16; the module's prefill path adds the 128 terms of the output Hadamard on the
    matrix pipe, the fold in butterfly order, so a result that sits on a rounding boundary
    can come out one fp16 step apart."""
    from ponyexl3_amd import EXL3Linear, make_exl3_layer, native

    layer = make_exl3_layer(k=4, in_features=256, out_features=256, seed=9)
    eye = torch.eye(256, dtype=torch.float16, device=cuda)
    fold, module = native.public_weight(layer, device=cuda).float(), EXL3Linear(layer)(eye).float()
    step = torch.maximum(fold.abs(), module.abs()) * 2.0 ** -10 + 2.0 ** -24  # one fp16 step at that size
    assert bool(((fold - module).abs() <= step).all())
    assert float((fold != module).float().mean()) < 0.01


@pytest.mark.parametrize("bias", [False, True])
def test_folded_linear_tracks_exact_layer(cuda, oracle, bias):
    from ponyexl3_amd import make_exl3_layer, native

    layer = make_exl3_layer(k=4, in_features=512, out_features=384, seed=31, mcg=True, bias=bias)
    lin = native.folded_linear_from_exl3(layer, device=cuda)
    assert isinstance(lin, torch.nn.Linear) and lin.weight.dtype == torch.float16
    assert tuple(lin.weight.shape) == (384, 512) and (lin.bias is not None) == bias
    rng = np.random.default_rng(3)
    x = rng.standard_normal((5, 512)).astype(np.float16)
    y = lin(torch.from_numpy(x).to(cuda)).cpu().numpy()
    ref = oracle.linear_forward(layer.trellis, 4, int(layer.codebook_mode), layer.suh, layer.svh, x,
                                bias=layer.bias)
    assert rel_l2(y, ref) < 2e-3
