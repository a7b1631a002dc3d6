"""Writes the golden vectors under tests/golden/ by running the reference's CPU
codec (``ponyexl3.ref``) in the build container.

Run once, by hand, where ``/root/reference`` is mounted:

    python tests/golden/make_golden.py

The reference never travels with the repository; only the input/output vectors
written here do. Covered functions (those a self-consistent but wrong pair of
pack/unpack or decode implementations could otherwise slip past):

  codebook_tables.npz   decode_3inst over all 65536 codewords x {DEFAULT, MCG, MUL1}
  perm.npz              tensor_core_perm + its inverse
  tiles.npz             pack_trellis_tile / unpack_trellis_tile, K = 1..8
  decoded_layers.npz    decode_packed_trellis on 32x48 layers, every (K, codebook)
  forwards.npz          linear_forward_reconstruct on 128x256 layers
                        (+ bias, + packed int16 signs, + public weights)
"""

from __future__ import annotations

import os
import sys

import numpy as np

REFERENCE_ROOT = os.environ.get("EXL3_REFERENCE_ROOT", "/root/reference")
sys.path.insert(0, REFERENCE_ROOT)

from ponyexl3.ref.codebook import CodebookMode, decode_3inst  # noqa: E402
from ponyexl3.ref.decode import decode_packed_trellis  # noqa: E402
from ponyexl3.ref.forward import linear_forward_reconstruct  # noqa: E402
from ponyexl3.ref.layer import EXL3Layer  # noqa: E402
from ponyexl3.ref.perm import tensor_core_perm, tensor_core_perm_inverse  # noqa: E402
from ponyexl3.ref.reconstruct import reconstruct_public_weights  # noqa: E402
from ponyexl3.ref.synthetic import make_exl3_layer  # noqa: E402
from ponyexl3.ref.trellis import (  # noqa: E402
    pack_trellis_tile,
    unpack_trellis,
    unpack_trellis_tile,
)

HERE = os.path.dirname(os.path.abspath(__file__))


def save(name, **arrays):
    path = os.path.join(HERE, name)
    np.savez_compressed(path, **arrays)
    print(f"wrote {name}: {os.path.getsize(path)} bytes", flush=True)


def codebook_tables():
    out = {}
    for mode in (CodebookMode.DEFAULT, CodebookMode.MCG, CodebookMode.MUL1):
        tab = np.empty(65536, dtype=np.float16)
        for cw in range(65536):
            tab[cw] = decode_3inst(cw, mode)
        out[f"cb{int(mode)}"] = tab.view(np.uint16)
    save("codebook_tables.npz", **out)


def perm():
    save("perm.npz", perm=tensor_core_perm(), inverse=tensor_core_perm_inverse())


def tiles():
    out = {}
    for k in range(1, 9):
        enc, packed, unpacked = [], [], []
        raw, raw_unpacked = [], []
        for s in range(4):
            rng = np.random.default_rng(100 * k + s)
            e = (rng.integers(0, 2**16, size=256, dtype=np.uint32) & ((1 << k) - 1)).astype(
                np.uint16
            )
            p = pack_trellis_tile(e, k)
            enc.append(e)
            packed.append(p)
            unpacked.append(unpack_trellis_tile(p, k))
            # any uint16 fill is a legal stream: unpack raw random words too
            r = rng.integers(0, 2**16, size=16 * k, dtype=np.uint16)
            raw.append(r)
            raw_unpacked.append(unpack_trellis_tile(r, k))
        out[f"k{k}_encoded"] = np.stack(enc)
        out[f"k{k}_packed"] = np.stack(packed)
        out[f"k{k}_unpacked"] = np.stack(unpacked)
        out[f"k{k}_raw"] = np.stack(raw)
        out[f"k{k}_raw_unpacked"] = np.stack(raw_unpacked)
        # the reference's second, tensor-level statement of the same format
        out[f"k{k}_raw_unpacked_tensor"] = unpack_trellis(np.stack(raw)[None], k)[0]
    save("tiles.npz", **out)


def decoded_layers():
    out = {}
    for k in range(1, 9):
        for cb in (0, 1, 2):
            rng = np.random.default_rng(7000 + 10 * k + cb)
            trellis = rng.integers(0, 2**16, size=(2, 3, 16 * k), dtype=np.uint16)
            w = decode_packed_trellis(trellis, k, CodebookMode(cb))
            out[f"k{k}_cb{cb}_trellis"] = trellis
            out[f"k{k}_cb{cb}_w"] = w.view(np.uint16)
    save("decoded_layers.npz", **out)


def forwards():
    out = {}
    cases = [(k, cb, False, False) for k in (1, 2, 3, 4, 5, 6, 7, 8) for cb in (0, 1)]
    cases += [(4, 2, False, False), (4, 0, True, False), (3, 1, False, True)]
    for k, cb, bias, packed_signs in cases:
        tag = f"k{k}_cb{cb}" + ("_bias" if bias else "") + ("_bf" if packed_signs else "")
        layer = make_exl3_layer(
            k=k, in_features=128, out_features=256, seed=40 + k + 10 * cb,
            mcg=(cb == 1), mul1=(cb == 2), bias=bias,
        )
        rng = np.random.default_rng(900 + k + 10 * cb)
        if packed_signs:
            layer.suh = rng.integers(-(2**15), 2**15, size=128 // 16).astype(np.int16)
            layer.svh = rng.integers(-(2**15), 2**15, size=256 // 16).astype(np.int16)
        x = rng.standard_normal((3, 128)).astype(np.float16)
        y = linear_forward_reconstruct(layer, x)
        out[f"{tag}_trellis"] = layer.trellis
        out[f"{tag}_suh"] = layer.suh if packed_signs else layer.suh.view(np.uint16)
        out[f"{tag}_svh"] = layer.svh if packed_signs else layer.svh.view(np.uint16)
        if bias:
            out[f"{tag}_bias"] = layer.bias.view(np.uint16)
        out[f"{tag}_x"] = x.view(np.uint16)
        out[f"{tag}_y"] = y.view(np.uint16)
        print(tag, float(np.abs(y.astype(np.float32)).max()), flush=True)
    # public-weight fold on one layer (ref/reconstruct.py:26-49)
    layer = make_exl3_layer(k=4, in_features=128, out_features=256, seed=77)
    out["pub_trellis"] = layer.trellis
    out["pub_suh"] = layer.suh.view(np.uint16)
    out["pub_svh"] = layer.svh.view(np.uint16)
    out["pub_w"] = reconstruct_public_weights(layer.trellis, layer.suh, layer.svh, 4).view(
        np.uint16
    )
    save("forwards.npz", **out)


if __name__ == "__main__":
    which = sys.argv[1:] or ["perm", "tiles", "decoded_layers", "codebook_tables", "forwards"]
    for name in which:
        globals()[name]()
