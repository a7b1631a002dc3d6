"""Writes tests/golden/search_exact.npz by running the reference's exact trellis
search (``ponyexl3.convert.reference_search.quantize_tile_reference``, numpy only)
in the build container.

Run once, by hand, where ``/root/reference`` is mounted:

    python tests/golden/make_golden_search.py

What the vectors pin that mathematics alone does not: the closing heuristic of the
search (a free pass, then passes pinned to the previous pass's last state until the
path closes, at most four), its tie-breaking (numpy argmin = first minimum) and its
float64 cost arithmetic. The forward recursion itself is also checked by brute
force in tests/test_oracle_search.py.

  search_exact.npz   per case "k{K}_cb{cb}": tile (256,) fp32 in kernel order,
                     states (256,) uint16, decoded (256,) fp32
"""

from __future__ import annotations

import os
import sys

import numpy as np

REFERENCE_ROOT = os.environ.get("EXL3_REFERENCE_ROOT", "/root/reference")
sys.path.insert(0, REFERENCE_ROOT)

from ponyexl3.convert.reference_search import quantize_tile_reference  # noqa: E402
from ponyexl3.ref.codebook import CodebookMode  # noqa: E402

HERE = os.path.dirname(os.path.abspath(__file__))

# (K, codebook): the pairs of the reference's own quality test
# (tests/test_convert_metal.py:44-53) with its seeds and scale, plus K = 5
CASES = [(2, 1), (3, 1), (4, 0), (4, 1), (4, 2), (5, 1)]


def main() -> None:
    out = {}
    for k, cb in CASES:
        scale = 1.0 if cb == 2 else 1.24371088
        rng = np.random.default_rng(100 + 10 * k + cb)
        tile = (rng.standard_normal((1, 256)) * scale).astype(np.float32)[0]
        states, decoded = quantize_tile_reference(tile, k, CodebookMode(cb))
        tag = f"k{k}_cb{cb}"
        out[tag + "_tile"] = tile
        out[tag + "_states"] = np.asarray(states, dtype=np.uint16)
        out[tag + "_decoded"] = np.asarray(decoded, dtype=np.float32)
        print(tag, "mse", float(np.mean((decoded - tile) ** 2)), flush=True)
    np.savez_compressed(os.path.join(HERE, "search_exact.npz"), **out)


if __name__ == "__main__":
    main()
