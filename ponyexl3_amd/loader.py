"""Converted-checkpoint reader: ``quantization_config.json`` + safetensors ->
``EXL3Layer`` objects, expert stacking and the sibling-fusion policy.

Host-side only (numpy + safetensors; torch is touched where modules are built).
Mirrors ``ponyexl3/ref/loader.py:41-173`` (same function names, same errors) and
the module-building helpers of ``ponyexl3/mlx/model.py``: the multiplier check
(:261-283), expert stacking (:77-127) and the fusion policy (:325-432).

On-disk schema per module key (``ponyexl3/convert/discovery.py:191-212``):
``{key}.trellis`` int16 ``(in/16, out/16, 16K)`` (reinterpreted as uint16),
``{key}.suh`` / ``{key}.svh`` fp16 (or legacy ``su`` / ``sv``: packed int16 sign
bitfields), optional ``{key}.bias``, ``{key}.mcg`` / ``{key}.mul1`` int32 scalars
holding the codebook multiplier, and in ``quantization_config.json`` the
``tensor_storage[key]`` record with ``quant_format == "exl3"``,
``stored_tensors``, ``bits_per_weight``, ``mcg_multiplier``, ``mul1_multiplier``.
"""

from __future__ import annotations

import json
import os
from glob import glob
from typing import Any

import numpy as np

from .layer import EXL3Layer

MCG_MULT = 0xCBAC1FED  # ponyexl3/ref/codebook.py:19-20
MUL1_MULT = 0x83DCD12D

_WEIGHT_INDEX_CACHE: dict[str, dict[str, str] | None] = {}


def clear_weight_index_cache(model_dir: str) -> None:
    """Drop the cached safetensors index for a model directory."""
    _WEIGHT_INDEX_CACHE.pop(model_dir, None)


def _weight_index(model_dir: str) -> dict[str, str] | None:
    if model_dir not in _WEIGHT_INDEX_CACHE:
        path = os.path.join(model_dir, "model.safetensors.index.json")
        if os.path.isfile(path):
            with open(path, encoding="utf-8") as f:
                _WEIGHT_INDEX_CACHE[model_dir] = json.load(f).get("weight_map", {})
        else:
            _WEIGHT_INDEX_CACHE[model_dir] = None
    return _WEIGHT_INDEX_CACHE[model_dir]


def list_exl3_layers(model_dir: str) -> list[dict[str, Any]]:
    """EXL3 linear modules named by quantization_config.json, sorted by key."""
    qpath = os.path.join(model_dir, "quantization_config.json")
    if not os.path.isfile(qpath):
        raise FileNotFoundError(f"missing {qpath}")
    with open(qpath, encoding="utf-8") as f:
        qcfg = json.load(f)
    layers = []
    for key, info in qcfg.get("tensor_storage", {}).items():
        if info.get("quant_format") != "exl3":
            continue
        layers.append({
            "key": key,
            "bits_per_weight": info.get("bits_per_weight"),
            "stored_tensors": info.get("stored_tensors", {}),
            "mcg": bool(info.get("mcg_multiplier")),
            "mul1": bool(info.get("mul1_multiplier")),
        })
    return sorted(layers, key=lambda x: x["key"])


def layer_meta_from_config(model_dir: str, module_key: str) -> dict[str, Any]:
    """Layer dimensions and on-disk sizes without loading weight tensors."""
    meta = {x["key"]: x for x in list_exl3_layers(model_dir)}
    if module_key not in meta:
        raise KeyError(f"{module_key!r} not in quantization_config tensor_storage")
    info = meta[module_key]
    stored = info["stored_tensors"]
    trellis_key = f"{module_key}.trellis"
    if trellis_key not in stored:
        raise KeyError(f"missing {trellis_key}")
    shape = stored[trellis_key]["shape"]
    in_tiles, out_tiles, packed_size = int(shape[0]), int(shape[1]), int(shape[2])
    return {
        "key": module_key,
        "k": packed_size * 16 // 256,
        "bits_per_weight": info.get("bits_per_weight"),
        "in_features": in_tiles * 16,
        "out_features": out_tiles * 16,
        "in_tiles": in_tiles,
        "out_tiles": out_tiles,
        "n_tiles": in_tiles * out_tiles,
        "trellis_shape": (in_tiles, out_tiles, packed_size),
        "trellis_bytes": int(stored[trellis_key].get("n_bytes", 0)),
        "weight_fp16_bytes": in_tiles * out_tiles * 512,
        "mcg": info["mcg"],
        "mul1": info["mul1"],
    }


def _find_shard(model_dir: str, tensor_key: str) -> str:
    from safetensors import safe_open

    index = _weight_index(model_dir)
    if index is not None:
        shard = index.get(tensor_key)
        if shard is not None:
            path = os.path.join(model_dir, shard)
            if os.path.isfile(path):
                return path
    for pattern in (os.path.join(model_dir, "*.safetensors"),
                    os.path.join(model_dir, "**", "*.safetensors")):
        for path in sorted(glob(pattern, recursive=True)):
            with safe_open(path, framework="np") as st:
                if tensor_key in st.keys():
                    return path
    raise FileNotFoundError(f"tensor {tensor_key!r} not found under {model_dir}")


def _load_tensor(model_dir: str, tensor_key: str) -> np.ndarray | None:
    from safetensors import safe_open

    try:
        path = _find_shard(model_dir, tensor_key)
    except FileNotFoundError:
        return None
    with safe_open(path, framework="np") as st:
        return np.array(st.get_tensor(tensor_key))


def has_exl3_layer_weights(model_dir: str, module_key: str) -> bool:
    """True when trellis weights exist on disk (vs a plan-only quantization_config)."""
    try:
        _find_shard(model_dir, f"{module_key}.trellis")
    except FileNotFoundError:
        return False
    return True


def check_multiplier(model_dir: str, module_key: str, name: str, expected: int) -> None:
    """The codebooks hard-code the default multipliers; a checkpoint quantized with
    another one must be refused rather than decoded to garbage
    (``_check_multiplier``, ponyexl3/mlx/model.py:261-270). A missing scalar passes."""
    t = _load_tensor(model_dir, f"{module_key}.{name}")
    if t is None:
        return
    got = int(np.asarray(t).astype(np.int64).reshape(-1)[0]) & 0xFFFFFFFF
    if got != int(expected):
        raise ValueError(
            f"{module_key}: stored {name} multiplier {got:#x} != supported {int(expected):#x}")


def load_exl3_layer(model_dir: str, module_key: str) -> EXL3Layer:
    """Load one EXL3 linear layer by module key (e.g. model.layers.0.mlp.gate_proj)."""
    if not has_exl3_layer_weights(model_dir, module_key):
        raise FileNotFoundError(f"{module_key}.trellis")
    cfg = layer_meta_from_config(model_dir, module_key)
    trellis = _load_tensor(model_dir, f"{module_key}.trellis")
    if trellis is None:
        raise FileNotFoundError(f"{module_key}.trellis")
    if trellis.dtype not in (np.uint16, np.int16):
        raise ValueError(f"{module_key}.trellis has dtype {trellis.dtype}, expected int16/uint16")
    if cfg["mcg"]:
        check_multiplier(model_dir, module_key, "mcg", MCG_MULT)
    if cfg["mul1"]:
        check_multiplier(model_dir, module_key, "mul1", MUL1_MULT)
    suh = _load_tensor(model_dir, f"{module_key}.suh")
    if suh is None:
        suh = _load_tensor(model_dir, f"{module_key}.su")
    svh = _load_tensor(model_dir, f"{module_key}.svh")
    if svh is None:
        svh = _load_tensor(model_dir, f"{module_key}.sv")
    bias = _load_tensor(model_dir, f"{module_key}.bias")
    layer = EXL3Layer(
        key=module_key, in_features=cfg["in_features"], out_features=cfg["out_features"],
        k=cfg["k"], trellis=trellis.view(np.uint16), suh=suh, svh=svh, bias=bias,
        mcg=cfg["mcg"], mul1=cfg["mul1"],
    )
    layer.validate()
    return layer


def load_all_exl3_layers(model_dir: str) -> dict[str, EXL3Layer]:
    """Every EXL3 module of the checkpoint whose weights are on disk, by key."""
    return {info["key"]: load_exl3_layer(model_dir, info["key"])
            for info in list_exl3_layers(model_dir)
            if has_exl3_layer_weights(model_dir, info["key"])}


# ---------------------------------------------------------------------------
# module building (torch)

def stack_expert_switch_glu(expert_prefixes: list[str], layers: dict[str, EXL3Layer], *,
                            activation: str = "silu", device="cuda"):
    """Stack per-expert ``{prefix}.gate_proj / up_proj / down_proj`` layers into one
    ``EXL3SwitchGLU`` (``_stack_expert_switch_glu``, ponyexl3/mlx/model.py:77-127:
    all gates then all ups along the tile columns). Returns (module, consumed keys)."""
    from .moe import EXL3SwitchGLU

    gate, up, down, consumed = [], [], [], set()
    for ep in expert_prefixes:
        for proj, bucket in (("gate_proj", gate), ("up_proj", up), ("down_proj", down)):
            key = f"{ep}.{proj}"
            if key not in layers:
                raise KeyError(f"missing expert projection {key}")
            bucket.append(layers[key])
            consumed.add(key)
    return EXL3SwitchGLU.from_layers(gate, up, down, activation=activation, device=device), consumed


# Sibling projections called on the same input within one decoder layer: candidates
# for one-launch fused groups, longest first (ponyexl3/mlx/model.py:334-339).
FUSE_SIBLINGS = (
    ("mlp", ("gate_proj", "up_proj")),
    ("self_attn", ("q_proj", "k_proj", "v_proj")),
    ("self_attn", ("q_proj", "k_proj")),
    ("linear_attn", ("in_proj_qkv", "in_proj_z")),
)

# Groups at or below this many fp16-equivalent weight bytes stay unfused (the
# reference's HUGE_WEIGHT_BYTES default, ponyexl3/mlx/model.py:342-354).
FUSE_MIN_BYTES = 64 * 1024 * 1024


def swap_exl3_linears(model, layers: dict[str, EXL3Layer], *, prefix: str = "", device="cuda") -> int:
    """Replace every ``torch.nn.Linear`` of ``model`` whose qualified name (with
    ``prefix``) is a key of ``layers`` by an ``EXL3Linear`` (the module swap of
    ponyexl3/mlx/model.py:625-650). Returns the number of modules replaced."""
    import torch

    from .linear import EXL3Linear

    n = 0
    for name, module in list(model.named_modules()):
        for child_name, child in list(module.named_children()):
            full = ".".join(p for p in (prefix, name, child_name) if p)
            if isinstance(child, torch.nn.Linear) and full in layers:
                setattr(module, child_name, EXL3Linear(layers[full], device=device))
                n += 1
    return n


def fuse_exl3_siblings(model, *, min_bytes: int = FUSE_MIN_BYTES) -> int:
    """Replace same-K ``EXL3Linear`` sibling groups by ``FusedEXL3Group`` views
    (``fuse_exl3_siblings``, ponyexl3/mlx/model.py:357-432): only groups above
    ``min_bytes`` of fp16-equivalent weights that pass ``fusable``."""
    from .fused import FusedEXL3Group, FusedEXL3Sibling, fusable
    from .linear import EXL3Linear

    n = 0
    for owner_parent in list(model.modules()):
        for owner_name, names in FUSE_SIBLINGS:
            owner = getattr(owner_parent, owner_name, None)
            if owner is None:
                continue
            mods = [getattr(owner, nm, None) for nm in names]
            if any(isinstance(m, FusedEXL3Sibling) for m in mods):
                continue
            if not all(isinstance(m, EXL3Linear) for m in mods):
                continue
            members = [m._exl3 for m in mods]
            group_bytes = sum(l.in_features * l.out_features * 2 for l in members)
            if group_bytes <= min_bytes or not fusable(members):
                continue
            group = FusedEXL3Group(members)
            for i, nm in enumerate(names):
                setattr(owner, nm, group.sibling(i))
            n += 1
    return n
