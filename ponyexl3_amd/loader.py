"""Converted-checkpoint reader: ``quantization_config.json`` + safetensors ->
``EXL3Layer`` objects, expert stacking and the sibling-fusion policy.

Host-side only (numpy; torch is touched where modules are built). A model
directory is scanned once into a ``Checkpoint``: the EXL3 records of the config and
a tensor-name -> shard table from the index file or the shard headers; tensors are
views into memory-mapped shards. The module-level functions keep the names of
``ponyexl3/ref/loader.py:41-173``; the module-building helpers follow
``ponyexl3/mlx/model.py``: multiplier check (:261-283), expert stacking (:77-127),
fusion policy (:325-432).

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
import mmap
import os
import struct
from dataclasses import asdict, dataclass
from typing import Any, Iterator

import numpy as np

from .layer import EXL3Layer

MCG_MULT = 0xCBAC1FED  # ponyexl3/ref/codebook.py:19-20
MUL1_MULT = 0x83DCD12D

# safetensors dtype tag -> numpy dtype, for the tensors an EXL3 module stores
_ST_DTYPES = {"I16": np.int16, "U16": np.uint16, "F16": np.float16, "F32": np.float32,
              "I32": np.int32, "U32": np.uint32, "I64": np.int64, "U8": np.uint8, "I8": np.int8}


class _Shard:
    """One .safetensors file: 8-byte little-endian header length, a JSON header
    {name: {dtype, shape, data_offsets}}, then the raw tensor bytes. The header is
    parsed once; tensors are read-only views into one memory map of the file."""

    def __init__(self, path: str):
        self.path = path
        size = os.path.getsize(path)
        with open(path, "rb") as f:
            head = f.read(8)
            if len(head) < 8:
                raise ValueError(f"{path}: too short for a safetensors file")
            (hlen,) = struct.unpack("<Q", head)
            if 8 + hlen > size:
                raise ValueError(f"{path}: header of {hlen} bytes runs past the end of the file ({size} bytes)")
            header = json.loads(f.read(hlen))
        header.pop("__metadata__", None)
        self.entries: dict[str, dict] = header
        self._base = 8 + hlen
        self._data_bytes = size - self._base
        self._map: mmap.mmap | None = None

    def names(self) -> Iterator[str]:
        return iter(self.entries)

    def tensor(self, name: str) -> np.ndarray:
        e = self.entries[name]
        dt = _ST_DTYPES.get(e["dtype"])
        if dt is None:
            raise ValueError(f"{self.path}: tensor {name!r} has unsupported dtype {e['dtype']}")
        if self._map is None:
            with open(self.path, "rb") as f:
                self._map = mmap.mmap(f.fileno(), 0, access=mmap.ACCESS_READ)
        lo, hi = (int(v) for v in e["data_offsets"])
        if not 0 <= lo <= hi <= self._data_bytes:
            raise ValueError(f"{self.path}: tensor {name!r} has data offsets [{lo}, {hi}) outside the "
                             f"{self._data_bytes} data bytes of the file")
        n = int(np.prod(e["shape"], dtype=np.int64)) if e["shape"] else 1
        if hi - lo != n * np.dtype(dt).itemsize:
            raise ValueError(f"{self.path}: tensor {name!r} has {hi - lo} bytes for shape {e['shape']}")
        return np.frombuffer(self._map, dtype=dt, count=n, offset=self._base + lo).reshape(e["shape"])


@dataclass(frozen=True)
class LayerMeta:
    """Dimensions of one EXL3 module as recorded in quantization_config.json."""

    key: str
    k: int
    bits_per_weight: Any
    in_features: int
    out_features: int
    in_tiles: int
    out_tiles: int
    n_tiles: int
    trellis_shape: tuple
    trellis_bytes: int
    weight_fp16_bytes: int
    mcg: bool
    mul1: bool

    def __getitem__(self, name: str):  # meta["k"], as callers of the reference's dict expect
        return getattr(self, name)

    def as_dict(self) -> dict[str, Any]:
        return asdict(self)


class Checkpoint:
    """A converted model directory, scanned once: the EXL3 records of
    quantization_config.json and a tensor-name -> shard table built from
    model.safetensors.index.json or, without one, from the headers of every
    *.safetensors file below the directory. Shards stay mapped while the object lives."""

    def __init__(self, model_dir: str):
        self.model_dir = model_dir
        qpath = os.path.join(model_dir, "quantization_config.json")
        if not os.path.isfile(qpath):
            raise FileNotFoundError(f"no quantization_config.json in {model_dir}")
        with open(qpath, encoding="utf-8") as f:
            storage = json.load(f).get("tensor_storage", {})
        self.records: dict[str, dict] = {key: rec for key, rec in storage.items()
                                         if rec.get("quant_format") == "exl3"}
        self._shards: dict[str, _Shard] = {}
        self._where: dict[str, str] = {}
        index = os.path.join(model_dir, "model.safetensors.index.json")
        listed: dict[str, str] = {}
        if os.path.isfile(index):
            with open(index, encoding="utf-8") as f:
                listed = json.load(f).get("weight_map", {})
        for name, rel in listed.items():
            path = os.path.join(model_dir, rel)
            if os.path.isfile(path):
                self._where[name] = path
        self._scanned = False
        if len(self._where) < len(listed) or not listed:
            # no index, or one that names files that are not there: read the headers
            self._scan_shards()

    def _scan_shards(self) -> None:
        """Reads the header of every *.safetensors file below the directory once and
        adds the tensors no index entry covers."""
        if self._scanned:
            return
        self._scanned = True
        for root, _dirs, files in sorted(os.walk(self.model_dir)):
            for fn in sorted(files):
                if fn.endswith(".safetensors"):
                    shard = self._shard(os.path.join(root, fn))
                    for name in shard.names():
                        self._where.setdefault(name, shard.path)

    def _shard(self, path: str) -> _Shard:
        if path not in self._shards:
            self._shards[path] = _Shard(path)
        return self._shards[path]

    def has(self, tensor_name: str) -> bool:
        path = self._where.get(tensor_name)
        if path is None or tensor_name not in self._shard(path).entries:
            # an index may omit tensors that a shard holds (the reference looks through
            # the shards per tensor, ponyexl3/ref/loader.py:108-125): scan once, then trust
            # the table
            self._scan_shards()
            path = self._where.get(tensor_name)
            if path is not None and tensor_name not in self._shard(path).entries:
                for shard in self._shards.values():
                    if tensor_name in shard.entries:
                        path = self._where[tensor_name] = shard.path
                        break
        return path is not None and tensor_name in self._shard(path).entries

    def tensor(self, tensor_name: str) -> np.ndarray | None:
        """A copy of the stored tensor, or None when no shard holds it."""
        if not self.has(tensor_name):
            return None
        return np.array(self._shard(self._where[tensor_name]).tensor(tensor_name))

    def keys(self) -> list[str]:
        return sorted(self.records)

    def meta(self, key: str) -> LayerMeta:
        rec = self.records.get(key)
        if rec is None:
            raise KeyError(f"quantization_config.json has no EXL3 record for {key!r}")
        stored = rec.get("stored_tensors", {})
        entry = stored.get(f"{key}.trellis")
        if entry is None:
            raise KeyError(f"record of {key!r} lists no trellis tensor")
        in_tiles, out_tiles, packed = (int(v) for v in entry["shape"])
        return LayerMeta(
            key=key, k=packed // 16, bits_per_weight=rec.get("bits_per_weight"),
            in_features=16 * in_tiles, out_features=16 * out_tiles, in_tiles=in_tiles,
            out_tiles=out_tiles, n_tiles=in_tiles * out_tiles,
            trellis_shape=(in_tiles, out_tiles, packed), trellis_bytes=int(entry.get("n_bytes", 0)),
            weight_fp16_bytes=in_tiles * out_tiles * 256 * 2, mcg=bool(rec.get("mcg_multiplier")),
            mul1=bool(rec.get("mul1_multiplier")))

    def check_multiplier(self, key: str, name: str, expected: int) -> None:
        stored = self.tensor(f"{key}.{name}")
        if stored is None:
            return  # older checkpoints carry only the flag
        got = int(stored.astype(np.int64).ravel()[0]) & 0xFFFFFFFF
        if got != int(expected):
            raise ValueError(f"{key}: the checkpoint was quantized with {name} multiplier {got:#010x}; "
                             f"the kernels implement {int(expected):#010x} only")

    def layer(self, key: str) -> EXL3Layer:
        meta = self.meta(key)
        trellis = self.tensor(f"{key}.trellis")
        if trellis is None:
            raise FileNotFoundError(f"{key}.trellis is listed in quantization_config.json but in no shard")
        if trellis.dtype.itemsize != 2 or trellis.dtype.kind not in "iu":
            raise ValueError(f"{key}.trellis must be a 16-bit integer tensor, found {trellis.dtype}")
        if meta.mcg:
            self.check_multiplier(key, "mcg", MCG_MULT)
        if meta.mul1:
            self.check_multiplier(key, "mul1", MUL1_MULT)

        def first(*names):
            for n in names:
                t = self.tensor(f"{key}.{n}")
                if t is not None:
                    return t
            return None

        layer = EXL3Layer(key=key, in_features=meta.in_features, out_features=meta.out_features,
                          k=meta.k, trellis=trellis.view(np.uint16), suh=first("suh", "su"),
                          svh=first("svh", "sv"), bias=first("bias"), mcg=meta.mcg, mul1=meta.mul1)
        layer.validate()
        return layer


_CHECKPOINTS: dict[str, Checkpoint] = {}


def open_checkpoint(model_dir: str) -> Checkpoint:
    """The (cached) scan of a model directory."""
    ck = _CHECKPOINTS.get(model_dir)
    if ck is None:
        ck = _CHECKPOINTS[model_dir] = Checkpoint(model_dir)
    return ck


def clear_weight_index_cache(model_dir: str) -> None:
    """Forget the scan of a model directory (its files changed)."""
    _CHECKPOINTS.pop(model_dir, None)


def list_exl3_layers(model_dir: str) -> list[dict[str, Any]]:
    """One entry per EXL3 module of quantization_config.json, sorted by key
    (the listing of ponyexl3/ref/loader.py:41-67)."""
    ck = open_checkpoint(model_dir)
    return [{"key": key, "bits_per_weight": ck.records[key].get("bits_per_weight"),
             "stored_tensors": ck.records[key].get("stored_tensors", {}),
             "mcg": bool(ck.records[key].get("mcg_multiplier")),
             "mul1": bool(ck.records[key].get("mul1_multiplier"))} for key in ck.keys()]


def layer_meta_from_config(model_dir: str, module_key: str) -> LayerMeta:
    """Shapes and sizes of a module from the config alone; no tensor is read
    (ponyexl3/ref/loader.py:70-103)."""
    return open_checkpoint(model_dir).meta(module_key)


def has_exl3_layer_weights(model_dir: str, module_key: str) -> bool:
    """Whether a shard holds the module's trellis (a plan-only config lists modules
    that were never written)."""
    return open_checkpoint(model_dir).has(f"{module_key}.trellis")


def check_multiplier(model_dir: str, module_key: str, name: str, expected: int) -> None:
    """The codebooks hard-code their multipliers; a checkpoint quantized with another
    one is refused rather than decoded to garbage (ponyexl3/mlx/model.py:261-270)."""
    open_checkpoint(model_dir).check_multiplier(module_key, name, expected)


def load_exl3_layer(model_dir: str, module_key: str) -> EXL3Layer:
    """One EXL3 module by key, e.g. model.layers.0.mlp.gate_proj
    (ponyexl3/ref/loader.py:138-173)."""
    return open_checkpoint(model_dir).layer(module_key)


def load_all_exl3_layers(model_dir: str) -> dict[str, EXL3Layer]:
    """Every EXL3 module whose trellis is on disk, by key."""
    ck = open_checkpoint(model_dir)
    return {key: ck.layer(key) for key in ck.keys() if ck.has(f"{key}.trellis")}


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
