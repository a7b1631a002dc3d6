"""Checkpoint reader against a checkpoint directory written on the fly in the
converted-model schema (quantization_config.json + safetensors), cf.
ponyexl3/ref/loader.py:41-173 and ponyexl3/convert/discovery.py:191-212."""
import json
import os

import numpy as np
import pytest
from safetensors.numpy import save_file

from ponyexl3_amd import loader, make_exl3_layer, unpack_signs_or_pass


def _pack_signs(signs):
    """+-1 fp16 (n,) -> int16 (n/16,) bitfield, bit set = negative (ponyexl3/ref/signs.py:8-19)."""
    bits = (np.asarray(signs, dtype=np.float32) < 0).astype(np.uint16).reshape(-1, 16)
    return (bits << np.arange(16, dtype=np.uint16)).sum(axis=1).astype(np.uint16).view(np.int16)


def _write_checkpoint(tmp_path, layers, *, shards=1, legacy_signs=(), wrong_mcg=None, plan_only=()):
    storage, tensors = {}, [dict() for _ in range(shards)]
    weight_map = {}
    for i, l in enumerate(layers):
        t = tensors[i % shards]
        fname = f"model-{i % shards:05d}.safetensors" if shards > 1 else "model.safetensors"
        stored = {}

        def put(name, arr):
            key = f"{l.key}.{name}"
            stored[key] = {"shape": list(arr.shape), "n_bytes": int(arr.nbytes)}
            if l.key not in plan_only:
                t[key] = np.ascontiguousarray(arr)
                weight_map[key] = fname

        put("trellis", l.trellis.view(np.int16))
        if l.key in legacy_signs:
            put("su", _pack_signs(l.suh))
            put("sv", _pack_signs(l.svh))
        else:
            put("suh", l.suh)
            put("svh", l.svh)
        if l.bias is not None:
            put("bias", l.bias)
        if l.mcg:
            mult = 0x12345678 if wrong_mcg == l.key else loader.MCG_MULT
            put("mcg", np.array(np.uint32(mult)).view(np.int32).reshape(()))
        if l.mul1:
            put("mul1", np.array(np.uint32(loader.MUL1_MULT)).view(np.int32).reshape(()))
        storage[l.key] = {"quant_format": "exl3", "bits_per_weight": l.k, "stored_tensors": stored,
                          "mcg_multiplier": bool(l.mcg), "mul1_multiplier": bool(l.mul1)}
    storage["model.norm"] = {"quant_format": "fp16"}
    (tmp_path / "quantization_config.json").write_text(json.dumps({"tensor_storage": storage}))
    for s in range(shards):
        fname = f"model-{s:05d}.safetensors" if shards > 1 else "model.safetensors"
        if tensors[s]:
            save_file(tensors[s], str(tmp_path / fname))
    if shards > 1:
        (tmp_path / "model.safetensors.index.json").write_text(json.dumps({"weight_map": weight_map}))
    loader.clear_weight_index_cache(str(tmp_path))
    return str(tmp_path)


def _layers():
    return [
        make_exl3_layer(k=4, in_features=256, out_features=128, seed=1, key="model.layers.0.mlp.gate_proj", mcg=True),
        make_exl3_layer(k=4, in_features=256, out_features=128, seed=2, key="model.layers.0.mlp.up_proj", mcg=True),
        make_exl3_layer(k=3, in_features=128, out_features=256, seed=3, key="model.layers.0.mlp.down_proj", bias=True),
        make_exl3_layer(k=6, in_features=128, out_features=128, seed=4, key="lm_head", mul1=True),
    ]


def test_list_meta_and_load(tmp_path):
    layers = _layers()
    d = _write_checkpoint(tmp_path, layers)
    infos = loader.list_exl3_layers(d)
    assert [i["key"] for i in infos] == sorted(l.key for l in layers)  # the fp16 entry is skipped
    meta = loader.layer_meta_from_config(d, "model.layers.0.mlp.down_proj")
    assert (meta["k"], meta["in_features"], meta["out_features"]) == (3, 128, 256)
    assert meta["trellis_shape"] == (8, 16, 48) and meta["n_tiles"] == 128
    assert meta["weight_fp16_bytes"] == 128 * 256 * 2 and not meta["mcg"]
    for l in layers:
        got = loader.load_exl3_layer(d, l.key)
        assert (got.k, got.in_features, got.out_features, got.mcg, got.mul1) == \
               (l.k, l.in_features, l.out_features, l.mcg, l.mul1)
        assert got.trellis.dtype == np.uint16
        np.testing.assert_array_equal(got.trellis, l.trellis)
        np.testing.assert_array_equal(got.suh, l.suh)
        np.testing.assert_array_equal(got.svh, l.svh)
        assert (got.bias is None) == (l.bias is None)
    assert set(loader.load_all_exl3_layers(d)) == {l.key for l in layers}


def test_sharded_index_and_legacy_packed_signs(tmp_path):
    layers = _layers()
    d = _write_checkpoint(tmp_path, layers, shards=3, legacy_signs={"lm_head"})
    got = loader.load_exl3_layer(d, "lm_head")
    assert got.suh.dtype == np.int16 and got.suh.shape == (8,)  # stored packed, unpacked on use
    np.testing.assert_array_equal(unpack_signs_or_pass(got.suh), layers[3].suh)
    np.testing.assert_array_equal(unpack_signs_or_pass(got.svh), layers[3].svh)
    np.testing.assert_array_equal(loader.load_exl3_layer(d, layers[1].key).trellis, layers[1].trellis)


def test_errors(tmp_path):
    layers = _layers()
    d = _write_checkpoint(tmp_path, layers, wrong_mcg=layers[0].key, plan_only={layers[2].key})
    with pytest.raises(ValueError, match="multiplier"):
        loader.load_exl3_layer(d, layers[0].key)
    loader.load_exl3_layer(d, layers[1].key)  # its multiplier is the supported one
    assert not loader.has_exl3_layer_weights(d, layers[2].key)  # in the config, not on disk
    with pytest.raises(FileNotFoundError):
        loader.load_exl3_layer(d, layers[2].key)
    with pytest.raises(KeyError):
        loader.layer_meta_from_config(d, "model.layers.9.mlp.gate_proj")
    with pytest.raises(FileNotFoundError):
        loader.list_exl3_layers(os.path.join(d, "nowhere"))


def test_directory_is_scanned_once_and_shards_found_without_an_index(tmp_path):
    """No index file and shards in a sub-directory: the tensor table comes from the
    shard headers, every shard is parsed once however many tensors are read, and the
    meta record is the package's own type (attribute and item access)."""
    layers = _layers()
    d = _write_checkpoint(tmp_path, layers, shards=2)
    os.remove(os.path.join(d, "model.safetensors.index.json"))
    sub = tmp_path / "shards"
    sub.mkdir()
    for fn in os.listdir(d):
        if fn.endswith(".safetensors"):
            os.rename(os.path.join(d, fn), str(sub / fn))
    loader.clear_weight_index_cache(d)
    opened = []
    orig = loader._Shard.__init__

    def counting(self, path):
        opened.append(path)
        orig(self, path)

    loader._Shard.__init__ = counting
    try:
        got = loader.load_all_exl3_layers(d)
        loader.load_exl3_layer(d, "lm_head")
    finally:
        loader._Shard.__init__ = orig
    assert sorted(os.path.basename(p) for p in opened) == ["model-00000.safetensors", "model-00001.safetensors"]
    for l in layers:
        np.testing.assert_array_equal(got[l.key].trellis, l.trellis)
    meta = loader.layer_meta_from_config(d, "lm_head")
    assert isinstance(meta, loader.LayerMeta) and meta.k == meta["k"] == 6
    assert meta.as_dict()["trellis_shape"] == (8, 8, 96)
    ck = loader.open_checkpoint(d)
    assert ck is loader.open_checkpoint(d) and ck.tensor("no.such.tensor") is None


def test_index_that_omits_tensors_and_corrupt_headers(tmp_path):
    """An index that lists the trellis but not the scales, bias or multiplier of a layer:
    the shards are looked through once and the layer still loads complete
    (ponyexl3/ref/loader.py:108-125 searches the shards per tensor). Offsets or a header
    length that point outside the file are refused."""
    import struct

    layers = _layers()
    d = _write_checkpoint(tmp_path, layers, shards=2)
    index_path = os.path.join(d, "model.safetensors.index.json")
    weight_map = json.load(open(index_path))["weight_map"]
    kept = {n: f for n, f in weight_map.items() if n.endswith(".trellis")}
    assert len(kept) < len(weight_map)
    json.dump({"weight_map": kept}, open(index_path, "w"))
    loader.clear_weight_index_cache(d)
    for l in layers:
        got = loader.load_exl3_layer(d, l.key)
        np.testing.assert_array_equal(got.suh, l.suh)
        np.testing.assert_array_equal(got.svh, l.svh)
        assert (got.bias is None) == (l.bias is None)
    # the multiplier check still runs for tensors the index does not list
    d2 = tmp_path / "wrong"
    d2.mkdir()
    d2 = _write_checkpoint(d2, layers, shards=2, wrong_mcg=layers[0].key)
    wm = json.load(open(os.path.join(d2, "model.safetensors.index.json")))["weight_map"]
    json.dump({"weight_map": {n: f for n, f in wm.items() if not n.endswith(".mcg")}},
              open(os.path.join(d2, "model.safetensors.index.json"), "w"))
    loader.clear_weight_index_cache(d2)
    with pytest.raises(ValueError, match="multiplier"):
        loader.load_exl3_layer(d2, layers[0].key)

    # data offsets beyond the file
    d3 = tmp_path / "corrupt"
    d3.mkdir()
    d3 = _write_checkpoint(d3, layers[:1])
    path = os.path.join(d3, "model.safetensors")
    raw = open(path, "rb").read()
    (hlen,) = struct.unpack("<Q", raw[:8])
    header = json.loads(raw[8 : 8 + hlen])
    name = layers[0].key + ".trellis"
    lo, hi = header[name]["data_offsets"]
    header[name]["data_offsets"] = [lo + (1 << 30), hi + (1 << 30)]
    blob = json.dumps(header).encode()
    open(path, "wb").write(struct.pack("<Q", len(blob)) + blob + raw[8 + hlen :])
    loader.clear_weight_index_cache(d3)
    with pytest.raises(ValueError, match="outside"):
        loader.load_exl3_layer(d3, layers[0].key)
    # header length beyond the file
    open(path, "wb").write(struct.pack("<Q", 1 << 40) + blob)
    loader.clear_weight_index_cache(d3)
    with pytest.raises(ValueError, match="past the end"):
        loader.load_exl3_layer(d3, layers[0].key)
