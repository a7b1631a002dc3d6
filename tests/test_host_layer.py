"""Host-side mirror of the reference's layer API (no GPU needed)."""
import numpy as np
import pytest

from ponyexl3_amd import (CodebookMode, EXL3Layer, codebook_mode_from_flags, make_exl3_layer,
                          unpack_sign_bitfield, unpack_signs_or_pass)


def test_codebook_flags():
    assert codebook_mode_from_flags() == CodebookMode.DEFAULT == 0
    assert codebook_mode_from_flags(mcg=True) == CodebookMode.MCG == 1
    assert codebook_mode_from_flags(mul1=True) == CodebookMode.MUL1 == 2
    assert codebook_mode_from_flags(mcg=True, mul1=True) == CodebookMode.MCG


def test_layer_validate():
    l = make_exl3_layer(k=3, in_features=128, out_features=256, seed=1)
    l.validate()
    assert l.packed_tile_size == 48 and l.trellis.shape == (8, 16, 48)
    assert l.codebook_mode == 0
    bad = EXL3Layer("x", 128, 256, 4, l.trellis)
    with pytest.raises(ValueError):
        bad.validate()
    with pytest.raises(ValueError):
        EXL3Layer("x", 120, 256, 3, l.trellis).validate()
    with pytest.raises(ValueError):
        EXL3Layer("x", 128, 256, 9, l.trellis).validate()


def test_sign_bitfield(oracle):
    bf = np.array([0x0001, -32768, 0x00F0], dtype=np.int16)
    s = unpack_sign_bitfield(bf)
    assert s.dtype == np.float16 and s.shape == (48,)
    assert s[0] == -1 and (s[1:16] == 1).all()
    assert s[31] == -1 and (s[16:31] == 1).all()
    assert (s[36:40] == -1).all() and (s[32:36] == 1).all()
    np.testing.assert_array_equal(s, oracle.unpack_signs_or_pass(bf))
    f = np.array([1, -1], dtype=np.float32)
    assert unpack_signs_or_pass(f).dtype == np.float16
    assert unpack_signs_or_pass(None) is None


def test_synthetic_layer_is_seeded():
    a = make_exl3_layer(k=4, in_features=128, out_features=128, seed=5, bias=True)
    b = make_exl3_layer(k=4, in_features=128, out_features=128, seed=5, bias=True)
    c = make_exl3_layer(k=4, in_features=128, out_features=128, seed=6)
    np.testing.assert_array_equal(a.trellis, b.trellis)
    np.testing.assert_array_equal(a.suh, b.suh)
    np.testing.assert_array_equal(a.bias, b.bias)
    assert (a.trellis != c.trellis).any()
    assert set(np.unique(a.suh).tolist()) == {-1.0, 1.0}


def test_fusable_rules():
    from ponyexl3_amd.fused import fusable

    mk = lambda k, out, seed, **kw: make_exl3_layer(k=k, in_features=256, out_features=out, seed=seed, **kw)
    assert fusable([mk(4, 384, 1), mk(4, 128, 2)])
    assert not fusable([mk(4, 384, 1)])
    assert not fusable([mk(4, 384, 1), mk(3, 128, 2)])
    assert not fusable([mk(4, 384, 1), mk(4, 128, 2, mcg=True)])
    assert not fusable([mk(4, 384, 1), mk(4, 128, 2, bias=True)])
    assert not fusable([mk(4, 384, 1), mk(4, 128, 2, suh=None)])
    assert not fusable([mk(4, 384, 1), mk(4, 144, 2)])
    assert not fusable([mk(4, 384, 1), make_exl3_layer(k=4, in_features=128, out_features=128)])


def test_group_sub_from_tile_sub():
    from ponyexl3_amd.ops import group_sub_from_tile_sub

    ts = np.repeat(np.arange(3, dtype=np.uint32), [24, 16, 8])
    assert group_sub_from_tile_sub(ts).tolist() == [0, 0, 0, 1, 1, 2]
    with pytest.raises(ValueError):
        group_sub_from_tile_sub(np.array([0] * 4 + [1] * 4))
    with pytest.raises(ValueError):
        group_sub_from_tile_sub(np.zeros(12))


def test_ops_reject_cpu_tensors():
    import torch

    from ponyexl3_amd import ops

    with pytest.raises(ValueError):
        ops.decode_full(torch.zeros((1, 1, 64), dtype=torch.int16), 4, 0)
    with pytest.raises(ValueError):
        ops.had128_pre(torch.zeros((1, 128), dtype=torch.float16), None)


def test_tensor_core_perm_closed_form(oracle):
    """The package's closed form equals the oracle's table (itself pinned by the
    reference-written one) and is a bijection."""
    from ponyexl3_amd.layer import tensor_core_perm, tensor_core_perm_inverse

    perm = tensor_core_perm()
    np.testing.assert_array_equal(perm, oracle.tensor_core_perm())
    assert sorted(perm.tolist()) == list(range(256))
    np.testing.assert_array_equal(perm[tensor_core_perm_inverse()], np.arange(256))


def test_ref_compatible_synthetic_layers_match_the_reference_bit_for_bit():
    """make_exl3_layer(ref_compatible=True) against the layers that the reference's own
    make_exl3_layer produced for tests/golden/forwards.npz (seed = 40 + K + 10*cb,
    128 -> 256): trellis words, both sign vectors and the bias."""
    from conftest import golden
    from ponyexl3_amd import make_exl3_layer

    g = golden("forwards.npz")
    cases = [(k, cb, False) for k in range(1, 9) for cb in (0, 1)] + [(4, 2, False), (4, 0, True)]
    for k, cb, bias in cases:
        tag = f"k{k}_cb{cb}" + ("_bias" if bias else "")
        layer = make_exl3_layer(k=k, in_features=128, out_features=256, seed=40 + k + 10 * cb,
                                mcg=cb == 1, mul1=cb == 2, bias=bias, ref_compatible=True)
        assert layer.key == "test.layer"
        np.testing.assert_array_equal(layer.trellis, g[tag + "_trellis"], err_msg=tag)
        np.testing.assert_array_equal(layer.suh.view(np.uint16), g[tag + "_suh"], err_msg=tag)
        np.testing.assert_array_equal(layer.svh.view(np.uint16), g[tag + "_svh"], err_msg=tag)
        if bias:
            np.testing.assert_array_equal(layer.bias.view(np.uint16), g[tag + "_bias"].view(np.uint16))
    pub = make_exl3_layer(k=4, in_features=128, out_features=256, seed=77, ref_compatible=True)
    np.testing.assert_array_equal(pub.trellis, g["pub_trellis"])
    np.testing.assert_array_equal(pub.suh.view(np.uint16), g["pub_suh"])


def test_pack_trellis_tiles_matches_the_oracle_packer(oracle):
    from ponyexl3_amd.layer import pack_trellis_tiles

    rng = np.random.default_rng(3)
    for k in range(1, 9):
        sym = rng.integers(0, 65536, size=(3, 2, 256), dtype=np.uint16)
        got = pack_trellis_tiles(sym, k)
        want = oracle.pack_trellis((sym & ((1 << k) - 1)).astype(np.uint16), k)
        np.testing.assert_array_equal(got, want)
