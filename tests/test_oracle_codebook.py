"""Pins oracle.exl3o_decode_cw (restates ponyexl3/ref/codebook.py:66-91)."""
import numpy as np
import pytest

from conftest import golden


@pytest.mark.parametrize("cb", [0, 1, 2])
def test_full_table_matches_reference(oracle, cb):
    ref = golden("codebook_tables.npz")[f"cb{cb}"]
    got = oracle.decode_table(cb).view(np.uint16)
    np.testing.assert_array_equal(got, ref)


def test_known_answers(oracle):
    # hand-derived from x = cw*M + A; (x & 0x8FFF8FFF) ^ 0x3B603B60; half add
    kat = {
        (0, 0): 0x3A25, (0, 1): 0x3F60, (0, 2): 0xC2E8,
        (1, 0): 0xBB5B, (1, 1): 0x304E, (1, 2): 0x3921,
        (0xFFFF, 0): 0xB110, (0xFFFF, 1): 0x3ACD, (0xFFFF, 2): 0xB936,
    }
    for (cw, cb), bits in kat.items():
        assert int(oracle.decode_cw(cw, cb).view(np.uint16)) == bits, (cw, cb)


def _half_add_bits(x):
    lo = (x & 0xFFFF).astype(np.uint16).view(np.float16)
    hi = (x >> 16).astype(np.uint16).view(np.float16)
    return (lo + hi).view(np.uint16)  # numpy fp16 add: one rounding


@pytest.mark.parametrize("cb,mult,add", [(0, 89226354, 64248484), (1, 0xCBAC1FED, 0)])
def test_closed_form_all_codewords(oracle, cb, mult, add):
    """Independent vectorised restatement: 64-bit product wrapped to 32 bits,
    LOP3 0x6A == c ^ (a & b) (tests/test_codebook.py:16-31), numpy half add."""
    cw = np.arange(65536, dtype=np.uint64)
    x = ((cw * np.uint64(mult) + np.uint64(add)) & np.uint64(0xFFFFFFFF)).astype(np.uint32)
    x = (x & np.uint32(0x8FFF8FFF)) ^ np.uint32(0x3B603B60)
    np.testing.assert_array_equal(oracle.decode_table(cb).view(np.uint16), _half_add_bits(x))


def test_lop3_truth_table():
    a, b, c = 0xA5A5A5A5, 0x8FFF8FFF, 0x3B603B60
    out = 0
    for bit in range(32):
        idx = (((a >> bit) & 1) << 2) | (((b >> bit) & 1) << 1) | ((c >> bit) & 1)
        out |= ((0x6A >> idx) & 1) << bit
    assert out == (a & b) ^ c


def test_mul1_is_affine_in_byte_sum(oracle):
    cw = np.arange(65536, dtype=np.uint64)
    x = ((cw * np.uint64(0x83DCD12D)) & np.uint64(0xFFFFFFFF)).astype(np.uint32)
    s = (x & 0xFF) + ((x >> 8) & 0xFF) + ((x >> 16) & 0xFF) + (x >> 24)
    k_inv = float(np.array([0x1EEE], dtype=np.uint16).view(np.float16)[0])
    k_bias = float(np.array([0xC931], dtype=np.uint16).view(np.float16)[0])
    expect = ((1024.0 + s.astype(np.float64)) * k_inv + k_bias).astype(np.float16)
    np.testing.assert_array_equal(oracle.decode_table(2).view(np.uint16), expect.view(np.uint16))


@pytest.mark.parametrize("cb", [0, 1, 2])
def test_finite_and_bounded(oracle, cb):
    v = oracle.decode_table(cb).astype(np.float32)
    assert np.isfinite(v).all()
    assert np.abs(v).max() < 16.0  # tests/test_codebook.py:34-40 (actual bound < 4 / < 11)


def test_codebook_scale(oracle):
    # 3INST table std == CODEBOOK_SCALE = 1.24371088 (convert/regularize.py:13)
    assert abs(float(oracle.decode_table(0).astype(np.float64).std()) - 1.24371088) < 1e-5
