"""Pins the oracle's packers (src/packing.py:10-97) without running the reference:
hand-computed known answers, exhaustive byte values, closed forms per lane,
the reference kernels' own shift formulas, and the independent C restatement."""
import json
import os

import numpy as np
import pytest

from oracle import c_oracle
from oracle import hqq_oracle as o

GOLD = os.path.join(os.path.dirname(__file__), "golden", "packing_known_answers.json")


def _cases():
    with open(GOLD) as f:
        for c in json.load(f)["cases"]:
            codes = np.array(c["codes"], dtype=np.uint8)
            if "packed" in c:
                packed = np.array(c["packed"], dtype=np.uint8)
            else:
                packed = np.array([[int(w, 8) for w in row] for row in c["packed_octal"]], dtype=np.int64).astype(np.int32)
            yield c["nbits"], codes, packed


@pytest.mark.parametrize("impl", ["numpy", "c"])
def test_known_answers(impl):
    n = 0
    for nbits, codes, packed in _cases():
        got = o.PACK[nbits](codes) if impl == "numpy" else c_oracle.pack(codes, nbits)
        assert got.dtype == packed.dtype
        np.testing.assert_array_equal(got, packed)
        back = o.UNPACK[nbits](packed) if impl == "numpy" else c_oracle.unpack(packed, nbits)
        np.testing.assert_array_equal(back[: codes.shape[0]], codes)
        assert not back[codes.shape[0]:].any()  # spare rows of a 3-bit tail are zero
        n += 1
    assert n >= 8


def test_exhaustive_bytes_4bit_2bit():
    b = np.arange(256, dtype=np.uint8).reshape(1, 256)
    u4 = o.unpack_4bit_u8(b)
    np.testing.assert_array_equal(u4[0], np.arange(256) // 16)
    np.testing.assert_array_equal(u4[1], np.arange(256) % 16)
    np.testing.assert_array_equal(o.pack_4bit_u8(u4), b)
    u2 = o.unpack_2bit_u8(b)
    for i in range(4):
        np.testing.assert_array_equal(u2[i], (np.arange(256) // 4 ** (3 - i)) % 4)
    np.testing.assert_array_equal(o.pack_2bit_u8(u2), b)
    np.testing.assert_array_equal(c_oracle.unpack(b, 4), u4)
    np.testing.assert_array_equal(c_oracle.unpack(b, 2), u2)


def test_3bit_every_code_in_every_lane():
    for lane in range(10):
        for code in range(8):
            q = np.zeros((10, 1), np.uint8)
            q[lane, 0] = code
            w = o.pack_3bit_i32(q)
            assert w.shape == (1, 1) and w.dtype == np.int32
            assert int(w[0, 0]) == code * 8 ** (9 - lane)  # closed form: octal digit
            assert int(w[0, 0]) >> 30 == 0  # top two bits stay clear
            np.testing.assert_array_equal(o.unpack_3bit_i32(w), q)
            np.testing.assert_array_equal(c_oracle.pack(q, 3), w)


@pytest.mark.parametrize("h", list(range(1, 26)))
def test_3bit_tail_heights(h):
    rng = np.random.default_rng(h)
    q = rng.integers(0, 8, size=(h, 3), dtype=np.uint8)
    w = o.pack_3bit_i32(q)
    assert w.shape == ((h + 9) // 10, 3)
    u = o.unpack_3bit_i32(w)
    assert u.shape == (10 * w.shape[0], 3)
    np.testing.assert_array_equal(u[:h], q)
    assert not u[h:].any()
    # closed form of every word: sum of octal digits
    for p in range(w.shape[0]):
        for c in range(3):
            want = sum(int(q[10 * p + i, c]) * 8 ** (9 - i) for i in range(10) if 10 * p + i < h)
            assert int(w[p, c]) == want
    np.testing.assert_array_equal(c_oracle.pack(q, 3), w)
    np.testing.assert_array_equal(c_oracle.unpack(w, 3), u)


@pytest.mark.parametrize("nbits,h", [(4, 16), (2, 24), (3, 37), (3, 40)])
def test_against_reference_kernel_shift_formulas(nbits, h):
    """src/triton_kernels.py:91,279,469 state independently which bits of which
    word hold weight (n, k); the packers must agree with them."""
    rng = np.random.default_rng(nbits * 100 + h)
    q = rng.integers(0, 2 ** nbits, size=(h, 5), dtype=np.uint8)
    packed = o.PACK[nbits](q)
    for n in range(h):
        for k in range(5):
            assert o.kernel_code(packed, nbits, n, k) == int(q[n, k])


@pytest.mark.parametrize("nbits", [2, 3, 4])
def test_numpy_vs_c_random_and_roundtrip(nbits):
    rng = np.random.default_rng(nbits)
    h = {4: 128, 2: 128, 3: 126}[nbits]
    q = rng.integers(0, 2 ** nbits, size=(h, 67), dtype=np.uint8)
    p_np = o.PACK[nbits](q)
    np.testing.assert_array_equal(c_oracle.pack(q, nbits), p_np)
    np.testing.assert_array_equal(o.UNPACK[nbits](p_np)[:h], q)
    np.testing.assert_array_equal(c_oracle.unpack(p_np, nbits)[:h], q)


def test_pack_does_not_mask_like_the_reference():
    # src/packing.py:15 shifts in uint8 and ORs the odd row unmasked
    q = np.array([[0x13], [0x25]], dtype=np.uint8)
    assert int(o.pack_4bit_u8(q)[0, 0]) == ((0x13 << 4) & 0xFF) | 0x25


def test_asserts_like_the_reference():
    with pytest.raises(AssertionError):
        o.pack_4bit_u8(np.zeros((3, 1), np.uint8))  # src/packing.py:12
    with pytest.raises(AssertionError):
        o.unpack_3bit_i32(np.zeros((1, 1), np.uint8))  # src/packing.py:88


def test_repack_from_quantise_layout():
    """src/custom_layers.py:41-47: the quantiser's (gs, N*K/gs) layout has the
    same flat order as W, padded at the end for 3 bit."""
    n, k, gs = 20, 8, 4
    rng = np.random.default_rng(0)
    q_nk = rng.integers(0, 8, size=(n, k), dtype=np.uint8)
    quant_layout = q_nk.reshape(gs, -1)
    padded = np.concatenate([quant_layout, np.zeros((10 - gs, quant_layout.shape[1]), np.uint8)])
    for src in (quant_layout, padded):
        packed = o.repack(src, (n, k), 3)
        np.testing.assert_array_equal(o.unpack_3bit_i32(packed)[:n], q_nk)
