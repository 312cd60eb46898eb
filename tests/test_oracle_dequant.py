"""Pins the oracle's dequantise / meta-dequantise / matmul restatements
(src/custom_layers.py:55-116, src/triton_kernels.py:86-131) by closed forms,
scalar brute force with the group-index identity, an integer-only fp16
rounding in C, and fp64 brute force."""
import numpy as np
import pytest

from oracle import c_oracle
from oracle import hqq_oracle as o

F16 = np.float16


def test_c_half_conversion_matches_ieee_all_halves_and_ties():
    lib = c_oracle.lib()
    bits = np.arange(65536, dtype=np.uint16)
    halves = bits.view(F16)
    for b in range(0, 65536, 7):  # every 7th pattern: all classes covered
        f = lib.oracle_h2f(int(b))
        if np.isnan(halves[b]):
            assert np.isnan(f)
            continue
        assert np.float32(f) == np.float32(halves[b])
        assert lib.oracle_f2h(float(np.float32(halves[b]))) == b
    rng = np.random.default_rng(0)
    vals = np.concatenate([
        rng.standard_normal(20000).astype(np.float32) * np.float32(10) ** rng.integers(-9, 6, 20000).astype(np.float32),
        # exact ties between neighbouring halves, and their float neighbours
        ((halves[1024:2048].astype(np.float32) + halves[1025:2049].astype(np.float32)) / 2),
        np.nextafter((halves[1024:2048].astype(np.float32) + halves[1025:2049].astype(np.float32)) / 2, np.float32(0)),
        np.array([65504, 65519.996, 65520, 1e9, 2.0 ** -25, np.nextafter(np.float32(2.0 ** -25), np.float32(1)), 2.0 ** -24,
                  3 * 2.0 ** -25, 6.1e-5, 0.0, -0.0], dtype=np.float32),
    ]).astype(np.float32)
    with np.errstate(over="ignore"):
        want = vals.astype(F16).view(np.uint16)
    got = np.array([lib.oracle_f2h(float(v)) for v in vals], dtype=np.uint16)
    np.testing.assert_array_equal(got, want)


def test_two_roundings_hand_example():
    # q=3, z=fp16(1.3), s=fp16(0.0123): t = fp16(3-1.2998046875) = 1.7001953125 (exact),
    # w = fp16(1.7001953125 * 0.0123):  checked by exact rational arithmetic below.
    from fractions import Fraction

    z, s = F16(1.3), F16(0.0123)
    t = Fraction(3) - Fraction(float(z))
    # round t to fp16 by hand: fp16 spacing in [1,2) is 2^-10
    t16 = Fraction(round(t * 1024), 1024)
    prod = t16 * Fraction(float(s))
    # spacing of fp16 near 0.0209 is 2^-16
    w_exact = Fraction(round(prod * 65536), 65536)
    layer = {"nbits": 4, "group_size": 2, "shape": (2, 1), "W_q": o.pack_4bit_u8(np.array([[3], [3]], np.uint8)),
             "scale": np.array([[s]], F16), "zero": np.array([[z]], F16)}
    w = o.dequantize(layer)
    assert Fraction(float(w[0, 0])) == w_exact


def _tiny_layers():
    rng = np.random.default_rng(7)
    for nbits, n, k, gs, mgs in [(4, 16, 8, 4, 4), (4, 32, 16, 8, 8), (2, 32, 8, 4, 4), (2, 64, 16, 16, 8),
                                 (3, 20, 8, 4, 8), (3, 40, 16, 8, 16), (3, 64, 8, 16, 4)]:
        for qs, qz in [(True, True), (False, False), (True, False)]:
            layer, w = o.random_layer(rng, n, k, nbits, gs, qs, qz, meta_group_size=mgs)
            yield layer, w


def test_group_index_identity_brute_force():
    """dequantize() uses the reference's reshape((gs,-1)); dequantize_scalar()
    uses the kernels' table row n % G.  They must be the same function."""
    cnt = 0
    for layer, _ in _tiny_layers():
        a = o.dequantize(layer)
        b = o.dequantize_scalar(layer)
        np.testing.assert_array_equal(a.view(np.uint16), b.view(np.uint16))
        cnt += 1
    assert cnt == 21


def test_dequantize_c_vs_numpy_bit_exact():
    for layer, _ in _tiny_layers():
        n, k = layer["shape"]
        s, z = o.expand_tables(layer)
        got = c_oracle.dequantize(layer["W_q"], layer["nbits"], n, k, layer["group_size"], s, z)
        np.testing.assert_array_equal(got.view(np.uint16), o.dequantize(layer).view(np.uint16))


def test_meta_dequant_layout_scalar_brute_force():
    """Scale entry i lives at scale_q[i // C, i % C] with meta column i % C
    (reshape of a (mgs, C) array to (1, S)); zero uses one scalar pair."""
    rng = np.random.default_rng(3)
    mgs, c = 8, 6
    q = rng.integers(0, 256, size=(mgs, c), dtype=np.uint8)
    ms = (rng.random((1, c)) * 0.01).astype(F16)
    mz = (rng.random((1, c)) * 100).astype(F16)
    got = o.meta_dequant(q, ms, mz, (1, mgs * c))
    for i in range(mgs * c):
        t = F16(np.float32(q[i // c, i % c]) - np.float32(mz[0, i % c]))
        want = F16(np.float32(t) * np.float32(ms[0, i % c]))
        assert got[0, i].view(np.uint16) == want.view(np.uint16)
    np.testing.assert_array_equal(c_oracle.meta_dequant(q, ms, mz).reshape(1, -1).view(np.uint16), got.view(np.uint16))
    zq = rng.integers(0, 256, size=(1, 48), dtype=np.uint8)
    got = o.meta_dequant(zq, F16(0.02), F16(3.0), (1, 48))
    want = c_oracle.meta_dequant(zq, F16(0.02), F16(3.0))
    np.testing.assert_array_equal(want.view(np.uint16), got.view(np.uint16))


def test_dequant_is_close_to_the_weights_it_quantised():
    # sanity of the whole pipeline: 4-bit g64 reconstruction error is a fraction of one step
    rng = np.random.default_rng(5)
    layer, w = o.random_layer(rng, 256, 64, 4, 64)
    err = np.abs(o.dequantize(layer).astype(np.float32) - w.astype(np.float32)).max()
    assert err < 0.02 * 6 / 15


def test_matmul_fp64_brute_force_and_linearity():
    rng = np.random.default_rng(11)
    for layer, _ in _tiny_layers():
        n, k = layer["shape"]
        x = rng.standard_normal((3, k)).astype(F16)
        w = o.dequantize_scalar(layer)
        want = np.zeros((3, n))
        for m in range(3):
            for j in range(n):
                want[m, j] = sum(float(x[m, kk]) * float(w[j, kk]) for kk in range(k))
        y = o.matmul_transpose(x, layer)
        assert y.dtype == F16 and y.shape == (3, n)
        np.testing.assert_array_equal(y.view(np.uint16), want.astype(F16).view(np.uint16))
        yc = c_oracle.matmul_transpose(x, w)
        assert np.abs(yc.astype(np.float64) - want).max() <= 1e-3 * np.abs(want).max() + 1e-6
        # linearity in x (exact in the fp64 accumulator up to final rounding)
        y2 = o.matmul_transpose((x.astype(np.float32) * 2).astype(F16), layer)
        np.testing.assert_array_equal(y2.view(np.uint16), (want * 2).astype(F16).view(np.uint16))


def test_bias_and_leading_dims():
    rng = np.random.default_rng(2)
    layer, _ = o.random_layer(rng, 16, 8, 4, 4, meta_group_size=8)
    x = rng.standard_normal((2, 3, 8)).astype(F16)
    b = rng.standard_normal(16).astype(F16)
    y = o.matmul_transpose(x, layer, bias=b)
    assert y.shape == (2, 3, 16)
    y0 = o.matmul_transpose(x.reshape(6, 8), layer)
    np.testing.assert_array_equal(y.reshape(6, 16), (y0 + b).astype(F16))
