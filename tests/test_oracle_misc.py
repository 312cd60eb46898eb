"""Pins the remaining oracle pieces: expert FFN / router arithmetic, the
reference's slab layout (src/expert_wrapper.py:41-57) and the LRU model
(src/expert_cache.py:33-52,120-201)."""
import math

import numpy as np

from oracle import hqq_oracle as o

F16 = np.float16


def test_silu_and_ffn_scalar():
    x = np.array([-3.0, -0.5, 0.0, 0.7, 4.0], F16)
    want = [F16(float(v) / (1 + math.exp(-float(v)))) for v in x]
    np.testing.assert_array_equal(o.silu_f16(x), np.array(want, F16))
    rng = np.random.default_rng(0)
    w1, _ = o.random_layer(rng, 32, 16, 2, 16, meta_group_size=8)
    w3, _ = o.random_layer(rng, 32, 16, 2, 16, meta_group_size=8)
    w2, _ = o.random_layer(rng, 16, 32, 2, 16, meta_group_size=8)
    xx = rng.standard_normal((2, 16)).astype(F16)
    a = o.matmul_transpose(xx, w1)
    b = o.matmul_transpose(xx, w3)
    h = np.array([[F16(np.float32(F16(float(a[m, j]) / (1 + math.exp(-float(a[m, j]))))) * np.float32(b[m, j]))
                   for j in range(32)] for m in range(2)], F16)
    np.testing.assert_array_equal(o.expert_ffn(xx, w1, w2, w3), o.matmul_transpose(h, w2))


def test_router_closed_form():
    # logits chosen by hand: expert 3 and 1 win; weights = softmax renormalised over the two
    gate = np.zeros((8, 4), F16)
    gate[3, 0] = 2.0
    gate[1, 0] = 1.0
    gate[5, 0] = -1.0
    h = np.array([[1.0, 0, 0, 0]], F16)
    w, idx, logits = o.router(h, gate)
    assert idx.tolist() == [[3, 1]]
    e2, e1 = math.exp(2.0), math.exp(1.0)
    np.testing.assert_allclose(w.astype(np.float64), [[e2 / (e2 + e1), e1 / (e2 + e1)]], rtol=1e-3)
    assert logits.dtype == F16 and w.dtype == F16


def test_slab_layout_totals_mixtral_2bit_g16():
    """Closed-form byte counts of one 2-bit g16 Mixtral expert in the
    reference's unpadded single storage: 3 x 22,134,788 = 66,404,364 B."""

    def fake(n, k):
        s = n * k // 16
        return {"nbits": 2, "group_size": 16, "shape": (n, k), "quant_scale": True, "quant_zero": True,
                "W_q": np.lib.stride_tricks.as_strided(np.zeros(1, np.uint8), (n // 4, k), (0, 0)),
                "scale_q": np.lib.stride_tricks.as_strided(np.zeros(1, np.uint8), (128, s // 128), (0, 0)),
                "zero_q": np.lib.stride_tricks.as_strided(np.zeros(1, np.uint8), (1, s), (0, 0)),
                "meta_scale": {"scale": np.zeros((1, s // 128), F16), "zero": np.zeros((1, s // 128), F16)},
                "meta_zero": {"scale": np.zeros((), F16), "zero": np.zeros((), F16)}}

    # as_strided views report nbytes of the logical shape
    w1, w2, w3 = fake(14336, 4096), fake(4096, 14336), fake(14336, 4096)
    entries, total = o.slab_layout(w1, w2, w3)
    assert total == 66_404_364
    names = [e[0] for e in entries[:7]]
    assert names == ["w1.W_q", "w1.meta.meta_scale.scale", "w1.meta.meta_scale.zero", "w1.meta.meta_zero.scale",
                     "w1.meta.meta_zero.zero", "w1.meta.scale_q", "w1.meta.zero_q"]
    by = {e[0]: e for e in entries}
    assert by["w1.W_q"][2] == 14_680_064 and by["w1.meta.scale_q"][2] == 3_670_016
    assert by["w2.W_q"][1] == 22_134_788 and by["w2.W_q"][1] % 16 == 4  # why an aligned slab must pad
    assert by["w3.W_q"][1] % 16 == 8


def test_lru_hand_traces():
    m = o.LruModel(resident=[4, 5, 6, 7], offloaded=[0, 1, 2, 3])
    order, ev = m.load([5, 0])  # hit 5, miss 0 -> evicts LRU = 4
    assert order == [5, 0] and ev == [(0, 4)]
    assert list(m.main) == [6, 7, 5, 0] and (m.hits, m.misses) == (1, 1)
    order, ev = m.load([1, 6])  # resident first: 6 then 1; 6 was LRU but is refreshed before the eviction
    assert order == [6, 1] and ev == [(1, 7)]
    assert list(m.main) == [5, 0, 6, 1]
    order, ev = m.load([2, 3])  # two misses evict 5 then 0
    assert ev == [(2, 5), (3, 0)] and list(m.main) == [6, 1, 2, 3]
    assert (m.hits, m.misses) == (2, 4)
