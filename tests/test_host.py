"""CPU-side tests: the C ABI library loads and exports every symbol the header declares, the host-only LRU policy
agrees with the oracle model, and the torch restatement of the reference's PyTorch path agrees with the numpy oracle.
No GPU compute is called here."""
import ctypes
import os
import re

import numpy as np
import pytest
import torch

from oracle import hqq_oracle as o
from oracle import torch_path as tp

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_library_exports_every_declared_symbol():
    from mixtral_offloading_amd import _lib
    header = open(os.path.join(ROOT, "include", "hqq_mi355x.h")).read()
    header = re.sub(r"/\*.*?\*/", "", header, flags=re.S)
    declared = set(re.findall(r"\b(hqq_[a-z0-9_]+)\s*\(", header))
    assert len(declared) >= 25
    for name in sorted(declared):
        assert hasattr(_lib.lib, name), f"{name} is declared in include/hqq_mi355x.h but not exported"
    assert declared == set(_lib.EXPORTED), (declared ^ set(_lib.EXPORTED))
    assert _lib.lib.hqq_abi_version() == 1
    assert b"NULL" in _lib.lib.hqq_error_string(-1)


def test_argument_errors_without_touching_the_gpu():
    from mixtral_offloading_amd import _lib
    lin = _lib.HqqLinear()
    assert _lib.lib.hqq_dequantize(ctypes.byref(lin), None, None) == -1  # NULL codes
    lin.codes = 1 << 20
    lin.nbits = 5
    assert _lib.lib.hqq_matmul_kernel_family(ctypes.byref(lin), 1) == -2  # nbits
    lin.nbits, lin.N, lin.K, lin.group_size = 4, 100, 64, 64
    assert _lib.lib.hqq_matmul_kernel_family(ctypes.byref(lin), 1) == -3  # N % group_size
    assert _lib.lib.hqq_pack_4bit_u8(1 << 20, 3, 4, 1 << 21, None) == -3  # odd height (reference src/packing.py:12)
    assert _lib.lib.hqq_pack_4bit_u8(None, 2, 4, 1 << 21, None) == -1
    assert _lib.lib.hqq_pack_4bit_u8(None, 0, 4, None, None) == 0  # empty input, even without addresses
    # the decode-step entry points refuse bad arguments before any launch
    lib = _lib.lib
    assert lib.hqq_matmul_group(None, 3, 1 << 20, None, None, 0, None) == -1
    ok = _lib.HqqLinear()
    ok.nbits, ok.group_size, ok.N, ok.K, ok.codes = 4, 64, 256, 512, 1 << 20
    ok.scale.data = ok.zero.data = 1 << 21
    ptrs = (ctypes.POINTER(_lib.HqqLinear) * 1)(ctypes.pointer(ok))
    ys = (ctypes.c_void_p * 1)(1 << 22)
    assert lib.hqq_matmul_group(ptrs, 0, 1 << 20, ys, None, 0, None) == -3  # count out of 1..4
    assert lib.hqq_matmul_group(ptrs, 5, 1 << 20, ys, None, 0, None) == -3
    assert lib.hqq_matmul_group_workspace_bytes(ptrs, 5) == 0
    assert lib.hqq_matmul_group(ptrs, 1, 1 << 20, ys, None, 0, None) == -5  # no workspace
    assert lib.hqq_expert_pair_ffn_indexed(ctypes.byref(ok), ctypes.byref(ok), ctypes.byref(ok), None, None, None, None,
                                           None, 0, None, 0, None) == -3  # w2 must map ffn -> hidden
    other = _lib.HqqLinear()
    other.nbits, other.group_size, other.N, other.K, other.codes = 4, 64, 512, 512, 1 << 20
    other.scale.data = other.zero.data = 1 << 21
    assert lib.hqq_gate_up(ctypes.byref(ok), ctypes.byref(other), 1 << 20, 1, 1 << 22, 1 << 23, 1 << 20, None) == -3
    assert lib.hqq_gate_up_workspace_bytes(ctypes.byref(ok), ctypes.byref(other), 1) == 0
    assert lib.hqq_gate_up(ctypes.byref(ok), ctypes.byref(ok), None, 1, 1 << 22, 1 << 23, 1 << 20, None) == -1
    assert lib.hqq_gate_up(ctypes.byref(ok), ctypes.byref(ok), None, 0, None, None, 0, None) == 0  # empty batch
    assert lib.hqq_gate_up(ctypes.byref(ok), ctypes.byref(ok), 1 << 20, 1, 1 << 22, None, 0, None) == -5  # no workspace
    assert lib.hqq_gate_up_workspace_bytes(ctypes.byref(ok), ctypes.byref(ok), 3) > 0
    assert lib.hqq_add_rmsnorm_router(None, None, None, 1e-5, None, 4096, None, 8, None, None, None, None) == -1
    assert lib.hqq_add_rmsnorm_router(1 << 20, None, 1 << 21, 1e-5, 1 << 22, 4096, 1 << 23, 17, 1 << 24, 1 << 25, None,
                                      None) == -3  # more than 16 experts


def test_kernel_family_by_batch_size_is_host_logic():
    """Which family a call would use is decided on the host from the descriptor alone (fake, aligned addresses): the
    decode kernels up to 16 rows, the tile kernel above, de-quantise + library GEMM from a few hundred rows on, and
    the workspace query grows by the fp16 weights exactly there."""
    from mixtral_offloading_amd import _lib
    lib = _lib.lib

    def layer(nbits, n, k, gs):
        lin = _lib.HqqLinear()
        lin.nbits, lin.group_size, lin.N, lin.K, lin.codes = nbits, gs, n, k, 1 << 30
        g = n // gs
        for t, at in ((lin.scale, 2 << 30), (lin.zero, 3 << 30)):
            t.data, t.kind = at, _lib.HQQ_TABLE_U8
        lin.scale.meta_cols, lin.scale.meta_scale, lin.scale.meta_zero = g * k // 128, 4 << 30, 5 << 30
        lin.zero.meta_cols, lin.zero.meta_scale, lin.zero.meta_zero = 1, 6 << 30, 7 << 30
        return lin

    def fam(lin, m):
        return lib.hqq_matmul_kernel_family(ctypes.byref(lin), m)

    up, down, q, up3 = layer(2, 14336, 4096, 16), layer(2, 4096, 14336, 16), layer(4, 4096, 4096, 64), layer(3, 14336, 4096, 64)
    for lin in (up, down, q):
        assert [fam(lin, m) for m in (1, 2, 3, 16)] == [_lib.FAM_SMALLBATCH] * 4
        assert [fam(lin, m) for m in (17, 128, 512)] == [_lib.FAM_TILE] * 3
        assert fam(lin, 4096) == _lib.FAM_DQGEMM
    assert [fam(up, 639), fam(up, 640)] == [_lib.FAM_TILE, _lib.FAM_DQGEMM]
    assert [fam(down, 1279), fam(down, 1280)] == [_lib.FAM_TILE, _lib.FAM_DQGEMM]
    assert [fam(up3, m) for m in (1, 4, 8, 9, 16, 128, 319, 320)] == [_lib.FAM_VEC3, _lib.FAM_VEC3, _lib.FAM_VEC3, _lib.FAM_LDS,
                                                                      _lib.FAM_LDS, _lib.FAM_TILE, _lib.FAM_TILE,
                                                                      _lib.FAM_DQGEMM]
    small = layer(4, 1024, 1024, 64)  # a million weights: never worth two launches
    assert fam(small, 4096) == _lib.FAM_TILE
    fp16_weights = 2 * 14336 * 4096
    assert lib.hqq_matmul_workspace_bytes(ctypes.byref(up), 639) < fp16_weights
    assert lib.hqq_matmul_workspace_bytes(ctypes.byref(up), 640) >= fp16_weights


def _plan(lib, c, experts):
    n = len(experts)
    arr = (ctypes.c_int32 * n)(*experts)
    order, slot, victim = (ctypes.c_int32 * n)(), (ctypes.c_int32 * n)(), (ctypes.c_int32 * n)()
    rc = lib.hqq_lru_plan(c, arr, n, order, slot, victim)
    return rc, list(order), list(slot), list(victim)


def test_lru_policy_against_the_oracle_model():
    from mixtral_offloading_amd import _lib
    lib = _lib.lib
    rng = np.random.default_rng(0)
    for slots in (2, 4):
        c = lib.hqq_lru_create(8, slots)
        resident = list(range(8 - slots, 8))  # build_model keeps experts >= offload_per_layer on the device
        for e in resident:
            assert lib.hqq_lru_add_resident(c, e) >= 0
        assert lib.hqq_lru_add_resident(c, 0) == -7  # "Cache is full"
        model = o.LruModel(resident, [e for e in range(8) if e not in resident])
        slot_of = {e: lib.hqq_lru_slot_of(c, e) for e in resident}
        for _ in range(300):
            req = rng.choice(8, size=2, replace=False).tolist()
            rc, order, slot, victim = _plan(lib, c, req)
            assert rc == 0
            m_order, m_ev = model.load(req)
            assert order == m_order
            assert [(e, v) for e, v in zip(order, victim) if v >= 0] == m_ev
            for e, s, v in zip(order, slot, victim):
                if v >= 0:
                    assert slot_of.pop(v) == s  # the miss takes over its victim's slot
                    slot_of[e] = s
                else:
                    assert slot_of[e] == s
            assert sorted(slot_of) == sorted(model.main)
            assert lib.hqq_lru_hits(c) == model.hits and lib.hqq_lru_misses(c) == model.misses
        rc, *_ = _plan(lib, c, [1, 1])
        assert rc == -7  # duplicates (reference src/expert_cache.py:133)
        rc, *_ = _plan(lib, c, [9])
        assert rc == -7  # unknown expert
        lib.hqq_lru_destroy(c)


def test_lru_hand_trace_through_the_c_abi():
    from mixtral_offloading_amd import _lib
    lib = _lib.lib
    c = lib.hqq_lru_create(8, 4)
    for e in (4, 5, 6, 7):
        lib.hqq_lru_add_resident(c, e)
    assert _plan(lib, c, [5, 0])[1:] == ([5, 0], [1, 0], [-1, 4])
    assert _plan(lib, c, [1, 6])[1:] == ([6, 1], [2, 3], [-1, 7])
    assert _plan(lib, c, [2, 3])[1:] == ([2, 3], [1, 0], [5, 0])
    assert (lib.hqq_lru_hits(c), lib.hqq_lru_misses(c)) == (2, 4)
    lib.hqq_lru_destroy(c)


@pytest.mark.parametrize("nbits,n,k,gs,mgs", [(4, 64, 32, 16, 8), (2, 64, 32, 16, 8), (3, 40, 16, 8, 16)])
def test_torch_path_matches_numpy_oracle(nbits, n, k, gs, mgs):
    rng = np.random.default_rng(nbits)
    layer, _ = o.random_layer(rng, n, k, nbits, gs, meta_group_size=mgs)
    tl = tp.layer_from_numpy(layer)
    w = tp.dequantize(tl).numpy()
    np.testing.assert_array_equal(w.view(np.uint16), o.dequantize(layer).view(np.uint16))
    x = rng.standard_normal((3, k)).astype(np.float16)
    y = tp.forward(torch.from_numpy(x), tl).numpy().astype(np.float64)
    ref = o.matmul_transpose(x, layer).astype(np.float64)
    assert np.abs(y - ref).max() <= 1e-2 * np.abs(ref).max() + 1e-3


def test_torch_path_random_layer_is_in_kernel_layout():
    g = torch.Generator().manual_seed(0)
    for nbits, n in ((2, 32), (4, 32), (3, 24)):
        layer = tp.random_layer(g, n, 128, nbits, 8, 8)
        u = tp.unpack(layer["W_q"], nbits)[:n]
        assert int(u.max()) < 2 ** nbits
        np.testing.assert_array_equal(o.PACK[nbits](u.numpy()), layer["W_q"].numpy())
