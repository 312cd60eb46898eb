"""ctypes binding of ``libhqq_mi355x.so`` (declarations in ``include/hqq_mi355x.h``).

PyTorch is used for device memory and streams only: tensors reach the library
as raw ``data_ptr()`` values plus the ``hipStream_t`` of the current stream."""
from __future__ import annotations

import ctypes
import os
from ctypes import c_char_p, c_int, c_int32, c_int64, c_size_t, c_void_p

_PKG = os.path.dirname(os.path.abspath(__file__))
# HQQ_MI355X_LIB names another build of the library (a profiling or debug build); the default is the in-tree one
LIB_PATH = os.environ.get("HQQ_MI355X_LIB") or os.path.join(os.path.dirname(_PKG), "lib", "libhqq_mi355x.so")

if not os.path.exists(LIB_PATH):
    raise ImportError(
        f"{LIB_PATH} is missing: build it with `make -C mixtral-offloading_amd/csrc` "
        "(or __graft_entry__.build()).  There is no fallback path.")

lib = ctypes.CDLL(LIB_PATH)

HQQ_TABLE_F16, HQQ_TABLE_U8 = 0, 1
FAM_GENERAL, FAM_SMALLBATCH, FAM_TILE, FAM_VEC3, FAM_LDS, FAM_DQGEMM = 0, 1, 2, 3, 4, 5
HQQ_E_UNSUPPORTED = -6  # the library does not take the configuration (include/hqq_mi355x.h)


class HqqTable(ctypes.Structure):
    _fields_ = [("data", c_void_p), ("meta_scale", c_void_p), ("meta_zero", c_void_p),
                ("meta_cols", c_int64), ("kind", c_int32), ("reserved", c_int32)]


class HqqLinear(ctypes.Structure):
    _fields_ = [("nbits", c_int32), ("group_size", c_int32), ("N", c_int64), ("K", c_int64),
                ("codes", c_void_p), ("scale", HqqTable), ("zero", HqqTable), ("bias", c_void_p)]


_P = ctypes.POINTER
_SIGNATURES = {
    "hqq_abi_version": (c_int, []),
    "hqq_error_string": (c_char_p, [c_int]),
    "hqq_pack_4bit_u8": (c_int, [c_void_p, c_int64, c_int64, c_void_p, c_void_p]),
    "hqq_pack_2bit_u8": (c_int, [c_void_p, c_int64, c_int64, c_void_p, c_void_p]),
    "hqq_pack_3bit_i32": (c_int, [c_void_p, c_int64, c_int64, c_void_p, c_void_p]),
    "hqq_unpack_4bit_u8": (c_int, [c_void_p, c_int64, c_int64, c_void_p, c_void_p]),
    "hqq_unpack_2bit_u8": (c_int, [c_void_p, c_int64, c_int64, c_void_p, c_void_p]),
    "hqq_unpack_3bit_i32": (c_int, [c_void_p, c_int64, c_int64, c_void_p, c_void_p]),
    "hqq_table_to_f16": (c_int, [_P(HqqTable), c_int64, c_void_p, c_void_p]),
    "hqq_dequantize": (c_int, [_P(HqqLinear), c_void_p, c_void_p]),
    "hqq_matmul_workspace_bytes": (c_size_t, [_P(HqqLinear), c_int64]),
    "hqq_workspace_init": (c_int, [c_void_p, c_size_t, c_void_p]),
    "hqq_matmul_transpose": (c_int, [_P(HqqLinear), c_void_p, c_int64, c_void_p, c_void_p, c_size_t, c_void_p]),
    "hqq_matmul_transpose_ex": (c_int, [_P(HqqLinear), c_void_p, c_int64, c_void_p, c_void_p, c_size_t, c_int, c_void_p]),
    "hqq_matmul_kernel_family": (c_int, [_P(HqqLinear), c_int64]),
    "hqq_expert_ffn_workspace_bytes": (c_size_t, [_P(HqqLinear), _P(HqqLinear), _P(HqqLinear), c_int64]),
    "hqq_expert_ffn": (c_int, [_P(HqqLinear), _P(HqqLinear), _P(HqqLinear), c_void_p, c_int64, c_void_p, c_void_p,
                               c_int, c_void_p, c_size_t, c_void_p]),
    "hqq_expert_ffn_static": (c_int, [_P(HqqLinear), _P(HqqLinear), _P(HqqLinear), c_void_p, c_int64, c_void_p, c_void_p,
                                      c_int, c_void_p]),
    "hqq_expert_groups_ffn_workspace_bytes": (c_size_t, [c_void_p, c_void_p, c_void_p, c_int, c_void_p]),
    "hqq_expert_groups_ffn": (c_int, [c_void_p, c_void_p, c_void_p, c_int, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p,
                                      c_size_t, c_void_p]),
    "hqq_moe_group_pairs": (c_int, [c_void_p, c_void_p, c_int64, c_int, c_void_p, c_void_p, c_void_p, c_void_p]),
    "hqq_gate_up_workspace_bytes": (c_size_t, [_P(HqqLinear), _P(HqqLinear), c_int64]),
    "hqq_gate_up": (c_int, [_P(HqqLinear), _P(HqqLinear), c_void_p, c_int64, c_void_p, c_void_p, c_size_t, c_void_p]),
    "hqq_expert_record_bytes": (c_size_t, []),
    "hqq_expert_record_fill": (c_int, [_P(HqqLinear), c_void_p]),
    "hqq_expert_ffn_indexed": (c_int, [_P(HqqLinear), _P(HqqLinear), _P(HqqLinear), c_void_p, c_void_p, c_void_p, c_int64,
                                       c_void_p, c_void_p, c_int, c_void_p, c_size_t, c_void_p]),
    "hqq_expert_pair_ffn_workspace_bytes": (c_size_t, [_P(HqqLinear), _P(HqqLinear), _P(HqqLinear)]),
    "hqq_expert_pair_ffn_indexed": (c_int, [_P(HqqLinear), _P(HqqLinear), _P(HqqLinear), c_void_p, c_void_p, c_void_p,
                                            c_void_p, c_void_p, c_int, c_void_p, c_size_t, c_void_p]),
    "hqq_moe_pair_routed": (c_int, [_P(HqqLinear), _P(HqqLinear), _P(HqqLinear), c_void_p, c_void_p, c_void_p, c_void_p,
                                    ctypes.c_float, c_void_p, c_void_p, c_int32, c_void_p, c_void_p, c_void_p, c_int,
                                    c_void_p, c_size_t, c_void_p]),
    "hqq_matmul_group_workspace_bytes": (c_size_t, [_P(_P(HqqLinear)), c_int32]),
    "hqq_matmul_group": (c_int, [_P(_P(HqqLinear)), c_int32, c_void_p, _P(c_void_p), c_void_p, c_size_t, c_void_p]),
    "hqq_matmul_group_norm": (c_int, [_P(_P(HqqLinear)), c_int32, c_void_p, c_void_p, c_void_p, ctypes.c_float, c_void_p,
                                      _P(c_void_p), c_void_p, c_size_t, c_void_p]),
    "hqq_router_top2": (c_int, [c_void_p, c_void_p, c_int32, c_int64, c_void_p, c_void_p, c_void_p, c_void_p]),
    "hqq_add_rmsnorm": (c_int, [c_void_p, c_void_p, c_void_p, ctypes.c_float, c_void_p, c_int64, c_void_p]),
    "hqq_add_rmsnorm_rows": (c_int, [c_void_p, c_void_p, c_void_p, ctypes.c_float, c_void_p, c_int64, c_int64, c_void_p]),
    "hqq_router_top2_rows": (c_int, [c_void_p, c_void_p, c_int32, c_int64, c_int64, c_void_p, c_void_p, c_void_p, c_void_p]),
    "hqq_rope_append_rows": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int64, c_int64, c_void_p, c_void_p,
                                     c_int64, c_int32, c_int32, c_int32, c_void_p]),
    "hqq_add_rmsnorm_router": (c_int, [c_void_p, c_void_p, c_void_p, ctypes.c_float, c_void_p, c_int64, c_void_p, c_int32,
                                       c_void_p, c_void_p, c_void_p, c_void_p]),
    "hqq_attention_decode": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p,
                                     c_int64, c_int32, c_int32, c_int32, c_void_p, c_void_p]),
    "hqq_attention_chain_workspace_bytes": (c_size_t, []),
    "hqq_attention_chain_error_offset": (c_size_t, []),
    "hqq_attention_chain": (c_int, [_P(HqqLinear)] * 4 + [c_void_p, c_void_p, c_void_p, ctypes.c_float] + [c_void_p] * 5
                            + [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int64, c_int32, c_int32, c_int32, c_void_p,
                               c_void_p, c_size_t, c_void_p]),
    "hqq_quantize_workspace_bytes": (c_size_t, []),
    "hqq_quantize_groups": (c_int, [c_void_p, c_int32, c_int64, c_int64, c_int32, c_int32, c_int32, ctypes.c_float,
                                    ctypes.c_double, ctypes.c_double, c_void_p, c_void_p, c_void_p, c_void_p, c_size_t, c_void_p]),
    "hqq_quantize_whole": (c_int, [c_void_p, c_int64, c_int32, c_void_p, c_void_p, c_void_p, c_void_p, c_size_t, c_void_p]),
    "hqq_attention_decode_workspace_bytes": (c_size_t, [c_int64, c_int32, c_int32]),
    "hqq_attention_decode_ws": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p,
                                        c_int64, c_int32, c_int32, c_int32, c_void_p, c_void_p, c_size_t, c_void_p]),
    "hqq_slab_h2d_async": (c_int, [c_void_p, c_void_p, c_size_t, c_void_p, c_void_p]),
    "hqq_stream_wait_event": (c_int, [c_void_p, c_void_p]),
    "hqq_lru_create": (c_void_p, [c_int32, c_int32]),
    "hqq_lru_destroy": (None, [c_void_p]),
    "hqq_lru_add_resident": (c_int, [c_void_p, c_int32]),
    "hqq_lru_plan": (c_int, [c_void_p, _P(c_int32), c_int32, _P(c_int32), _P(c_int32), _P(c_int32)]),
    "hqq_lru_plan_guess": (c_int, [c_void_p, _P(c_int32), c_int32, _P(c_int32), c_int32, _P(c_int32), _P(c_int32), _P(c_int32),
                                   _P(c_int32)]),
    "hqq_lru_hits": (c_int64, [c_void_p]),
    "hqq_lru_misses": (c_int64, [c_void_p]),
    "hqq_lru_slot_of": (c_int, [c_void_p, c_int32]),
}

for _name, (_res, _args) in _SIGNATURES.items():
    _fn = getattr(lib, _name)  # AttributeError here = the library does not export what the header declares
    _fn.restype = _res
    _fn.argtypes = _args

EXPORTED = tuple(_SIGNATURES)


class HqqError(RuntimeError):
    def __init__(self, code: int, where: str):
        self.code = code
        super().__init__(f"{where}: {lib.hqq_error_string(code).decode()} (code {code})")


def check(code: int, where: str) -> None:
    if code != 0:
        # the reference reports argument problems as AssertionError (src/triton_kernels.py:150-153)
        if code in (-3,):
            raise AssertionError(f"{where}: sizes disagree")
        raise HqqError(code, where)


def current_stream_ptr(device=None) -> int:
    import torch

    return torch.cuda.current_stream(device).cuda_stream
