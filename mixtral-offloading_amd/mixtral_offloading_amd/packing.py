"""Bit packers of the kernel layout, run by the HIP library.

Same names and behaviour as the reference's ``src/packing.py``: codes are
interleaved along axis 0 (4 bit: two per uint8, 2 bit: four per uint8, 3 bit:
ten per int32), packed results carry the ``PackedTensor`` tag, un-tagged
inputs of the ``*_universal`` unpackers are in hqq's original step layout, and
``patch_packing()`` installs them in the ``Quantizer`` registries.

The work is done by ``hqq_pack_*`` / ``hqq_unpack_*`` of the C ABI on the
tensor's GPU; tensors that are not on a GPU are rejected (there is no CPU
path in this package)."""
from __future__ import annotations

import torch

from . import _lib
from .hqq_core import BitPack, Quantizer


class PackedTensor(torch.Tensor):
    """Type tag for codes in the interleaved kernel layout (reference
    src/packing.py:5-7)."""

    @staticmethod
    def __new__(cls, t: torch.Tensor):
        return t.detach().as_subclass(cls)

    def __init__(self, t: torch.Tensor):
        pass

    def __deepcopy__(self, memo):
        return PackedTensor(torch.Tensor.as_subclass(self, torch.Tensor).clone())

    @classmethod
    def __torch_function__(cls, func, types, args=(), kwargs=None):
        # plain tensors come out of every op; only explicit construction tags
        with torch._C.DisableTorchFunctionSubclass():
            return func(*args, **(kwargs or {}))


def _device_2d(t: torch.Tensor, what: str):
    if not t.is_cuda:
        raise RuntimeError(f"{what}: tensor is on {t.device}; the packers run on the GPU only")
    rows = t.shape[0]
    cols = 1
    for d in t.shape[1:]:
        cols *= d
    return t.contiguous(), rows, cols


def _run(fn_name, src, rows, cols, out):
    fn = getattr(_lib.lib, fn_name)
    with torch.cuda.device(src.device):
        _lib.check(fn(src.data_ptr(), rows, cols, out.data_ptr(), _lib.current_stream_ptr(src.device)), fn_name)
    return out


# 4 bit -> uint8 (reference src/packing.py:10-27)
def pack_4bit_u8_common(W_q: torch.Tensor):
    height = W_q.size(0)
    assert height % 2 == 0
    q, rows, cols = _device_2d(W_q.to(torch.uint8), "pack_4bit_u8_common")
    out = torch.empty((rows // 2,) + tuple(W_q.shape[1:]), dtype=torch.uint8, device=q.device)
    return PackedTensor(_run("hqq_pack_4bit_u8", q, rows, cols, out))


def unpack_4bit_u8_common(W_q: torch.Tensor):
    p, rows, cols = _device_2d(torch.Tensor.to(W_q, torch.uint8), "unpack_4bit_u8_common")
    out = torch.empty((2 * rows,) + tuple(W_q.shape[1:]), dtype=torch.uint8, device=p.device)
    return _run("hqq_unpack_4bit_u8", p, rows, cols, out)


def unpack_4bit_u8_universal(W_q: torch.Tensor):
    if isinstance(W_q, PackedTensor):
        return unpack_4bit_u8_common(W_q)
    return BitPack.unpack_4bit_u8(W_q)


# 2 bit -> uint8 (reference src/packing.py:36-59)
def pack_2bit_u8_common(W_q: torch.Tensor):
    assert W_q.size(0) % 4 == 0
    q, rows, cols = _device_2d(W_q.to(torch.uint8), "pack_2bit_u8_common")
    out = torch.empty((rows // 4,) + tuple(W_q.shape[1:]), dtype=torch.uint8, device=q.device)
    return PackedTensor(_run("hqq_pack_2bit_u8", q, rows, cols, out))


def unpack_2bit_u8_common(W_q: torch.Tensor):
    p, rows, cols = _device_2d(torch.Tensor.to(W_q, torch.uint8), "unpack_2bit_u8_common")
    out = torch.empty((4 * rows,) + tuple(W_q.shape[1:]), dtype=torch.uint8, device=p.device)
    return _run("hqq_unpack_2bit_u8", p, rows, cols, out)


def unpack_2bit_u8_universal(W_q: torch.Tensor):
    if isinstance(W_q, PackedTensor):
        return unpack_2bit_u8_common(W_q)
    return BitPack.unpack_2bit_u8(W_q)


# 3 bit -> int32, ten per word (reference src/packing.py:62-103)
def pack_3bit_i32_common(W_q: torch.Tensor):
    q, rows, cols = _device_2d(W_q.to(torch.uint8), "pack_3bit_i32_common")
    out = torch.empty(((rows + 9) // 10,) + tuple(W_q.shape[1:]), dtype=torch.int32, device=q.device)
    return PackedTensor(_run("hqq_pack_3bit_i32", q, rows, cols, out))


def unpack_3bit_i32_common(W_q: torch.Tensor):
    """There may be spare rows after unpacking (the height is rounded up to a multiple of 10)."""
    assert W_q.dtype == torch.int32
    p, rows, cols = _device_2d(W_q, "unpack_3bit_i32_common")
    out = torch.empty((10 * rows,) + tuple(W_q.shape[1:]), dtype=torch.uint8, device=p.device)
    return _run("hqq_unpack_3bit_i32", p, rows, cols, out)


def unpack_3bit_i32_universal(W_q: torch.Tensor):
    if isinstance(W_q, PackedTensor):
        return unpack_3bit_i32_common(W_q)
    return BitPack.unpack_3bit_32(W_q)


def patch_packing():
    Quantizer.pack["4bit_u8"] = pack_4bit_u8_common
    Quantizer.unpack["4bit_u8"] = unpack_4bit_u8_universal
    Quantizer.pack["2bit_u8"] = pack_2bit_u8_common
    Quantizer.unpack["2bit_u8"] = unpack_2bit_u8_universal
    Quantizer.pack["3bit_32"] = pack_3bit_i32_common
    Quantizer.unpack["3bit_32"] = unpack_3bit_i32_universal


patch_packing()
