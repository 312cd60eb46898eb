"""GPU parity of the bit packers (C ABI hqq_pack_* / hqq_unpack_*) against the
oracle: bit-exact, including ragged widths, the 3-bit tail and empty inputs."""
import numpy as np
import pytest
import torch

from oracle import hqq_oracle as o

pytestmark = pytest.mark.gpu


def _mods():
    from mixtral_offloading_amd import packing
    return packing


@pytest.mark.parametrize("nbits,h,w", [(4, 2, 1), (4, 64, 16), (4, 128, 4096), (4, 6, 37), (2, 4, 1), (2, 64, 48),
                                       (2, 256, 4096), (2, 12, 19), (3, 1, 1), (3, 10, 4), (3, 37, 16), (3, 64, 3),
                                       (3, 4096, 256), (3, 25, 4096)])
def test_pack_unpack_bit_exact(nbits, h, w):
    packing = _mods()
    rng = np.random.default_rng(nbits * 1000 + h + w)
    q = rng.integers(0, 2 ** nbits, size=(h, w), dtype=np.uint8)
    pack = {4: packing.pack_4bit_u8_common, 2: packing.pack_2bit_u8_common, 3: packing.pack_3bit_i32_common}[nbits]
    unpack = {4: packing.unpack_4bit_u8_common, 2: packing.unpack_2bit_u8_common,
              3: packing.unpack_3bit_i32_common}[nbits]
    p = pack(torch.from_numpy(q).cuda())
    assert isinstance(p, packing.PackedTensor)
    want = o.PACK[nbits](q)
    assert tuple(p.shape) == want.shape and p.dtype == torch.from_numpy(want).dtype
    np.testing.assert_array_equal(p.cpu().numpy(), want)
    u = unpack(p)
    np.testing.assert_array_equal(u.cpu().numpy(), o.UNPACK[nbits](want))
    assert u.dtype == torch.uint8


def test_unpack_every_packed_value():
    packing = _mods()
    b = np.arange(256, dtype=np.uint8).reshape(16, 16)
    np.testing.assert_array_equal(packing.unpack_4bit_u8_common(packing.PackedTensor(torch.from_numpy(b).cuda())).cpu().numpy(),
                                  o.unpack_4bit_u8(b))
    np.testing.assert_array_equal(packing.unpack_2bit_u8_common(packing.PackedTensor(torch.from_numpy(b).cuda())).cpu().numpy(),
                                  o.unpack_2bit_u8(b))
    rng = np.random.default_rng(0)
    w = rng.integers(0, 2 ** 30, size=(33, 20), dtype=np.int64).astype(np.int32)
    np.testing.assert_array_equal(packing.unpack_3bit_i32_common(torch.from_numpy(w).cuda()).cpu().numpy(),
                                  o.unpack_3bit_i32(w))


def test_pack_unmasked_like_the_reference():
    packing = _mods()
    q = np.array([[0x13, 7], [0x25, 9]], dtype=np.uint8)
    np.testing.assert_array_equal(packing.pack_4bit_u8_common(torch.from_numpy(q).cuda()).cpu().numpy(),
                                  o.pack_4bit_u8(q))
    q2 = np.array([[5], [6], [7], [0xF1]], dtype=np.uint8)
    np.testing.assert_array_equal(packing.pack_2bit_u8_common(torch.from_numpy(q2).cuda()).cpu().numpy(),
                                  o.pack_2bit_u8(q2))


def test_trailing_dims_empty_and_errors():
    packing = _mods()
    rng = np.random.default_rng(1)
    q = rng.integers(0, 16, size=(8, 3, 5), dtype=np.uint8)
    p = packing.pack_4bit_u8_common(torch.from_numpy(q).cuda())
    assert tuple(p.shape) == (4, 3, 5)
    np.testing.assert_array_equal(p.cpu().numpy(), o.pack_4bit_u8(q))
    e = packing.pack_2bit_u8_common(torch.zeros((0, 7), dtype=torch.uint8, device="cuda"))
    assert tuple(e.shape) == (0, 7)
    with pytest.raises(AssertionError):  # reference src/packing.py:12
        packing.pack_4bit_u8_common(torch.zeros((3, 2), dtype=torch.uint8, device="cuda"))
    with pytest.raises(AssertionError):  # reference src/packing.py:88
        packing.unpack_3bit_i32_common(torch.zeros((3, 2), dtype=torch.uint8, device="cuda"))
    with pytest.raises(RuntimeError):  # no CPU path
        packing.pack_4bit_u8_common(torch.zeros((2, 2), dtype=torch.uint8))


def test_universal_unpack_dispatches_on_the_tag():
    packing = _mods()
    from mixtral_offloading_amd.hqq_core import BitPack
    rng = np.random.default_rng(2)
    q = torch.from_numpy(rng.integers(0, 4, size=(16, 8), dtype=np.uint8)).cuda()
    tagged = packing.pack_2bit_u8_common(q)
    assert torch.equal(packing.unpack_2bit_u8_universal(tagged), q)
    step = BitPack.pack_2bit_u8(q)  # hqq's original layout, untagged
    assert torch.equal(packing.unpack_2bit_u8_universal(step), q)
    assert not torch.equal(step, torch.Tensor.as_subclass(tagged, torch.Tensor))


@pytest.mark.parametrize("nbits,n,k", [(2, 14336, 4096), (3, 14336, 4096), (4, 4096, 4096)])
def test_full_size_round_trip(nbits, n, k):
    """At Mixtral sizes: unpack(pack(q)) == q and a checksum of the packed words
    equals the closed form sum_i q[F*p+i] << shift_i computed with torch integer ops."""
    packing = _mods()
    g = torch.Generator(device="cuda").manual_seed(nbits)
    q = torch.randint(0, 2 ** nbits, (n, k), dtype=torch.uint8, device="cuda", generator=g)
    pack = {4: packing.pack_4bit_u8_common, 2: packing.pack_2bit_u8_common, 3: packing.pack_3bit_i32_common}[nbits]
    unpack = {4: packing.unpack_4bit_u8_common, 2: packing.unpack_2bit_u8_common,
              3: packing.unpack_3bit_i32_common}[nbits]
    p = pack(q)
    u = unpack(p)
    assert torch.equal(u[:n], q)
    assert not u[n:].any()
    f = {4: 2, 2: 4, 3: 10}[nbits]
    pad = (-n) % f
    qq = torch.cat([q, torch.zeros((pad, k), dtype=torch.uint8, device="cuda")]).to(torch.int64)
    want = torch.zeros((qq.shape[0] // f, k), dtype=torch.int64, device="cuda")
    for i in range(f):
        want += qq[i::f] << (nbits * (f - 1 - i))
    assert torch.equal(torch.Tensor.as_subclass(p, torch.Tensor).to(torch.int64), want)
