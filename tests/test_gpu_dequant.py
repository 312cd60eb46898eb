"""GPU parity of hqq_table_to_f16 and hqq_dequantize: bit-exact fp16 against the oracle."""
import numpy as np
import pytest
import torch

from oracle import hqq_oracle as o
from helpers import desc_of, layer_to_device, to_dev

pytestmark = pytest.mark.gpu

CASES = [(4, 64, 32, 16, 8, True, True), (4, 128, 64, 64, 128, True, True), (4, 32, 16, 8, 8, False, False),
         (2, 64, 32, 16, 8, True, True), (2, 256, 128, 16, 128, True, False), (2, 32, 24, 8, 4, False, True),
         (3, 40, 16, 8, 16, True, True), (3, 64, 128, 64, 128, True, True), (3, 20, 7, 4, 5, False, False),
         (4, 512, 512, 64, 128, True, True), (2, 896 * 2, 256, 16, 128, True, True), (3, 224 * 2, 256, 64, 128, True, True)]


@pytest.mark.parametrize("nbits,n,k,gs,mgs,qs,qz", CASES)
def test_dequantize_bit_exact(nbits, n, k, gs, mgs, qs, qz):
    from mixtral_offloading_amd import hip_kernels
    rng = np.random.default_rng(n + k + nbits)
    layer, _ = o.random_layer(rng, n, k, nbits, gs, qs, qz, meta_group_size=mgs)
    w = hip_kernels.dequantize(desc_of(layer)).cpu().numpy()
    want = o.dequantize(layer)
    np.testing.assert_array_equal(w.view(np.uint16), want.view(np.uint16))


def test_table_to_f16_bit_exact():
    from mixtral_offloading_amd import hip_kernels
    rng = np.random.default_rng(0)
    layer, _ = o.random_layer(rng, 256, 128, 2, 16, True, True, meta_group_size=128)
    _, meta = layer_to_device(layer)
    s_cnt = 256 * 128 // 16
    got = hip_kernels.table_to_f16(meta["scale_q"], {**meta["meta_scale"], "shape": (1, s_cnt)}).cpu().numpy()
    want = o.meta_dequant(layer["scale_q"], layer["meta_scale"]["scale"], layer["meta_scale"]["zero"], (1, s_cnt))
    np.testing.assert_array_equal(got.view(np.uint16), want.view(np.uint16))
    got = hip_kernels.table_to_f16(meta["zero_q"], {**meta["meta_zero"], "shape": (1, s_cnt)}).cpu().numpy()
    want = o.meta_dequant(layer["zero_q"], layer["meta_zero"]["scale"], layer["meta_zero"]["zero"], (1, s_cnt))
    np.testing.assert_array_equal(got.view(np.uint16), want.view(np.uint16))
    # every 8-bit code with awkward meta values (two roundings matter here)
    q = np.arange(256, dtype=np.uint8).reshape(1, 256)
    ms, mz = np.float16(0.0123), np.float16(101.3)
    got = hip_kernels.table_to_f16(to_dev(q), {"scale": to_dev(np.array([ms])), "zero": to_dev(np.array([mz])),
                                               "shape": (1, 256)}).cpu().numpy()
    np.testing.assert_array_equal(got.view(np.uint16), o.meta_dequant(q, ms, mz, (1, 256)).view(np.uint16))


@pytest.mark.parametrize("nbits,n,k,gs", [(4, 4096, 4096, 64), (2, 14336, 4096, 16), (3, 4096, 14336, 64)])
def test_full_size_dequantize_matches_torch_restatement(nbits, n, k, gs):
    """At Mixtral sizes the numpy oracle is slow, so compare with the same two-rounding formula written
    with torch half ops on the GPU (each op rounds once, like the reference's dequantize())."""
    from mixtral_offloading_amd import hip_kernels, packing
    g = torch.Generator(device="cuda").manual_seed(n + nbits)
    G = n // gs
    q = torch.randint(0, 2 ** nbits, (n, k), dtype=torch.uint8, device="cuda", generator=g)
    s_cnt = G * k
    scale_q = torch.randint(0, 256, (128, s_cnt // 128), dtype=torch.uint8, device="cuda", generator=g)
    zero_q = torch.randint(0, 256, (1, s_cnt), dtype=torch.uint8, device="cuda", generator=g)
    ms = (torch.rand((1, s_cnt // 128), device="cuda", generator=g) * 1e-3).half()
    mz = (torch.rand((1, s_cnt // 128), device="cuda", generator=g) * 50).half()
    zs, zz = torch.tensor([0.012], device="cuda").half(), torch.tensor([3.3], device="cuda").half()
    pack = {4: packing.pack_4bit_u8_common, 2: packing.pack_2bit_u8_common, 3: packing.pack_3bit_i32_common}[nbits]
    meta = {"nbits": nbits, "group_size": gs, "shape": (n, k), "quant_scale": True, "quant_zero": True,
            "scale_q": scale_q, "meta_scale": {"scale": ms, "zero": mz}, "zero_q": zero_q,
            "meta_zero": {"scale": zs, "zero": zz}}
    w = hip_kernels.dequantize(hip_kernels.LinearDesc(pack(q), meta))
    scale = ((scale_q.half() - mz) * ms).reshape(1, -1)
    zero = ((zero_q.half() - zz) * zs).reshape(1, -1)
    want = ((q.half().reshape(gs, -1) - zero) * scale).reshape(n, k)
    assert torch.equal(w.view(torch.int16), want.view(torch.int16))
