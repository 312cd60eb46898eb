"""GPU parity test of HQQLinearTritonSavable.repack (reference src/custom_layers.py:41-47): codes in the quantiser's
layout, (group_size, N*K/group_size) packed in hqq's step layout, must come out in the kernel layout exactly as the
oracle's restatement gives them -- including the 3-bit case, where the step packing pads the group dimension to a
multiple of ten and `[:N]` drops the pad rows."""
import numpy as np
import pytest
import torch

from oracle import hqq_oracle as o
from test_host_quantizer import STEP_PACK, STEP_UNPACK, step_cases

pytestmark = pytest.mark.gpu


def _empty_layer(nbits, n, k, gs):
    from mixtral_offloading_amd.custom_layers import HQQLinearTritonSavable
    from mixtral_offloading_amd.hqq_core import BaseQuantizeConfig
    cfg = BaseQuantizeConfig(nbits=nbits, group_size=64, quant_zero=True, quant_scale=True)
    cfg["weight_quant_params"]["group_size"] = gs  # the hand-computed cases use groups smaller than a config allows
    return HQQLinearTritonSavable(None, cfg, meta=HQQLinearTritonSavable.get_hqq_meta((k, n), cfg))


@pytest.mark.parametrize("nbits,n,k,gs", [(4, 256, 128, 64), (2, 256, 192, 16), (3, 640, 256, 64), (3, 1280, 128, 64),
                                          (3, 448, 64, 32), (2, 14336, 256, 16), (3, 14336, 128, 64)])
def test_repack_equals_oracle(nbits, n, k, gs):
    from mixtral_offloading_amd.packing import PackedTensor
    rng = np.random.default_rng(n + k + nbits)
    codes = rng.integers(0, 2 ** nbits, size=(n, k), dtype=np.uint8)
    quant_layout = codes.reshape(gs, -1)
    step_packed = STEP_PACK[nbits](torch.from_numpy(quant_layout))  # what the quantiser / a checkpoint holds
    unpacked = STEP_UNPACK[nbits](step_packed).numpy()
    if nbits == 3:
        assert unpacked.shape[0] == 10 * ((gs + 9) // 10) > gs  # pad rows exist, so `[:N]` has something to drop
    want = o.repack(unpacked, (n, k), nbits)
    np.testing.assert_array_equal(o.UNPACK[nbits](want)[:n], codes)
    lin = _empty_layer(nbits, n, k, gs)
    lin.W_q = step_packed.to("cuda")
    assert not lin.in_kernel_layout() or tuple(step_packed.shape) == tuple(want.shape)
    lin.repack()
    assert isinstance(lin.W_q, PackedTensor) and lin.in_kernel_layout()
    got = torch.Tensor.as_subclass(lin.W_q, torch.Tensor).cpu().numpy()
    assert got.dtype == want.dtype and got.shape == want.shape
    np.testing.assert_array_equal(got, want)
    # a second repack leaves the kernel layout alone
    lin.repack()
    np.testing.assert_array_equal(torch.Tensor.as_subclass(lin.W_q, torch.Tensor).cpu().numpy(), want)


@pytest.mark.parametrize("case", step_cases(), ids=lambda c: "w%d_%dx%d" % (c["nbits"], c["shape"][0], c["shape"][1]))
def test_repack_known_answers(case):
    nbits, (n, k), gs = case["nbits"], case["shape"], case["group_size"]
    lin = _empty_layer(nbits, n, k, gs)
    lin.W_q = torch.from_numpy(case["step_packed"]).to("cuda")
    lin.repack()
    np.testing.assert_array_equal(torch.Tensor.as_subclass(lin.W_q, torch.Tensor).cpu().numpy(), case["kernel_packed"])
