"""CPU tests of the quantise side (mixtral_offloading_amd.hqq_core, the stand-in for the absent hqq package; reference
call sites src/custom_layers.py:35-39, src/build_model.py:108-120) and of the step layout -> kernel layout conversion
at load (src/custom_layers.py:41-47, src/packing.py:29-33).

hqq's numerics are not available to compare with (parity unpinned), so the quantiser is held to what the mathematics
fixes: every code is the nearest level for the (scale, zero) it reports, the group minimum and maximum land on the
end levels when no refinement runs, and the reconstruction error is at most half a step.  The layout conversion is
checked against hand-computed known answers."""
import json
import os

import numpy as np
import pytest
import torch

from mixtral_offloading_amd.hqq_core import BaseQuantizeConfig, BitPack, Quantizer
from oracle import hqq_oracle as o

HERE = os.path.dirname(os.path.abspath(__file__))
STEP_UNPACK = {4: BitPack.unpack_4bit_u8, 2: BitPack.unpack_2bit_u8, 3: BitPack.unpack_3bit_32}
STEP_PACK = {4: BitPack.pack_4bit_u8, 2: BitPack.pack_2bit_u8, 3: BitPack.pack_3bit_32}


def _octal(rows):
    return np.array([[int(w, 8) for w in row] for row in rows], dtype=np.int64).astype(np.int32)


def step_cases():
    with open(os.path.join(HERE, "golden", "step_layout_known_answers.json")) as f:
        cases = json.load(f)["cases"]
    for c in cases:
        if c["nbits"] == 3:
            c["step_packed"], c["kernel_packed"] = _octal(c["step_packed_octal"]), _octal(c["kernel_packed_octal"])
        else:
            c["step_packed"] = np.array(c["step_packed"], dtype=np.uint8)
            c["kernel_packed"] = np.array(c["kernel_packed"], dtype=np.uint8)
    return cases


@pytest.mark.parametrize("case", step_cases(), ids=lambda c: "w%d_%dx%d" % (c["nbits"], c["shape"][0], c["shape"][1]))
def test_step_layout_to_kernel_layout_known_answers(case):
    nbits, (n, k), gs = case["nbits"], case["shape"], case["group_size"]
    codes = np.array(case["codes"], dtype=np.uint8)
    quant = np.array(case["quant_layout"], dtype=np.uint8)
    # the file is consistent with itself: the quantiser's view is a reshape, the kernel layout is the reference packer's
    np.testing.assert_array_equal(codes.reshape(gs, -1), quant)
    np.testing.assert_array_equal(o.PACK[nbits](codes), case["kernel_packed"])
    # the stand-in's step packer writes the recalled layout, and its unpacker inverts it (spare 3-bit rows are zero)
    packed = STEP_PACK[nbits](torch.from_numpy(quant))
    np.testing.assert_array_equal(packed.numpy(), case["step_packed"])
    unpacked = STEP_UNPACK[nbits](torch.from_numpy(case["step_packed"])).numpy()
    np.testing.assert_array_equal(unpacked[:gs], quant)
    assert not unpacked[gs:].any()
    # the conversion of the load path (oracle restatement of src/custom_layers.py:41-47)
    np.testing.assert_array_equal(o.repack(unpacked, (n, k), nbits), case["kernel_packed"])


@pytest.mark.parametrize("nbits,gs", [(2, 16), (3, 64), (4, 64), (8, 128)])
@pytest.mark.parametrize("round_zero", [False, True])
def test_quantizer_codes_are_the_nearest_levels(nbits, gs, round_zero):
    g = torch.Generator().manual_seed(nbits * 100 + gs)
    w = torch.randn((256, 96), generator=g) * 0.02
    w_q, meta = Quantizer.quantize(w, nbits=nbits, group_size=gs, optimize=False, round_zero=round_zero, bitpack=False)
    top = 2 ** nbits - 1
    q = w_q.float().reshape(gs, -1)
    wg = w.float().reshape(gs, -1)
    scale, zero = meta["scale"].float(), meta["zero"].float()  # dequant: (q - zero) * scale
    assert q.min() >= 0 and q.max() <= top and torch.equal(q, q.round())
    # nearest level: no other code reconstructs the weight better
    recon = (q - zero) * scale
    for other in (q - 1, q + 1):
        alt = (other.clamp(0, top) - zero) * scale
        assert bool(((recon - wg).abs() <= (alt - wg).abs() + 1e-7).all())
    step = scale.abs()
    if not round_zero:
        # the group minimum and maximum sit on the end levels, and the error is at most half a step
        assert bool((q.min(dim=0).values == 0).all()) and bool((q.max(dim=0).values == top).all())
        assert bool(((recon - wg).abs() <= 0.5 * step * (1 + 1e-4) + 1e-8).all())
    else:
        # a rounded zero point shifts the grid by at most half a step: end codes may clip, by less than one step
        assert bool(((recon - wg).abs() <= 1.0 * step * (1 + 1e-4) + 1e-8).all())
    # one step is the group's range over the number of levels
    rng = wg.max(dim=0).values - wg.min(dim=0).values
    assert torch.allclose(step.reshape(-1), rng / top, rtol=1e-4, atol=1e-9)


def test_quantizer_refinement_does_not_make_the_fit_worse():
    g = torch.Generator().manual_seed(5)
    w = torch.randn((512, 64), generator=g) * 0.02
    errs = {}
    for optimize in (False, True):
        w_q, meta = Quantizer.quantize(w, nbits=2, group_size=16, optimize=optimize, bitpack=False)
        recon = ((w_q.float().reshape(16, -1) - meta["zero"].float()) * meta["scale"].float()).reshape(w.shape)
        errs[optimize] = float((recon - w).abs().pow(0.7).mean())
    assert errs[True] <= errs[False] * 1.02  # the lp(0.7) error it minimises


@pytest.mark.parametrize("nbits,gs", [(2, 16), (3, 64), (4, 64)])
def test_whole_tensor_meta_and_packing_round_trip(nbits, gs):
    """What HQQLinear.quantize stores: packed codes (step layout) plus 8-bit meta-quantised tables whose
    de-quantisation is within half a meta step of the fp tables."""
    cfg = BaseQuantizeConfig(nbits=nbits, group_size=gs, quant_zero=True, quant_scale=True)
    g = torch.Generator().manual_seed(nbits)
    w = torch.randn((640, 128), generator=g) * 0.02
    # the step packers are named directly: other tests install the interleaved GPU packers in Quantizer's registry
    plain_q, meta = Quantizer.quantize(w, **{**cfg["weight_quant_params"], "optimize": False, "bitpack": False})
    w_q = STEP_PACK[nbits](plain_q)
    codes = STEP_UNPACK[nbits](w_q)[:gs]
    plain, _ = Quantizer.quantize(w, **{**cfg["weight_quant_params"], "optimize": False, "bitpack": False})
    assert torch.equal(codes.float(), plain.float().reshape(gs, -1))
    for key, params in (("scale", cfg["scale_quant_params"]), ("zero", cfg["zero_quant_params"])):
        t = meta[key]
        t_q, t_meta = Quantizer.quantize(t, **{**params, "bitpack": False})
        back = ((t_q.float() - t_meta["zero"].float()) * t_meta["scale"].float()).reshape(t.shape)
        step = t_meta["scale"].float().abs().max()
        assert float((back - t.float()).abs().max()) <= 0.5 * float(step) * 1.01 + 2e-3 * float(t.float().abs().max())
