"""The library's quantiser (hqq_quantize_groups / hqq_quantize_whole) against the oracle's restatement of hqq's
Quantizer.quantize.  Without the solver every output is a single correctly rounded fp32 operation of its inputs, so
codes, scale and zero must agree bit for bit; with the solver the shrinkage uses a power function whose last bit is
the library's own, so agreement is asked for up to a handful of codes on a rounding boundary.  (Both restate hqq from
memory: what is pinned here is that the GPU kernel and the CPU restatement are the same function, and, below, what the
mathematics fixes.)"""
import numpy as np
import pytest
import torch

from oracle import hqq_oracle as o

pytestmark = pytest.mark.gpu


def _weights(rng, n, k, dtype):
    w = (rng.standard_normal((n, k)) * 0.02).astype(np.float32)
    w[rng.integers(0, n, 8), rng.integers(0, k, 8)] *= 30.0  # a few outliers, as real weights have
    return w.astype(dtype)


@pytest.mark.parametrize("nbits,gs,round_zero", [(2, 16, False), (3, 64, False), (4, 64, True), (8, 128, False), (4, 32, False),
                                                 (2, 8, False)])
@pytest.mark.parametrize("dtype", [np.float16, np.float32])
def test_min_max_quantiser_equals_the_oracle_bit_for_bit(nbits, gs, round_zero, dtype):
    from mixtral_offloading_amd import hip_kernels
    rng = np.random.default_rng(nbits * 100 + gs)
    w = _weights(rng, 384, 320, dtype)
    q, scale, zero = o.hqq_quantize_tensor(w, nbits, gs, round_zero=round_zero)
    gq, gscale, gzero = hip_kernels.quantize_groups(torch.from_numpy(w).cuda(), gs, nbits, round_zero=round_zero)
    assert np.array_equal(gq.cpu().numpy(), q)
    assert np.array_equal(gscale.cpu().numpy().view(np.uint32), scale.reshape(1, -1).view(np.uint32))
    assert np.array_equal(gzero.cpu().numpy().view(np.uint32), zero.reshape(1, -1).view(np.uint32))


@pytest.mark.parametrize("gs,cols,off", [(16, 1613, 0), (32, 2047, 1), (64, 999, 2), (128, 2272, 3), (8, 1, 0), (16, 6, 1)])
def test_ragged_column_counts_and_unaligned_starts(gs, cols, off):
    """Column counts that are no multiple of the groups a thread takes, and tensors that start at any element of an
    allocation: the kernel falls back to narrower accesses and the result is the same."""
    from mixtral_offloading_amd import hip_kernels
    rng = np.random.default_rng(gs + cols)
    for dtype in (np.float16, np.float32):
        w = rng.standard_normal(gs * cols + off).astype(dtype)
        q, scale, zero = o.hqq_quantize_tensor(w[off:].reshape(gs, cols), 4, gs, round_zero=True)
        gq, gscale, gzero = hip_kernels.quantize_groups(torch.from_numpy(w).cuda()[off:], gs, 4, round_zero=True)
        assert np.array_equal(gq.cpu().numpy(), q)
        assert np.array_equal(gscale.cpu().numpy(), scale.reshape(1, -1)) and np.array_equal(gzero.cpu().numpy(), zero.reshape(1, -1))


def test_constant_and_tiny_groups():
    """max = min gives an infinite quotient that hqq clamps to 2e4; the codes are then all equal."""
    from mixtral_offloading_amd import hip_kernels
    w = np.zeros((64, 48), dtype=np.float32)
    w[:, 1] = 3.0
    w[:, 2] = np.linspace(0, 1e-6, 64)
    q, scale, zero = o.hqq_quantize_tensor(w, 4, 64)
    gq, gscale, gzero = hip_kernels.quantize_groups(torch.from_numpy(w).cuda(), 64, 4)
    assert np.array_equal(gq.cpu().numpy(), q)
    assert np.array_equal(gscale.cpu().numpy(), scale.reshape(1, -1)) and np.array_equal(gzero.cpu().numpy(), zero.reshape(1, -1))


@pytest.mark.parametrize("n", [1, 7, 4096, 100_003])
def test_whole_tensor_quantiser_equals_the_oracle(n):
    from mixtral_offloading_amd import hip_kernels
    rng = np.random.default_rng(n)
    x = (rng.standard_normal(n) * 3 + 1).astype(np.float32)
    q, scale, zero = o.hqq_quantize_tensor(x.reshape(1, n), 8, None, channel_wise=False)
    gq, gscale, gzero = hip_kernels.quantize_whole(torch.from_numpy(x).cuda().view(1, n), 8)
    assert np.array_equal(gq.cpu().numpy(), q.reshape(1, n))
    assert np.float32(gscale.item()) == np.float32(scale) and np.float32(gzero.item()) == np.float32(zero)


@pytest.mark.parametrize("nbits,gs", [(2, 16), (3, 64), (4, 64)])
def test_solver_agrees_with_the_oracle_and_lowers_the_error(nbits, gs):
    from mixtral_offloading_amd import hip_kernels
    rng = np.random.default_rng(7 + nbits)
    w = _weights(rng, 512, 256, np.float16)
    q, scale, zero = o.hqq_quantize_tensor(w, nbits, gs, optimize=True, round_zero=(nbits == 4))
    gq, gscale, gzero = hip_kernels.quantize_groups(torch.from_numpy(w).cuda(), gs, nbits, round_zero=(nbits == 4), iters=20)
    gq, gscale, gzero = gq.cpu().numpy(), gscale.cpu().numpy(), gzero.cpu().numpy()
    assert np.array_equal(gscale, scale.reshape(1, -1))  # the solver moves the zero only
    assert np.abs(gzero - zero.reshape(1, -1)).max() <= 1e-4 * (2 ** nbits)
    differ = gq != q
    assert differ.mean() <= 2e-4 and (not differ.any() or np.abs(gq.astype(int) - q.astype(int))[differ].max() == 1)
    # what the solver is for: a smaller l_p error (p = 0.7) of the reconstruction than plain min-max codes give
    wf = w.astype(np.float32).reshape(gs, -1)
    q0, s0, z0 = o.hqq_quantize_tensor(w, nbits, gs, round_zero=(nbits == 4))
    lp = lambda qq, ss, zz: float((np.abs(wf - (qq.astype(np.float32) - zz.reshape(1, -1)) * ss.reshape(1, -1)) ** 0.7).mean())  # noqa: E731
    assert lp(gq, gscale, gzero) < lp(q0, s0, z0)
    # and every code is the nearest level for the zero it ended with
    assert np.array_equal(gq, np.clip(np.round(wf / gscale + gzero), 0, 2 ** nbits - 1).astype(np.uint8)) or \
        (gq != np.clip(np.round(wf * (np.float32(1) / gscale) + gzero), 0, 2 ** nbits - 1)).mean() < 1e-3


def test_layer_quantised_on_the_gpu_equals_the_oracle_layer():
    """HQQLinearTritonSavable built from an fp16 nn.Linear on the GPU (codes through the quantiser, the packers and
    repack; 8-bit scale and zero tables through the quantiser again) against the oracle's layer, optimize off."""
    from mixtral_offloading_amd.custom_layers import HQQLinearTritonSavable
    from mixtral_offloading_amd.hqq_core import BaseQuantizeConfig
    rng = np.random.default_rng(3)
    for nbits, gs in [(2, 16), (3, 64), (4, 64)]:
        n, k = 640, 256
        w = _weights(rng, n, k, np.float16)
        cfg = BaseQuantizeConfig(nbits=nbits, group_size=gs, quant_zero=True, quant_scale=True)
        cfg["weight_quant_params"]["optimize"] = False
        lin = torch.nn.Linear(k, n, bias=False, dtype=torch.float16, device="cuda")
        lin.weight.data.copy_(torch.from_numpy(w))
        layer = HQQLinearTritonSavable(lin, cfg)
        want = o.hqq_quantize_layer(w, nbits, gs)
        assert np.array_equal(torch.Tensor.as_subclass(layer.W_q, torch.Tensor).cpu().numpy(), want["W_q"])
        assert np.array_equal(layer.meta["scale_q"].cpu().numpy(), want["scale_q"])
        assert np.array_equal(layer.meta["zero_q"].cpu().numpy().reshape(-1), want["zero_q"].reshape(-1))
        for t in ("meta_scale", "meta_zero"):
            for f in ("scale", "zero"):
                got = layer.meta[t][f].cpu().numpy().reshape(-1)
                assert np.array_equal(got.view(np.uint16), np.asarray(want[t][f], dtype=np.float16).reshape(-1).view(np.uint16)), (nbits, t, f)
