"""The committed golden vectors (tests/golden/hot_path_vectors.npz, written by tests/golden/make_hot_path_vectors.py):
the oracle must still reproduce them (CPU), and the HIP path must match them (GPU)."""
import os

import numpy as np
import pytest

from oracle import hqq_oracle as o

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "hot_path_vectors.npz")
CASES = ["w4_g64", "w2_g16", "w3_g64_tail", "w3_g13_f16", "w4_g16_f16"]


def load_layer(z, prefix):
    nbits, gs, n, k, qs, qz = (int(v) for v in z[f"{prefix}.info"])
    layer = {"nbits": nbits, "group_size": gs, "shape": (n, k), "quant_scale": bool(qs), "quant_zero": bool(qz),
             "W_q": z[f"{prefix}.W_q"]}
    for key in ("scale_q", "zero_q", "scale", "zero"):
        if f"{prefix}.{key}" in z.files:
            layer[key] = z[f"{prefix}.{key}"]
    for m in ("meta_scale", "meta_zero"):
        if f"{prefix}.{m}.scale" in z.files:
            layer[m] = {"scale": z[f"{prefix}.{m}.scale"], "zero": z[f"{prefix}.{m}.zero"]}
    return layer


@pytest.mark.parametrize("name", CASES)
def test_oracle_reproduces_golden_vectors(name):
    z = np.load(GOLDEN)
    layer = load_layer(z, name)
    assert np.array_equal(o.dequantize(layer).view(np.uint16), z[f"{name}.dequant_bits"])
    y = o.matmul_transpose(z[f"{name}.x"], layer, bias=z[f"{name}.bias"])
    assert np.array_equal(y.view(np.uint16), z[f"{name}.y"].view(np.uint16))


def test_oracle_reproduces_golden_ffn_and_router():
    z = np.load(GOLDEN)
    w1, w2, w3 = (load_layer(z, f"ffn.w{i}") for i in (1, 2, 3))
    assert np.array_equal(o.expert_ffn(z["ffn.x"], w1, w2, w3).view(np.uint16), z["ffn.y"].view(np.uint16))
    weights, experts, logits = o.router(z["ffn.x"], z["router.gate"], top_k=2)
    assert np.array_equal(experts, z["router.experts"])
    assert np.array_equal(weights.view(np.uint16), z["router.weights"].view(np.uint16))


@pytest.mark.gpu
@pytest.mark.parametrize("name", CASES)
def test_hip_path_matches_golden_vectors(name):
    from helpers import assert_matmul_close, desc_of, to_dev
    from mixtral_offloading_amd import hip_kernels
    z = np.load(GOLDEN)
    layer = load_layer(z, name)
    desc = desc_of(layer, bias=z[f"{name}.bias"])
    w = hip_kernels.dequantize(desc).cpu().numpy()
    assert np.array_equal(w.view(np.uint16), z[f"{name}.dequant_bits"].reshape(w.shape)), "dequantize is not bit-exact"
    x = z[f"{name}.x"]
    y = hip_kernels.matmul(desc, to_dev(x)).cpu().numpy()
    assert_matmul_close(y, z[f"{name}.y"], o.matmul_tolerance(x, layer).reshape(y.shape))


@pytest.mark.gpu
def test_hip_ffn_matches_golden_vectors():
    from helpers import assert_matmul_close, desc_of, to_dev
    from mixtral_offloading_amd import hip_kernels
    z = np.load(GOLDEN)
    w1, w2, w3 = (load_layer(z, f"ffn.w{i}") for i in (1, 2, 3))
    x = z["ffn.x"]
    y = hip_kernels.expert_ffn(desc_of(w1), desc_of(w2), desc_of(w3), to_dev(x)).cpu().numpy()
    h = (o.silu_f16(o.matmul_transpose(x, w1)).astype(np.float32) * o.matmul_transpose(x, w3).astype(np.float32))
    assert_matmul_close(y, z["ffn.y"], 4 * o.matmul_tolerance(h.astype(np.float16), w2), rtol=2e-2)
