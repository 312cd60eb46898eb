"""Shared helpers of the GPU parity tests: move an oracle layer (numpy) to the
device and wrap it in the library's descriptor."""
import numpy as np
import torch

from mixtral_offloading_amd import hip_kernels


def to_dev(a, device="cuda"):
    return torch.from_numpy(np.ascontiguousarray(a)).to(device)


def layer_to_device(layer: dict, device="cuda"):
    """Returns (W_q tensor, meta dict of device tensors) in the reference's meta schema."""
    n, k = layer["shape"]
    meta = {"nbits": layer["nbits"], "group_size": layer["group_size"], "shape": (n, k), "axis": 0,
            "quant_scale": layer["quant_scale"], "quant_zero": layer["quant_zero"]}
    if layer["quant_scale"]:
        meta["scale_q"] = to_dev(layer["scale_q"], device)
        meta["meta_scale"] = {"scale": to_dev(layer["meta_scale"]["scale"], device),
                              "zero": to_dev(layer["meta_scale"]["zero"], device)}
    else:
        meta["scale"] = to_dev(layer["scale"], device)
    if layer["quant_zero"]:
        meta["zero_q"] = to_dev(layer["zero_q"], device)
        meta["meta_zero"] = {"scale": to_dev(np.asarray(layer["meta_zero"]["scale"]).reshape(1), device),
                             "zero": to_dev(np.asarray(layer["meta_zero"]["zero"]).reshape(1), device)}
    else:
        meta["zero"] = to_dev(layer["zero"], device)
    return to_dev(layer["W_q"], device), meta


def desc_of(layer: dict, device="cuda", bias=None):
    wq, meta = layer_to_device(layer, device)
    b = None if bias is None else to_dev(bias, device)
    return hip_kernels.LinearDesc(wq, meta, b)


def assert_matmul_close(y_gpu: np.ndarray, y_ref: np.ndarray, atol: np.ndarray, rtol=1e-2):
    """|y - ref| <= rtol*|ref| + atol, with atol = 1e-3*||x||*||w|| per element
    (the tolerance the path is specified to)."""
    err = np.abs(y_gpu.astype(np.float64) - y_ref.astype(np.float64))
    bound = rtol * np.abs(y_ref.astype(np.float64)) + atol
    bad = err > bound
    assert not bad.any(), (f"{int(bad.sum())} of {bad.size} outputs out of tolerance; worst err {err.max():.4g}, "
                           f"worst err/bound {(err / bound).max():.3g}")
    return float((err / bound).max())
