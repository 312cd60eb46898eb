"""Writes tests/golden/hot_path_vectors.npz: small fixed inputs of the hot path with the outputs the numpy oracle
gives for them (de-quantised weights as fp16 bit patterns, matmul, expert FFN, router).  Run from the repository
root: ``python tests/golden/make_hot_path_vectors.py``.  The fixtures pin the oracle against later edits (the CPU
suite recomputes them) and give the GPU suite inputs that do not depend on a random generator's stream."""
import os
import sys

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)
from oracle import hqq_oracle as o  # noqa: E402

# (name, nbits, N, K, group size, 8-bit tables, batch)
CASES = [("w4_g64", 4, 128, 128, 64, True, 3), ("w2_g16", 2, 64, 256, 16, True, 2), ("w3_g64_tail", 3, 640, 64, 64, True, 2),
         ("w3_g13_f16", 3, 130, 64, 13, False, 1), ("w4_g16_f16", 4, 64, 64, 16, False, 5)]
LAYER_KEYS = ("W_q", "scale_q", "zero_q", "scale", "zero")


def flatten_layer(prefix, layer, out):
    for key in LAYER_KEYS:
        if key in layer and layer[key] is not None:
            out[f"{prefix}.{key}"] = np.asarray(layer[key])
    for m in ("meta_scale", "meta_zero"):
        if layer.get(m) is not None:
            out[f"{prefix}.{m}.scale"] = np.asarray(layer[m]["scale"], dtype=np.float16)
            out[f"{prefix}.{m}.zero"] = np.asarray(layer[m]["zero"], dtype=np.float16)
    out[f"{prefix}.info"] = np.array([layer["nbits"], layer["group_size"], layer["shape"][0], layer["shape"][1],
                                      int(layer["quant_scale"]), int(layer["quant_zero"])], dtype=np.int64)


def main():
    rng = np.random.default_rng(20240521)
    out = {}
    for name, nbits, n, k, gs, q8, m in CASES:
        layer, _ = o.random_layer(rng, n, k, nbits, gs, q8, q8, meta_group_size=min(128, n * k // gs))
        x = rng.standard_normal((m, k)).astype(np.float16)
        bias = rng.standard_normal(n).astype(np.float16)
        flatten_layer(name, layer, out)
        out[f"{name}.x"] = x
        out[f"{name}.bias"] = bias
        out[f"{name}.dequant_bits"] = o.dequantize(layer).view(np.uint16)
        out[f"{name}.y"] = o.matmul_transpose(x, layer, bias=bias)
    # one expert FFN and one router call
    hidden, ffn = 256, 256
    ws = [o.random_layer(rng, a, b, 2, 16)[0] for a, b in ((ffn, hidden), (hidden, ffn), (ffn, hidden))]
    x = rng.standard_normal((2, hidden)).astype(np.float16)
    for tag, layer in zip(("ffn.w1", "ffn.w2", "ffn.w3"), ws):
        flatten_layer(tag, layer, out)
    out["ffn.x"] = x
    out["ffn.y"] = o.expert_ffn(x, ws[0], ws[1], ws[2])
    gate = (rng.standard_normal((8, hidden)) * 0.05).astype(np.float16)
    weights, experts, logits = o.router(x, gate, top_k=2)
    out["router.gate"], out["router.weights"], out["router.experts"], out["router.logits"] = gate, weights, experts, logits
    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "hot_path_vectors.npz")
    np.savez_compressed(path, **out)
    print(path, os.path.getsize(path), "bytes,", len(out), "arrays")


if __name__ == "__main__":
    main()
