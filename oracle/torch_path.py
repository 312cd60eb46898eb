"""The reference's PyTorch path restated with torch CPU ops (test infrastructure:
the "port" CPU baseline of bench.py and a third implementation for the tests).

Follows ``HQQLinearTritonSavable.dequantize`` (src/custom_layers.py:95-116) with
the meta expansion it performs on every call (:100-103, hqq
``Quantizer.dequantize``), then ``x @ W.T``, and the expert FFN of
src/custom_layers.py:253-256.  Every elementwise op is a torch half op, so each
rounds once, as on the reference's device."""
from __future__ import annotations

import torch


def unpack(W_q: torch.Tensor, nbits: int) -> torch.Tensor:
    """src/packing.py:19-27, 43-53, 83-97."""
    if nbits == 4:
        out = torch.empty((2 * W_q.shape[0],) + tuple(W_q.shape[1:]), dtype=torch.uint8)
        out[0::2] = W_q >> 4
        out[1::2] = W_q & 0x0F
        return out
    if nbits == 2:
        out = torch.empty((4 * W_q.shape[0],) + tuple(W_q.shape[1:]), dtype=torch.uint8)
        for i in range(4):
            out[i::4] = (W_q >> (2 * (3 - i))) & 3
        return out
    out = torch.empty((10 * W_q.shape[0],) + tuple(W_q.shape[1:]), dtype=torch.uint8)
    for i in range(10):
        out[i::10] = ((W_q >> (3 * (9 - i))) & 7).to(torch.uint8)
    return out


def meta_dequant(q: torch.Tensor, meta: dict, shape) -> torch.Tensor:
    return ((q.half() - meta["zero"]) * meta["scale"]).reshape(shape)


def dequantize(layer: dict) -> torch.Tensor:
    n, k = layer["shape"]
    gs = layer["group_size"]
    s_cnt = n * k // gs
    scale = meta_dequant(layer["scale_q"], layer["meta_scale"], (1, s_cnt)) if layer.get("quant_scale") else layer["scale"]
    zero = meta_dequant(layer["zero_q"], layer["meta_zero"], (1, s_cnt)) if layer.get("quant_zero") else layer["zero"]
    w = unpack(layer["W_q"], layer["nbits"]).half()[:n].reshape(gs, -1)
    return ((w - zero) * scale).reshape(n, k)


def forward(x: torch.Tensor, layer: dict) -> torch.Tensor:
    """The reference's forward_pytorch-style path: dequantize, then matmul."""
    return torch.matmul(x, dequantize(layer).t())


def expert_ffn(x: torch.Tensor, w1: dict, w2: dict, w3: dict) -> torch.Tensor:
    h = torch.nn.functional.silu(forward(x, w1)) * forward(x, w3)
    return forward(h, w2)


def layer_from_numpy(layer: dict) -> dict:
    """Oracle (numpy) layer dict -> torch CPU tensors with the same keys."""
    import numpy as np

    def t(a):
        return torch.from_numpy(np.ascontiguousarray(a))

    out = {k: v for k, v in layer.items() if not hasattr(v, "dtype") and not isinstance(v, dict)}
    out["W_q"] = t(layer["W_q"])
    for key in ("scale_q", "zero_q", "scale", "zero"):
        if key in layer:
            out[key] = t(layer[key])
    for key in ("meta_scale", "meta_zero"):
        if key in layer:
            out[key] = {"scale": t(np.asarray(layer[key]["scale"])), "zero": t(np.asarray(layer[key]["zero"]))}
    return out


def random_layer(gen: torch.Generator, n: int, k: int, nbits: int, gs: int, meta_gs: int = 128) -> dict:
    """Synthetic layer with random codes and 8-bit tables (values in the range a quantiser of
    N(0, 0.02) weights gives); used where only speed matters."""
    s_cnt = n * k // gs
    step = 0.07 / (2 ** nbits - 1)
    q = torch.randint(0, 2 ** nbits, (n, k), dtype=torch.uint8, generator=gen)
    f = {4: 2, 2: 4, 3: 10}[nbits]
    if nbits == 3:
        pad = (-n) % 10
        qq = torch.cat([q, torch.zeros((pad, k), dtype=torch.uint8)]).to(torch.int32)
        W_q = torch.zeros((qq.shape[0] // 10, k), dtype=torch.int32)
        for i in range(10):
            W_q |= qq[i::10] << (3 * (9 - i))
    else:
        W_q = torch.zeros((n // f, k), dtype=torch.uint8)
        for i in range(f):
            W_q |= q[i::f] << (nbits * (f - 1 - i))
    return {"nbits": nbits, "group_size": gs, "shape": (n, k), "quant_scale": True, "quant_zero": True, "W_q": W_q,
            "scale_q": torch.randint(0, 256, (meta_gs, s_cnt // meta_gs), dtype=torch.uint8, generator=gen),
            "meta_scale": {"scale": torch.full((1, s_cnt // meta_gs), step / 255).half(),
                           "zero": torch.full((1, s_cnt // meta_gs), -128.0).half()},
            "zero_q": torch.randint(0, 256, (1, s_cnt), dtype=torch.uint8, generator=gen),
            "meta_zero": {"scale": torch.tensor((2 ** nbits - 1) / 255.0).half(), "zero": torch.tensor(0.0).half()}}
