"""Stand-in for the third-party ``hqq`` package (commit 37502bea) that the
reference imports (src/packing.py:2-3, src/custom_layers.py:6,
src/build_model.py:18) and that is not available offline.

It provides the same names with the same call signatures -- ``Quantizer``,
``BitPack``, ``BaseQuantizeConfig``, ``HQQLinear`` -- written with plain torch
ops so it runs on whichever device the tensors live on.  It is the quantise
side only (it manufactures ``W_q`` / ``meta``); the reference holds no test at
that boundary, so agreement with hqq's numerics is unpinned.  The hot path
(unpack, de-quantise, matmul) never runs here: it is the HIP library."""
from __future__ import annotations

import copy

import numpy as np
import torch
from torch import nn


class BitPack:
    """hqq's original "step" layout: code r of a column block lives ``step``
    rows apart instead of in adjacent rows.  On-disk hqq checkpoints use it;
    the reference converts it at load (src/custom_layers.py:41-47,
    src/packing.py:29-33)."""

    @staticmethod
    def pack_8bit_u8(W_q):
        return W_q.to(torch.uint8)

    @staticmethod
    def unpack_8bit_u8(W_q):
        return W_q

    @staticmethod
    def pack_4bit_u8(W_q):
        W_q = W_q.to(torch.uint8)
        step = W_q.shape[0] // 2
        return (W_q[:step] << 4) | W_q[step:]

    @staticmethod
    def unpack_4bit_u8(W_q):
        return torch.cat([(W_q & 0xF0) >> 4, W_q & 0x0F], dim=0)

    @staticmethod
    def pack_2bit_u8(W_q):
        W_q = W_q.to(torch.uint8)
        s = W_q.shape[0] // 4
        return (W_q[:s] << 6) | (W_q[s:2 * s] << 4) | (W_q[2 * s:3 * s] << 2) | W_q[3 * s:]

    @staticmethod
    def unpack_2bit_u8(W_q):
        return torch.cat([(W_q & 0xC0) >> 6, (W_q & 0x30) >> 4, (W_q & 0x0C) >> 2, W_q & 0x03], dim=0)

    @staticmethod
    def pack_3bit_32(W_q_in):
        rows = 10 * ((W_q_in.shape[0] + 9) // 10)
        W_q = torch.zeros((rows,) + tuple(W_q_in.shape[1:]), device=W_q_in.device, dtype=torch.int32)
        W_q[: W_q_in.shape[0]] = W_q_in
        s = rows // 10
        out = W_q[:s] << 27
        for i in range(1, 10):
            out = out | (W_q[i * s:(i + 1) * s] << (3 * (9 - i)))
        return out

    @staticmethod
    def unpack_3bit_32(W_q):
        return torch.cat([((W_q >> (3 * (9 - i))) & 7).to(torch.uint8) for i in range(10)], dim=0)


class Quantizer:
    SUPPORTED_BITS = [8, 4, 3, 2]
    bit_to_packing = {8: "8bit_u8", 4: "4bit_u8", 3: "3bit_32", 2: "2bit_u8"}
    pack = {"8bit_u8": BitPack.pack_8bit_u8, "4bit_u8": BitPack.pack_4bit_u8,
            "3bit_32": BitPack.pack_3bit_32, "2bit_u8": BitPack.pack_2bit_u8}
    unpack = {"8bit_u8": BitPack.unpack_8bit_u8, "4bit_u8": BitPack.unpack_4bit_u8,
              "3bit_32": BitPack.unpack_3bit_32, "2bit_u8": BitPack.unpack_2bit_u8}

    @classmethod
    def quantize(cls, tensor, nbits=4, channel_wise=True, group_size=64, optimize=False, round_zero=False,
                 axis=0, bitpack=True):
        assert nbits in cls.SUPPORTED_BITS
        assert axis in (0, 1)
        if group_size is not None:
            assert tensor.numel() % group_size == 0
        max_v = 2 ** nbits - 1
        if tensor.is_cuda and tensor.numel() > 0 and tensor.dtype in (torch.float16, torch.float32):
            # the library's quantiser for the two forms this path uses; anything else goes through the tensor ops below
            from . import hip_kernels
            got = None
            if channel_wise and axis == 0 and group_size in hip_kernels.QUANTIZE_GROUP_SIZES:
                iters = cls.OPT_PARAMS["iters"] if optimize else 0
                got = hip_kernels.quantize_groups(tensor.contiguous(), group_size, nbits, round_zero, iters,
                                                  cls.OPT_PARAMS["lp_norm"], cls.OPT_PARAMS["beta"], cls.OPT_PARAMS["kappa"])
            elif not channel_wise and not round_zero:
                got = hip_kernels.quantize_whole(tensor.float().contiguous(), nbits)
            if got is not None:
                W_q, inv_scale, zero = got
                meta = {"nbits": nbits, "group_size": group_size, "shape": tensor.shape, "scale": inv_scale, "zero": zero,
                        "axis": axis, "packing": cls.bit_to_packing[nbits]}
                if bitpack:
                    W_q = cls.pack[meta["packing"]](W_q)
                else:
                    W_q = W_q.to(tensor.dtype)
                    meta["packing"] = None
                return W_q, meta
        W = tensor.float()
        shape = W.shape
        if group_size is not None and channel_wise:
            W = W.reshape([-1, group_size]) if axis == 1 else W.reshape([group_size, -1])
        if not channel_wise:
            _min, _max = W.min(), W.max()
            optimize = False
        else:
            _min = W.min(axis=axis, keepdim=True)[0]
            _max = W.max(axis=axis, keepdim=True)[0]
        scale = (max_v / (_max - _min)).clamp(max=2e4)
        zero = -_min * scale
        if round_zero:
            zero = torch.round(zero)
        if optimize:
            scale, zero = cls.optimize_weights(W, scale, zero, (0, max_v), axis)
        W_q = torch.round(W * scale + zero).clamp(0, max_v)
        meta = {"nbits": nbits, "group_size": group_size, "shape": shape, "scale": 1.0 / scale, "zero": zero,
                "axis": axis, "packing": cls.bit_to_packing[nbits]}
        if bitpack:
            W_q = cls.pack[meta["packing"]](W_q)
        else:
            W_q = W_q.to(tensor.dtype)
            meta["packing"] = None
        return W_q, meta

    OPT_PARAMS = {"lp_norm": 0.7, "beta": 1e1, "kappa": 1.01, "iters": 20}

    @classmethod
    def optimize_weights(cls, tensor, scale, zero, min_max, axis=0, opt_params=None, verbose=False):
        """Half-quadratic proximal refinement of the zero point (lp norm 0.7)."""
        p = dict(cls.OPT_PARAMS)
        if opt_params:
            p.update(opt_params)
        lp, beta, kappa = p["lp_norm"], p["beta"], p["kappa"]
        W_f = tensor.float()
        scale, zero = scale.float(), zero.float()

        def shrink(x):
            return torch.sign(x) * torch.relu(torch.abs(x) - (1.0 / beta) * torch.pow(torch.abs(x) + 1e-8, lp - 1))

        best = 1e4
        for _ in range(p["iters"]):
            W_q = torch.round(W_f * scale + zero).clamp(min_max[0], min_max[1])
            W_r = (W_q - zero) / scale
            W_e = shrink(W_f - W_r)
            zero = torch.mean(W_q - (W_f - W_e) * scale, axis=axis, keepdim=True)
            beta *= kappa
            err = float(torch.abs(W_f - W_r).mean())
            if err < best:
                best = err
            else:
                break
        return scale, zero

    @classmethod
    def dequantize(cls, W_q, meta):
        if meta["packing"]:
            W_r = cls.unpack[meta["packing"]](W_q).half()
            if meta["group_size"] is not None and meta["nbits"] == 3:
                W_r = W_r[: meta["group_size"]] if meta["axis"] == 0 else W_r[:, : meta["group_size"]]
        else:
            W_r = W_q.half()
        return ((W_r - meta["zero"]) * meta["scale"]).reshape(meta["shape"])

    @classmethod
    def to_device(cls, W_q, meta, device):
        meta_c = {k: (v.half().to(device) if isinstance(v, torch.Tensor) else v) for k, v in meta.items()}
        return W_q.to(device), meta_c


def hqq_base_quant_config(nbits=4, group_size=64, quant_zero=True, quant_scale=False):
    assert nbits in Quantizer.SUPPORTED_BITS
    if group_size is not None:
        assert group_size % 8 == 0, "group_size must be a multiple of 8"
    weight = {"nbits": nbits, "channel_wise": True, "group_size": group_size, "optimize": True,
              "round_zero": nbits == 4}
    scale = {"nbits": 8, "channel_wise": True, "group_size": 128, "optimize": False} if quant_scale else None
    zero = {"nbits": 8, "channel_wise": False, "group_size": None, "optimize": False} if quant_zero else None
    return {"weight_quant_params": weight, "scale_quant_params": scale, "zero_quant_params": zero}


BaseQuantizeConfig = hqq_base_quant_config


class HQQLinear(nn.Module):
    """Minimal base with the attributes the reference's subclass relies on:
    ``W_q``, ``meta``, ``bias``, ``ready``, ``quant_config``."""

    def __init__(self, linear_layer, quant_config, del_orig=True):
        super().__init__()
        self.ready = False
        self.in_gpu = False
        self.quant_config = copy.deepcopy(quant_config)
        self.bias = None
        self.W_q = None
        if linear_layer is not None:
            self.bias = None if linear_layer.bias is None else linear_layer.bias.detach().half()
            self.quantize(linear_layer.weight.data, **self.quant_config)
        if del_orig and linear_layer is not None:
            del linear_layer

    def quantize(self, W, weight_quant_params, scale_quant_params, zero_quant_params):
        quant_scale = scale_quant_params is not None
        quant_zero = zero_quant_params is not None
        self.in_features, self.out_features = W.t().shape
        W_q, meta = Quantizer.quantize(W, **weight_quant_params)
        meta.update({"quant_scale": quant_scale, "quant_zero": quant_zero})
        if quant_scale:
            meta["scale_q"], meta["meta_scale"] = Quantizer.quantize(meta["scale"], **scale_quant_params)
            del meta["scale"]
        if quant_zero:
            meta["zero_q"], meta["meta_zero"] = Quantizer.quantize(meta["zero"], **zero_quant_params)
            del meta["zero"]
        dev = W.device
        self.W_q, self.meta = Quantizer.to_device(W_q, meta, dev)
        if quant_scale:
            self.meta["scale_q"], self.meta["meta_scale"] = Quantizer.to_device(
                self.meta["scale_q"], self.meta["meta_scale"], dev)
        if quant_zero:
            self.meta["zero_q"], self.meta["meta_zero"] = Quantizer.to_device(
                self.meta["zero_q"], self.meta["meta_zero"], dev)
        # scale_q / zero_q are 8-bit codes, not fp16 values: undo the blanket half() of to_device
        if quant_scale:
            self.meta["scale_q"] = self.meta["scale_q"].to(torch.uint8)
        if quant_zero:
            self.meta["zero_q"] = self.meta["zero_q"].to(torch.uint8)
        self.ready = True
        self.in_gpu = self.W_q.device.type == "cuda"


def closed_form_meta(linear_shape, quant_config):
    """Non-tensor meta of a layer of ``nn.Linear(*linear_shape)`` without
    quantising a throw-away layer (the reference's get_hqq_meta does that,
    src/custom_layers.py:118-134)."""
    in_f, out_f = linear_shape
    w = quant_config["weight_quant_params"]
    nbits, gs = w["nbits"], w["group_size"]
    s_cnt = in_f * out_f // gs
    meta = {"nbits": nbits, "group_size": gs, "shape": torch.Size([out_f, in_f]), "axis": w.get("axis", 0),
            "packing": Quantizer.bit_to_packing[nbits],
            "quant_scale": quant_config["scale_quant_params"] is not None,
            "quant_zero": quant_config["zero_quant_params"] is not None}
    for key, params in (("meta_scale", quant_config["scale_quant_params"]),
                        ("meta_zero", quant_config["zero_quant_params"])):
        if params is not None:
            meta[key] = {"nbits": params["nbits"], "group_size": params["group_size"],
                         "shape": torch.Size([1, s_cnt]), "axis": 0,
                         "packing": Quantizer.bit_to_packing[params["nbits"]]}
    return meta
