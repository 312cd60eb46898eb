"""Quantised linear, expert FFN and sparse-MoE block with the reference's
module surface (reference ``src/custom_layers.py``), computing on the HIP
library.

``HQQLinearTritonSavable`` keeps its reference name although nothing here is
Triton: the name is the drop-in contract.  Differences that do not change
results: the 8-bit scale / zero tables are de-quantised inside the matmul
kernel rather than expanded to fp16 per call (reference :62-66), the code
layout is tracked by an explicit flag next to the ``PackedTensor`` tag
(reference src/packing.py:29-33 relies on the tag alone), and the non-tensor
meta is computed in closed form (reference :118-134 quantises a dummy layer)."""
from __future__ import annotations

import copy
from typing import Any, Dict

import numpy as np
import torch
from torch import nn
from torch.nn import functional as F

from . import hip_kernels
from .hqq_core import HQQLinear, Quantizer, closed_form_meta
from .packing import PackedTensor

_META_TENSOR_KEYS = {"scale_q", "meta_scale.scale", "meta_scale.zero", "zero_q", "meta_zero.scale",
                     "meta_zero.zero", "scale", "zero"}


def _codes_shape(meta) -> tuple:
    n, k = int(meta["shape"][0]), int(meta["shape"][1])
    nbits = meta["nbits"]
    if nbits == 3:
        return ((n + 9) // 10, k)
    return (n * nbits // 8, k)


class HQQLinearTritonSavable(HQQLinear):
    def __init__(self, layer, quant_config, meta=None, **kwargs):
        """``meta`` for an empty layer comes from ``get_hqq_meta((in, out), quant_config)``."""
        assert quant_config["weight_quant_params"]["nbits"] in [2, 3, 4]
        super().__init__(layer, quant_config, **kwargs)
        self._desc_cache = None
        if not hasattr(self, "meta"):
            assert meta is not None
            self.meta = copy.deepcopy(meta)
        self._register_state_dict_hook(self._add_to_state_dict_hook)
        self._register_load_state_dict_pre_hook(self._load_from_state_dict_hook)

    # ---------------------------------------------------------------- layout
    def quantize(self, *args, **kwargs):
        super().quantize(*args, **kwargs)
        self.repack()

    # Layout of the codes a state dict brings in: "hqq" (the quantiser's (gs/f, N*K/gs) step layout, what the
    # reference's checkpoints hold and what the reference assumes of every untagged tensor, src/packing.py:29-33) or
    # "kernel" ((N/f, K) interleaved, written by save_quantized_checkpoint(layout="kernel")).  The two shapes can
    # coincide (N == group_size), so the layout is never guessed from the shape: the loader sets this from the
    # checkpoint's index.
    checkpoint_layout = "hqq"

    def in_kernel_layout(self) -> bool:
        """Codes are in the kernel layout when they carry the interleaved packers' tag and have the (N/f, K) shape.
        (Tagged codes of that shape cannot be anything else: the quantiser's view (gs, N*K/gs) has it only when
        gs == N, where the two layouts are the same array.)  Untagged codes never are: they hold hqq's step layout."""
        return isinstance(self.W_q, PackedTensor) and tuple(self.W_q.shape) == _codes_shape(self.meta)

    def repack(self):
        """Quantise-time layout (gs/f, N*K/gs) -> kernel layout (N/f, K)
        (reference src/custom_layers.py:41-47).  Untagged codes are in hqq's step layout, as in the reference; tagged
        ones were packed by the interleaved packers (the patched registry) in the quantiser's shape."""
        if not self.in_kernel_layout():
            sh = tuple(int(v) for v in self.meta["shape"])
            codes = Quantizer.unpack[self.meta["packing"]](self.W_q)
            codes = codes.reshape((-1,) + sh[1:])[: sh[0], ...]
            self.W_q = Quantizer.pack[self.meta["packing"]](codes.contiguous())
        assert tuple(self.W_q.shape) == _codes_shape(self.meta), "codes do not have the kernel layout's shape"
        self._desc_cache = None

    # --------------------------------------------------------------- compute
    def _desc(self) -> hip_kernels.LinearDesc:
        meta = self.meta
        ptrs = (self.W_q.data_ptr(),
                meta["scale_q"].data_ptr() if meta.get("quant_scale") else meta["scale"].data_ptr(),
                meta["zero_q"].data_ptr() if meta.get("quant_zero") else meta["zero"].data_ptr(),
                self.bias.data_ptr() if getattr(self, "bias", None) is not None else 0)
        if self._desc_cache is None or self._desc_cache[0] != ptrs:
            assert self.in_kernel_layout(), "codes are not in the kernel layout; call repack()"
            self._desc_cache = (ptrs, hip_kernels.LinearDesc(self.W_q, meta, getattr(self, "bias", None)))
        return self._desc_cache[1]

    def forward(self, x):
        return self.forward_triton(x)

    def set_backend(self, backend):
        pass

    @torch.inference_mode()
    def forward_triton(self, x):
        """y = x @ dequant(W).T (+ bias) (reference src/custom_layers.py:55-92)."""
        assert self.ready, "model was not quantized"
        assert self.meta["axis"] == 0
        if self.meta["nbits"] not in (2, 3, 4):
            raise RuntimeError(f"nbits == {self.meta['nbits']} isn't yet supported")
        if x.dtype != torch.float16:
            x = x.to(torch.float16)
        return hip_kernels.matmul(self._desc(), x.contiguous())

    forward_hip = forward_triton

    @torch.inference_mode()
    def dequantize(self):
        """fp16 (N, K) weights, bit-exact ``(q - z) * s`` (reference src/custom_layers.py:95-116)."""
        assert self.ready, "model was not quantized"
        return hip_kernels.dequantize(self._desc()).reshape(tuple(self.meta["shape"]))

    @classmethod
    def get_hqq_meta(cls, linear_shape, quant_config):
        return closed_form_meta(linear_shape, quant_config)

    # ------------------------------------------------------------ state dict
    @staticmethod
    def _add_to_state_dict_hook(self, state_dict, prefix, local_metadata):
        """Flat key schema of the reference (src/custom_layers.py:136-166)."""
        assert set(self._get_tensor_paths(self.meta)).issubset(_META_TENSOR_KEYS)
        out = {"W_q": torch.Tensor.as_subclass(self.W_q, torch.Tensor)}
        if self.bias is not None:
            out["bias"] = self.bias
        meta = self.meta
        if "meta_scale" in meta and "scale_q" in meta:
            out["meta.scale_q"] = meta["scale_q"]
            out["meta.meta_scale.scale"] = meta["meta_scale"]["scale"]
            out["meta.meta_scale.zero"] = meta["meta_scale"]["zero"]
        else:
            out["meta.scale"] = meta["scale"]
        if "meta_zero" in meta and "zero_q" in meta:
            out["meta.zero_q"] = meta["zero_q"]
            out["meta.meta_zero.scale"] = meta["meta_zero"]["scale"]
            out["meta.meta_zero.zero"] = meta["meta_zero"]["zero"]
        else:
            out["meta.zero"] = meta["zero"]
        for name, value in out.items():
            state_dict[prefix + name] = value
        return state_dict

    def _load_from_state_dict_hook(self, state_dict, prefix, local_metadata, strict, missing_keys, unexpected_keys,
                                   error_msgs):
        """Inverse of the hook above (reference src/custom_layers.py:168-222); ends in ``repack``."""
        mine = [k[len(prefix):] for k in state_dict if k.startswith(prefix)]
        assert {k[len("meta."):] for k in mine if k.startswith("meta.")}.issubset(_META_TENSOR_KEYS)

        def take(name):
            return state_dict.pop(prefix + name)

        self.W_q = take("W_q")
        if self.checkpoint_layout == "kernel":
            assert tuple(self.W_q.shape) == _codes_shape(self.meta), "a kernel-layout checkpoint holds (N/f, K) codes"
            self.W_q = PackedTensor(torch.Tensor.as_subclass(self.W_q, torch.Tensor))
        else:
            self.W_q = torch.Tensor.as_subclass(self.W_q, torch.Tensor)  # untagged: hqq's step layout
        self.bias = take("bias") if (prefix + "bias") in state_dict else None
        if not hasattr(self, "meta"):
            self.meta = {}
        meta = self.meta
        if (prefix + "meta.meta_scale.scale") in state_dict:
            meta["scale_q"] = take("meta.scale_q")
            meta["quant_scale"] = True
            meta.setdefault("meta_scale", {})
            meta["meta_scale"].update(scale=take("meta.meta_scale.scale"), zero=take("meta.meta_scale.zero"))
            if meta["scale_q"].dtype != torch.uint8:  # codes saved as fp16 numbers 0..255
                meta["scale_q"] = meta["scale_q"].to(torch.uint8)
        else:
            meta["scale"] = take("meta.scale")
            meta["quant_scale"] = False
        if (prefix + "meta.meta_zero.scale") in state_dict:
            meta["zero_q"] = take("meta.zero_q")
            meta["quant_zero"] = True
            meta.setdefault("meta_zero", {})
            meta["meta_zero"].update(scale=take("meta.meta_zero.scale"), zero=take("meta.meta_zero.zero"))
            if meta["zero_q"].dtype != torch.uint8:
                meta["zero_q"] = meta["zero_q"].to(torch.uint8)
        else:
            meta["zero"] = take("meta.zero")
            meta["quant_zero"] = False
        self.ready = True
        self.repack()

    @classmethod
    def _get_tensor_paths(cls, state: Dict[str, Any], prefix=""):
        paths = []
        for k, v in state.items():
            if isinstance(v, dict):
                paths += cls._get_tensor_paths(v, prefix=k + ".")
            elif isinstance(v, torch.Tensor):
                paths.append(prefix + k)
        return paths

    def state_dict(self, *args, **kwargs):
        return nn.Module.state_dict(self, *args, **kwargs)

    def load_state_dict(self, *args, **kwargs):
        nn.Module.load_state_dict(self, *args, **kwargs)


class MixtralBLockSparseTop2MLP_HQQ(nn.Module):
    """Expert FFN ``w2(act(w1 x) * w3 x)`` (reference src/custom_layers.py:243-256).

    ``config`` only needs ``hidden_act``; SiLU runs fused in the HIP library,
    any other activation takes three separate matmuls."""

    def __init__(self, config, quant_config: Dict[str, Any], meta1, meta2):
        super().__init__()
        self.w1 = HQQLinearTritonSavable(None, quant_config, meta1)
        self.w2 = HQQLinearTritonSavable(None, quant_config, meta2)
        self.w3 = HQQLinearTritonSavable(None, quant_config, meta1)
        self.hidden_act = getattr(config, "hidden_act", "silu")

    @torch.inference_mode()
    def forward(self, hidden_states, out=None, row_scale=None, accumulate=False):
        if self.hidden_act != "silu":
            from transformers.activations import ACT2FN

            y = self.w2(ACT2FN[self.hidden_act](self.w1(hidden_states)) * self.w3(hidden_states))
            if row_scale is not None:
                y = y * row_scale[:, None]
            if out is None:
                return y
            return out.add_(y) if accumulate else out.copy_(y)
        x = hidden_states.to(torch.float16).contiguous()
        y = hip_kernels.expert_ffn(self.w1._desc(), self.w2._desc(), self.w3._desc(), x, out=out,
                                   row_scale=row_scale, accumulate=accumulate)
        return y.view(hidden_states.shape[:-1] + (y.shape[-1],)) if out is None else out


class SparseMoeWrapper(nn.Module):
    """Router + expert dispatch over an ``ExpertCache`` (reference src/custom_layers.py:259-314).

    Returns ``(hidden_states, router_logits)`` like the reference.  Each expert's FFN runs as the fused library
    call with the routing weight and the accumulation into the output folded in (reference :307-312 gathers,
    multiplies and ``index_add_``s with separate kernels)."""

    def __init__(self, config, layer_id, gate, expert_cache):
        super().__init__()
        self.hidden_dim = config.hidden_size
        self.ffn_dim = config.intermediate_size
        self.num_experts = config.num_local_experts
        self.top_k = config.num_experts_per_tok
        self.layer_id = layer_id
        self.gate = gate
        self.experts = expert_cache

    def _resident_group(self):
        """The layer's experts as ``hip_kernels.ExpertGroup`` when all of them are resident and none can be evicted
        (their device modules then never move), else None."""
        modules = self.experts.resident_group(self.layer_id) if hasattr(self.experts, "resident_group") else None
        if modules is None or len(modules) != self.num_experts:
            return None
        layers = []
        for m in modules:
            ffn = m._expert[0] if hasattr(m, "_expert") else m
            if getattr(ffn, "hidden_act", "silu") != "silu" or not all(hasattr(ffn, n) for n in ("w1", "w2", "w3")):
                return None
            layers.append((ffn.w1._desc(), ffn.w2._desc(), ffn.w3._desc()))
        key = tuple(id(d) for t in layers for d in t)
        if getattr(self, "_group_cache", None) is None or self._group_cache[0] != key:
            self._group_cache = (key, hip_kernels.ExpertGroup(layers))
        return self._group_cache[1]

    @torch.inference_mode()
    def forward_routed(self, hidden_states: torch.Tensor, selected: torch.Tensor, weights: torch.Tensor,
                       out: torch.Tensor, chosen=None) -> torch.Tensor:
        """One token whose router has already run on the device (``hip_kernels.add_rmsnorm_router``): ``selected``
        int32[2] and ``weights`` fp16[2] are device tensors.  The host reads the choice (the one synchronisation of the
        layer, as the cache is driven from the host; ``chosen`` hands it in when the caller has read it already),
        loads what is missing and runs the experts into ``out``."""
        if chosen is None:
            chosen = selected.cpu().tolist()
        first = True
        for (_layer_index, expert_idx), expert_layer in self.experts.load_experts(
                *((self.layer_id, expert_idx) for expert_idx in sorted(set(chosen))), unordered=True):
            k = chosen.index(expert_idx)
            expert_layer(hidden_states, out=out, row_scale=weights[k:k + 1], accumulate=not first)
            first = False
        return out

    @torch.inference_mode()
    def forward(self, hidden_states: torch.Tensor):
        batch_size, sequence_length, hidden_dim = hidden_states.shape
        hidden_states = hidden_states.reshape(-1, hidden_dim)
        if (hidden_states.is_cuda and hidden_states.dtype == torch.float16 and self.top_k == 2 and self.num_experts <= 16
                and hidden_dim % 8 == 0 and self.gate.bias is None and hidden_states.is_contiguous()):
            # the five lines below as one launch (one block per token)
            selected_experts, routing_weights, router_logits = hip_kernels.router_top2_rows(hidden_states, self.gate.weight)
        else:
            router_logits = self.gate(hidden_states)  # (tokens, n_experts)
            routing_weights = F.softmax(router_logits, dim=1, dtype=torch.float)
            routing_weights, selected_experts = torch.topk(routing_weights, self.top_k, dim=-1)
            routing_weights /= routing_weights.sum(dim=-1, keepdim=True)
            routing_weights = routing_weights.to(hidden_states.dtype)

        tokens = hidden_states.shape[0]
        final_hidden_states = torch.zeros((tokens, hidden_dim), dtype=hidden_states.dtype, device=hidden_states.device)
        if tokens > 1 and selected_experts.dtype == torch.int32 and routing_weights.dtype == torch.float16:
            # Several tokens, router on the device: the (token, slot) pairs are grouped by expert there as well, the
            # rows of every expert are gathered at once, and only then does the host wait, for the experts' row counts
            # alone (reference :288-312 does a where / gather / index_add_ per expert).  Each token receives the same
            # two fp16 terms in the index_add_ below, and their sum does not depend on the order.
            counts_dev, top_x, scales = hip_kernels.moe_group_pairs(selected_experts, routing_weights, self.num_experts)
            gathered = hidden_states.index_select(0, top_x)
            weighted = torch.empty_like(gathered)
            group = self._resident_group()
            counts = counts_dev.cpu().numpy()  # the one host sync of the layer
            starts = np.concatenate(([0], np.cumsum(counts)))
            if group is not None:
                # every expert of the layer is resident for good: all of them from one library call
                hip_kernels.expert_groups_ffn(group, gathered, starts, scales, weighted)
            else:
                active_experts = [e for e in range(self.num_experts) if counts[e] > 0]
                for (_layer_index, expert_idx), expert_layer in self.experts.load_experts(
                        *((self.layer_id, expert_idx) for expert_idx in active_experts), unordered=True):
                    lo, hi = int(starts[expert_idx]), int(starts[expert_idx + 1])
                    expert_layer(gathered[lo:hi], out=weighted[lo:hi], row_scale=scales[lo:hi])
            final_hidden_states.index_add_(0, top_x, weighted)
            return final_hidden_states.reshape(batch_size, sequence_length, hidden_dim), router_logits
        sel_host = selected_experts.cpu()  # one host sync per layer: the cache is driven from the host
        if tokens == 1:
            selected = sel_host[0].tolist()
            for (_layer_index, expert_idx), expert_layer in self.experts.load_experts(
                    *((self.layer_id, expert_idx) for expert_idx in sorted(set(selected))), unordered=True):
                k = selected.index(expert_idx)
                expert_layer(hidden_states, out=final_hidden_states, row_scale=routing_weights[0, k:k + 1],
                             accumulate=True)
            return final_hidden_states.reshape(batch_size, sequence_length, hidden_dim), router_logits

        # Several tokens: the (token, slot) pairs are grouped by expert on the host from that one copy, a single index
        # tensor goes back to the device, the rows of every expert are gathered at once and their weighted outputs
        # are added back with one index_add_ (reference :298-312 does a where / gather / index_add_ per expert; each
        # token receives the same two fp16 terms, and their sum does not depend on the order).
        flat = sel_host.reshape(-1).numpy()                     # pair p = token * top_k + slot
        order = np.argsort(flat, kind="stable")
        counts = np.bincount(flat, minlength=self.num_experts)
        starts = np.concatenate(([0], np.cumsum(counts)))
        order_dev = torch.from_numpy(order).to(hidden_states.device)
        top_x = torch.div(order_dev, self.top_k, rounding_mode="floor")
        scales = routing_weights.reshape(-1).index_select(0, order_dev)
        gathered = hidden_states.index_select(0, top_x)
        weighted = torch.empty_like(gathered)
        active_experts = [e for e in range(self.num_experts) if counts[e] > 0]
        for (_layer_index, expert_idx), expert_layer in self.experts.load_experts(
                *((self.layer_id, expert_idx) for expert_idx in active_experts), unordered=True):
            lo, hi = int(starts[expert_idx]), int(starts[expert_idx + 1])
            expert_layer(gathered[lo:hi], out=weighted[lo:hi], row_scale=scales[lo:hi])
        final_hidden_states.index_add_(0, top_x, weighted)
        return final_hidden_states.reshape(batch_size, sequence_length, hidden_dim), router_logits
