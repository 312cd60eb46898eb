"""One contiguous slab per expert, so that moving an expert is one copy.

Same role and surface as the reference's ``MixtralExpertWrapper``
(``src/expert_wrapper.py``): every tensor of ``w1``, ``w2``, ``w3`` is
re-homed into a single ``torch.UntypedStorage`` (``.storage``) in the
reference's order -- sorted keys, i.e. per layer ``W_q``, ``bias``,
``meta.meta_scale.{scale,zero}``, ``meta.meta_zero.{scale,zero}``,
``meta.scale_q``, ``meta.zero_q`` -- and the modules are re-pointed at views
of it.  One difference: every tensor starts at a multiple of 256 bytes (the
reference packs them back to back, ``src/expert_wrapper.py:50-57``, which
leaves ``w2.W_q`` at an offset of 4 mod 16 and rules out 128-bit loads)."""
from __future__ import annotations

import typing as tp

import torch
from torch import nn

from .packing import PackedTensor
from .utils import nested_flatten, nested_pack

SLAB_ALIGN = 256


def _align(n: int) -> int:
    return (n + SLAB_ALIGN - 1) // SLAB_ALIGN * SLAB_ALIGN


class MixtralExpertWrapper(nn.Module):
    def __init__(self, expert_module: tp.Any, device: torch.device):
        super().__init__()
        expert_module, self.storage = self.replace_layer_storage(expert_module, device)
        self._expert = [expert_module]  # kept out of nn.Module registration: the slab is the only state
        self.expert_module = lambda *args, **kwargs: self._expert[0](*args, **kwargs)
        self._register_state_dict_hook(self._add_storage_to_state_dict_hook)
        self._register_load_state_dict_pre_hook(self._load_storage_from_state_dict_hook)

    @staticmethod
    def _add_storage_to_state_dict_hook(self, state_dict, prefix, local_metadata):
        state_dict[prefix + "storage"] = torch.as_tensor(self.storage, dtype=torch.uint8)
        return state_dict

    def _load_storage_from_state_dict_hook(self, state_dict, prefix, local_metadata, strict, missing_keys,
                                           unexpected_keys, error_msgs):
        self.storage.copy_(state_dict.pop(prefix + "storage").untyped_storage())

    def forward(self, *args, **kwargs):
        return self.expert_module(*args, **kwargs)

    @staticmethod
    def slab_layout(layer: tp.Any):
        """([(offset, nbytes)] per tensor in flatten order, total bytes)."""
        state = MixtralExpertWrapper._state_of(layer)
        offsets, total = [], 0
        for x in nested_flatten(state):
            if isinstance(x, torch.Tensor):
                offsets.append((total, x.nbytes))
                total = _align(total + x.nbytes)
        return offsets, total

    @staticmethod
    def _state_of(layer):
        return {f"w{i}": {"W_q": getattr(layer, f"w{i}").W_q, "meta": getattr(layer, f"w{i}").meta,
                          "bias": getattr(layer, f"w{i}").bias} for i in range(1, 4)}

    @staticmethod
    def replace_layer_storage(layer: tp.Any, device: torch.device):
        state = MixtralExpertWrapper._state_of(layer)
        offsets, total = MixtralExpertWrapper.slab_layout(layer)
        storage = torch.UntypedStorage(total, device=device)
        whole = torch.as_tensor(storage, dtype=torch.uint8, device=device)
        flat, i = [], 0
        for x in nested_flatten(state):
            if not isinstance(x, torch.Tensor):
                flat.append(x)
                continue
            start, nbytes = offsets[i]
            i += 1
            view = whole[start:start + nbytes].view(x.dtype).view(x.shape)
            view.copy_(torch.Tensor.as_subclass(x, torch.Tensor))
            assert view.data_ptr() == storage.data_ptr() + start
            flat.append(PackedTensor(view) if isinstance(x, PackedTensor) else view)
        packed = nested_pack(flat, state)
        for name, st in packed.items():
            sub = getattr(layer, name)
            sub.W_q, sub.meta, sub.bias = st["W_q"], st["meta"], st["bias"]
            sub._desc_cache = None
        return layer, storage
