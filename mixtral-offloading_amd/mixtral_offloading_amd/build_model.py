"""Model assembly with the reference's entry points (``src/build_model.py``):
``OffloadConfig``, ``QuantConfig``, ``replace_attn_layers``, ``make_empty_expert``,
``build_model``.  Without a ``state_path`` the model gets seeded random weights of the
Mixtral architecture, quantised on the GPU (what the benchmark runs on); with one, the
expert and trunk tensors are read from the reference's safetensors shards."""
from __future__ import annotations

import copy
import json
import os
import typing as tp
from dataclasses import dataclass
from functools import cache

import torch
from torch import nn

from .custom_layers import HQQLinearTritonSavable, MixtralBLockSparseTop2MLP_HQQ, SparseMoeWrapper
from .expert_cache import ExpertCache
from .expert_wrapper import MixtralExpertWrapper
from .hqq_core import BaseQuantizeConfig, BitPack
from .packing import unpack_2bit_u8_common, unpack_3bit_i32_common, unpack_4bit_u8_common
from .mixtral_model import MixtralForCausalLM
from .utils import with_default_dtype


@dataclass(frozen=True)
class OffloadConfig:
    main_size: int
    offload_size: int
    buffer_size: int
    offload_per_layer: int


class QuantConfig:
    def __init__(self, ffn_config, attn_config):
        self.ffn_config = ffn_config
        self.attn_config = attn_config

    @cache
    def get_ffn_metas(self, hidden_dim: int, ffn_dim: int) -> tuple:
        return (HQQLinearTritonSavable.get_hqq_meta((hidden_dim, ffn_dim), self.ffn_config),
                HQQLinearTritonSavable.get_hqq_meta((ffn_dim, hidden_dim), self.ffn_config))


def mixtral_config(**overrides):
    """Mixtral-8x7B architecture (the reference fetches it by name, src/build_model.py:172)."""
    from transformers.models.mixtral.configuration_mixtral import MixtralConfig

    base = dict(vocab_size=32000, hidden_size=4096, intermediate_size=14336, num_hidden_layers=32,
                num_attention_heads=32, num_key_value_heads=8, hidden_act="silu", rms_norm_eps=1e-5,
                rope_theta=1e6, num_experts_per_tok=2, num_local_experts=8)
    base.update(overrides)
    cfg = MixtralConfig(**base)
    cfg.rope_theta = base["rope_theta"]
    return cfg


def default_quant_config() -> QuantConfig:
    """The repository's demo settings: attention 4-bit g64, experts 2-bit g16, 8-bit meta."""
    attn = BaseQuantizeConfig(nbits=4, group_size=64, quant_zero=True, quant_scale=True)
    ffn = BaseQuantizeConfig(nbits=2, group_size=16, quant_zero=True, quant_scale=True)
    return QuantConfig(ffn_config=ffn, attn_config=attn)


def replace_attn_layers(model, config, quant_config: QuantConfig, device: torch.device) -> None:
    """q/k/v/o become empty quantized linears, the router an fp16 linear (reference src/build_model.py:55-105)."""
    attn_quant_config = quant_config.attn_config
    hidden_size = config.hidden_size
    num_heads = config.num_attention_heads
    head_dim = hidden_size // num_heads
    num_key_value_heads = config.num_key_value_heads
    shapes = {"q_proj": (hidden_size, num_heads * head_dim), "k_proj": (hidden_size, num_key_value_heads * head_dim),
              "v_proj": (hidden_size, num_key_value_heads * head_dim), "o_proj": (num_heads * head_dim, hidden_size)}
    metas = {shape: HQQLinearTritonSavable.get_hqq_meta(shape, attn_quant_config) for shape in set(shapes.values())}
    for layer in model.model.layers:
        layer.block_sparse_moe.gate = nn.Linear(config.hidden_size, config.num_local_experts, dtype=torch.float16,
                                                device=device, bias=False)
        for name, shape in shapes.items():
            setattr(layer.self_attn, name, HQQLinearTritonSavable(None, attn_quant_config, meta=metas[shape]))


@cache
def get_default_ffn_quant_config(ffn_dim: int = 14336, hidden_dim: int = 4096):
    quant_config = BaseQuantizeConfig(nbits=2, group_size=16, quant_zero=True, quant_scale=True)
    meta1 = HQQLinearTritonSavable.get_hqq_meta((hidden_dim, ffn_dim), quant_config)
    meta2 = HQQLinearTritonSavable.get_hqq_meta((ffn_dim, hidden_dim), quant_config)
    return quant_config, meta1, meta2


def make_empty_expert(model_config, quant_config: QuantConfig) -> MixtralBLockSparseTop2MLP_HQQ:
    meta1, meta2 = quant_config.get_ffn_metas(model_config.hidden_size, model_config.intermediate_size)
    return MixtralBLockSparseTop2MLP_HQQ(model_config, quant_config.ffn_config, meta1, meta2)


def _quantize_linear(weight: torch.Tensor, quant_config) -> HQQLinearTritonSavable:
    lin = nn.Linear(weight.shape[1], weight.shape[0], bias=False, device=weight.device, dtype=torch.float16)
    lin.weight.data = weight
    return HQQLinearTritonSavable(lin, quant_config)


def _random_weight(shape, gen: torch.Generator, device) -> torch.Tensor:
    return (torch.randn(shape, device=device, generator=gen) * 0.02).half()


def make_random_expert(model_config, quant_config: QuantConfig, gen: torch.Generator, device,
                       fast: bool = True) -> MixtralBLockSparseTop2MLP_HQQ:
    """A seeded random expert, quantised on the GPU.  ``fast`` skips hqq's proximal refinement, which changes the
    values of the codes, not the speed or the layout of anything downstream."""
    cfg = {k: (dict(v) if isinstance(v, dict) else v) for k, v in quant_config.ffn_config.items()}
    if fast:
        cfg["weight_quant_params"]["optimize"] = False
    expert = make_empty_expert(model_config, quant_config)
    h, f = model_config.hidden_size, model_config.intermediate_size
    for name, shape in (("w1", (f, h)), ("w2", (h, f)), ("w3", (f, h))):
        q = _quantize_linear(_random_weight(shape, gen, device), cfg)
        tgt = getattr(expert, name)
        tgt.W_q, tgt.meta, tgt.bias, tgt.ready = q.W_q, q.meta, None, True
        tgt._desc_cache = None
    return expert


def checkpoint_layout(index: dict) -> str:
    """Code layout of a checkpoint directory, from its index: the reference's files carry no such entry and hold
    hqq's step layout; save_quantized_checkpoint records what it wrote."""
    layout = (index.get("metadata") or {}).get("layout", "hqq")
    if layout not in ("hqq", "kernel"):
        raise ValueError(f"unknown code layout {layout!r} in model.safetensors.index.json")
    return layout


def set_checkpoint_layout(module, layout: str) -> None:
    for sub in module.modules():
        if isinstance(sub, HQQLinearTritonSavable):
            sub.checkpoint_layout = layout


def make_and_load_expert_wrapper(config, quant_config: QuantConfig, states_dir: str, expert_uid: tuple,
                                 device: torch.device) -> MixtralExpertWrapper:
    """Reads one expert from the reference's safetensors shards (src/build_model.py:137-155)."""
    from safetensors.torch import load_file

    layer_idx, expert_idx = expert_uid
    with open(os.path.join(states_dir, "model.safetensors.index.json")) as f:
        module_idx = f"model.layers.{layer_idx}.block_sparse_moe.experts.{expert_idx}"
        index = json.load(f)
        state_fpath = index["weight_map"][f"{module_idx}.w1.W_q"]
    state_dict = load_file(os.path.join(states_dir, state_fpath), device=str(device))
    expert = make_empty_expert(config, quant_config)
    set_checkpoint_layout(expert, checkpoint_layout(index))
    expert.load_state_dict(state_dict, strict=True)
    return MixtralExpertWrapper(expert, device)


_STEP_PACK = {"4bit_u8": (unpack_4bit_u8_common, BitPack.pack_4bit_u8), "2bit_u8": (unpack_2bit_u8_common, BitPack.pack_2bit_u8),
              "3bit_32": (unpack_3bit_i32_common, BitPack.pack_3bit_32)}


def codes_in_checkpoint_layout(lin: HQQLinearTritonSavable) -> torch.Tensor:
    """The codes of a layer as hqq wrote them and as the reference's checkpoints hold them: the ``(N, K)`` codes viewed
    as ``(group_size, N*K/group_size)`` and packed in hqq's step layout (code rows one ``step`` apart share a byte or
    word).  It is the inverse of what ``repack`` does at load (reference src/custom_layers.py:41-47)."""
    meta = lin.meta
    unpack, pack = _STEP_PACK[meta["packing"]]
    n = int(meta["shape"][0])
    codes = unpack(lin.W_q)[:n]
    return pack(codes.reshape(int(meta["group_size"]), -1)).contiguous()


def iterate_experts(model) -> tp.Iterator[tp.Tuple[tp.Tuple[int, int], MixtralBLockSparseTop2MLP_HQQ]]:
    """Every registered expert, in uid order, as a module on the device.  All of them are views of one scratch slab
    that the next iteration overwrites (filled from the expert's pinned host copy, or from its device slot when it has none)."""
    cache_ = model.expert_cache
    scratch = MixtralExpertWrapper(copy.deepcopy(cache_.slots[0]._expert[0]), cache_.device)
    for uid, info in sorted(cache_.registered_experts.items()):
        scratch.storage.copy_(cache_.expert_bytes(uid).untyped_storage())
        yield uid, scratch._expert[0]


def save_quantized_checkpoint(model, state_path: str, layout: str = "hqq") -> None:
    """Writes the directory that ``build_model(..., state_path)`` reads (reference src/build_model.py:137-205):
    ``model.safetensors.index.json`` whose ``weight_map`` names, for every key, one of the safetensors files beside
    it -- one file for the trunk (embedding, norms, attention, routers, head) and one per expert, keys in the flat
    schema of ``HQQLinearTritonSavable`` (reference src/custom_layers.py:136-166).

    ``layout="hqq"`` stores the codes as the reference's checkpoints do (quantise-time shape, step layout), so the
    reference can read the directory as well; ``layout="kernel"`` stores them as they sit in memory, ``(N/f, K)``
    interleaved, which only this package reads (the index records the layout under ``metadata.layout``; a directory without that
    entry, like the reference's, is read as hqq's)."""
    from safetensors.torch import save_file

    assert layout in ("hqq", "kernel")
    os.makedirs(state_path, exist_ok=True)
    weight_map: tp.Dict[str, str] = {}

    def plain(state):
        return {k: torch.Tensor.as_subclass(v, torch.Tensor).detach().cpu().contiguous().clone() for k, v in state.items()}

    def linears_in_file_layout(module, state, prefix):
        if layout == "hqq":
            for name, sub in module.named_modules():
                if isinstance(sub, HQQLinearTritonSavable):
                    state[prefix + (name + "." if name else "") + "W_q"] = codes_in_checkpoint_layout(sub)
        return state

    def write(fname, state, index_prefix=""):
        save_file(plain(state), os.path.join(state_path, fname))
        weight_map.update({index_prefix + k: fname for k in state})

    write("trunk.safetensors", linears_in_file_layout(model, dict(model.state_dict()), ""))
    for (layer_idx, expert_idx), expert in iterate_experts(model):
        prefix = f"model.layers.{layer_idx}.block_sparse_moe.experts.{expert_idx}."
        # an expert's file holds the keys of the expert module itself (``w1.W_q`` ...): the reference hands the whole
        # file to ``expert.load_state_dict`` (src/build_model.py:151-153); only the index carries the full names
        write(f"expert-{layer_idx}-{expert_idx}.safetensors", linears_in_file_layout(expert, dict(expert.state_dict()), ""),
              index_prefix=prefix)
    with open(os.path.join(state_path, "model.safetensors.index.json"), "w") as f:
        json.dump({"metadata": {"layout": layout}, "weight_map": weight_map}, f)


def build_model(device: torch.device, quant_config: QuantConfig, offload_config: OffloadConfig,
                state_path: tp.Optional[str] = None, model_config=None, seed: int = 0, max_positions: int = 4096):
    """The reference's ``build_model(device, quant_config, offload_config, state_path)`` (src/build_model.py:166-241).

    ``state_path=None`` builds the same model with seeded random weights (no checkpoint, no network)."""
    device = torch.device(device)
    model_config = model_config or mixtral_config()
    gen = torch.Generator(device=device).manual_seed(seed)

    template = make_random_expert(model_config, quant_config, gen, device)

    def _make_module():
        # device slots only need the right shapes; their contents are overwritten when an expert moves in
        return MixtralExpertWrapper(copy.deepcopy(template), device=device)

    with with_default_dtype(torch.float16):
        model = MixtralForCausalLM(model_config, device, max_positions=max_positions)
    replace_attn_layers(model, model_config, quant_config, device)

    if state_path is not None:
        from safetensors.torch import load_file

        with open(os.path.join(state_path, "model.safetensors.index.json")) as f:
            index = json.load(f)
        weight_map = index["weight_map"]
        set_checkpoint_layout(model, checkpoint_layout(index))
        trunk = load_file(os.path.join(state_path, weight_map["model.embed_tokens.weight"]), device=str(device))
        model.load_state_dict(trunk, strict=True)
    else:
        attn_cfg = {k: (dict(v) if isinstance(v, dict) else v) for k, v in quant_config.attn_config.items()}
        attn_cfg["weight_quant_params"]["optimize"] = False
        for layer in model.model.layers:
            for name in ("q_proj", "k_proj", "v_proj", "o_proj"):
                tgt = getattr(layer.self_attn, name)
                n, k = int(tgt.meta["shape"][0]), int(tgt.meta["shape"][1])
                q = _quantize_linear(_random_weight((n, k), gen, device), attn_cfg)
                tgt.W_q, tgt.meta, tgt.bias, tgt.ready = q.W_q, q.meta, None, True
                tgt._desc_cache = None
            layer.block_sparse_moe.gate.weight.data = _random_weight(layer.block_sparse_moe.gate.weight.shape, gen, device)
        model.model.embed_tokens.weight.data = _random_weight(model.model.embed_tokens.weight.shape, gen, device)
        model.lm_head.weight.data = _random_weight(model.lm_head.weight.shape, gen, device)

    expert_cache = ExpertCache(make_module=_make_module, main_size=offload_config.main_size,
                               offload_size=offload_config.offload_size, buffer_size=offload_config.buffer_size)
    for layer_idx in range(model_config.num_hidden_layers):
        curr_layer = model.model.layers[layer_idx]
        curr_layer.block_sparse_moe = SparseMoeWrapper(model_config, layer_idx, curr_layer.block_sparse_moe.gate,
                                                       expert_cache)
        for expert_idx in range(model_config.num_local_experts):
            do_offload = expert_idx < offload_config.offload_per_layer
            if state_path is not None:
                wrapper = make_and_load_expert_wrapper(model_config, quant_config, state_path,
                                                       (layer_idx, expert_idx), device)
            else:
                wrapper = MixtralExpertWrapper(make_random_expert(model_config, quant_config, gen, device), device)
            expert_cache.add_expert(uid=(layer_idx, expert_idx), module=wrapper, eviction_group=layer_idx,
                                    offload=do_offload)
            del wrapper
    torch.cuda.synchronize(device)
    model.expert_cache = expert_cache
    return model
