"""Minimal Mixtral decoder used as the harness around the quantized-linear hot path.

The reference builds on HF ``MixtralForCausalLM`` (transformers 4.36.1,
``src/build_model.py:182-190``); this is the same architecture written with plain
torch ops -- RMSNorm, rotary embedding (theta 1e6), grouped-query attention with a
KV cache, sparse top-2 MoE -- with the same module names (``model.layers[i].self_attn.q_proj``,
``.block_sparse_moe.gate`` ...) so that ``replace_attn_layers`` and ``build_model``
read like the reference.  The four attention projections and the expert FFNs are the
HIP library's kernels; everything else here is plumbing, not the measured path."""
from __future__ import annotations

import math
import warnings
from typing import Optional

import torch
from torch import nn
from torch.nn import functional as F


class RMSNorm(nn.Module):
    def __init__(self, hidden_size, eps=1e-5, device=None):
        super().__init__()
        self.weight = nn.Parameter(torch.ones(hidden_size, dtype=torch.float16, device=device), requires_grad=False)
        self.variance_epsilon = eps

    def forward(self, x, delta=None):
        """``weight * rmsnorm(x)``; with ``delta`` (device path only) ``x += delta`` in place first."""
        if x.is_cuda and x.dtype == torch.float16 and x.dim() == 2 and x.is_contiguous():
            from . import hip_kernels

            return hip_kernels.add_rmsnorm_rows(x, delta, self.weight, self.variance_epsilon)
        if delta is not None:
            x.add_(delta)
        xf = x.float()
        xf = xf * torch.rsqrt(xf.pow(2).mean(-1, keepdim=True) + self.variance_epsilon)
        return self.weight * xf.to(x.dtype)


class Rotary:
    def __init__(self, head_dim, max_positions, theta, device):
        inv_freq = 1.0 / (theta ** (torch.arange(0, head_dim, 2, dtype=torch.float32, device=device) / head_dim))
        t = torch.arange(max_positions, dtype=torch.float32, device=device)
        freqs = torch.outer(t, inv_freq)
        emb = torch.cat((freqs, freqs), dim=-1)
        self.cos, self.sin = emb.cos().half(), emb.sin().half()

    @staticmethod
    def rotate_half(x):
        h = x.shape[-1] // 2
        return torch.cat((-x[..., h:], x[..., :h]), dim=-1)

    def causal_bias(self, T, start, g):
        """fp32 (g * T, start + T): 0 where row r (token r % T at position start + r % T) may attend, -inf elsewhere.
        The last one made is kept while a pass runs (its layers all ask for the same one); forward_tokens drops it
        at the end of the pass, a long prompt's bias being hundreds of megabytes."""
        key = (T, start, g)
        if getattr(self, "_bias_key", None) != key:
            dev = self.cos.device
            tok = torch.arange(T, device=dev).repeat(g)  # row -> token index
            allowed = torch.arange(start + T, device=dev)[None, :] <= (start + tok)[:, None]
            self._bias = torch.zeros(allowed.shape, dtype=torch.float32, device=dev).masked_fill_(~allowed, float("-inf"))
            self._bias_key = key
        return self._bias

    def drop_causal_bias(self):
        self._bias, self._bias_key = None, None

    def apply(self, q, k, positions):
        cos, sin = self.cos[positions][:, None, :], self.sin[positions][:, None, :]  # (T, 1, hd)
        return q * cos + self.rotate_half(q) * sin, k * cos + self.rotate_half(k) * sin


class Attention(nn.Module):
    def __init__(self, config, device):
        super().__init__()
        self.num_heads = config.num_attention_heads
        self.num_kv_heads = config.num_key_value_heads
        self.head_dim = config.hidden_size // config.num_attention_heads
        hs = config.hidden_size
        mk = dict(bias=False, dtype=torch.float16, device=device)
        # fp16 placeholders; replace_attn_layers swaps in the quantized linears
        self.q_proj = nn.Linear(hs, self.num_heads * self.head_dim, **mk)
        self.k_proj = nn.Linear(hs, self.num_kv_heads * self.head_dim, **mk)
        self.v_proj = nn.Linear(hs, self.num_kv_heads * self.head_dim, **mk)
        self.o_proj = nn.Linear(self.num_heads * self.head_dim, hs, **mk)

    def forward(self, x, rotary: Rotary, cache_k, cache_v, start: int):
        """x (T, hidden) for one sequence; cache_k / cache_v (kv_heads, max_len, hd); start = tokens already cached."""
        T = x.shape[0]
        q = self.q_proj(x).view(T, self.num_heads, self.head_dim)
        k = self.k_proj(x).view(T, self.num_kv_heads, self.head_dim)
        v = self.v_proj(x).view(T, self.num_kv_heads, self.head_dim)
        g = self.num_heads // self.num_kv_heads
        if x.is_cuda and q.dtype == torch.float16 and cache_k.is_contiguous() and cache_v.is_contiguous():
            # rope of q (in place) and k, and the cache append, in one launch
            from . import hip_kernels

            hip_kernels.rope_append_rows(q, k, v, rotary.cos, rotary.sin, start, cache_k, cache_v)
        else:
            positions = torch.arange(start, start + T, device=x.device)
            q, k = rotary.apply(q, k, positions)
            cache_k[:, start:start + T] = k.transpose(0, 1)
            cache_v[:, start:start + T] = v.transpose(0, 1)
        keys, values = cache_k[:, :start + T], cache_v[:, :start + T]  # (kv, L, hd)
        qh = q.transpose(0, 1).reshape(self.num_kv_heads, g * T, self.head_dim)  # heads of a kv group, then tokens
        scores = torch.bmm(qh, keys.transpose(1, 2)).float()  # (kv, g*T, L)
        # scaled, and every position after a row's own token at -inf (the same table for every layer of a pass)
        scores = torch.add(rotary.causal_bias(T, start, g), scores, alpha=1.0 / math.sqrt(self.head_dim))
        probs = torch.softmax(scores, dim=-1).to(x.dtype)
        out = torch.bmm(probs, values)  # (kv, g*T, hd)
        out = out.view(self.num_kv_heads, g, T, self.head_dim).permute(2, 0, 1, 3).reshape(T, -1)
        return self.o_proj(out)


class MoePlaceholder(nn.Module):
    """Holds the router until build_model installs the SparseMoeWrapper (reference src/build_model.py:212-217)."""

    def __init__(self, config, device):
        super().__init__()
        self.gate = nn.Linear(config.hidden_size, config.num_local_experts, bias=False, dtype=torch.float16,
                              device=device)


class DecoderLayer(nn.Module):
    def __init__(self, config, device):
        super().__init__()
        self.input_layernorm = RMSNorm(config.hidden_size, config.rms_norm_eps, device)
        self.self_attn = Attention(config, device)
        self.post_attention_layernorm = RMSNorm(config.hidden_size, config.rms_norm_eps, device)
        self.block_sparse_moe = MoePlaceholder(config, device)

    def forward(self, x, rotary, cache_k, cache_v, start, inplace=False):
        """x (T, hidden).  With ``inplace`` the residual stream is updated in x itself (the caller owns it)."""
        if x.is_cuda and x.dtype == torch.float16 and x.is_contiguous():
            if not inplace:
                x = x.clone()
            attn = self.self_attn(self.input_layernorm(x), rotary, cache_k, cache_v, start)
            moe_out, _ = self.block_sparse_moe(self.post_attention_layernorm(x, attn)[None])  # x += attn, then the norm
            return x.add_(moe_out[0])
        x = x + self.self_attn(self.input_layernorm(x), rotary, cache_k, cache_v, start)
        moe_out, _ = self.block_sparse_moe(self.post_attention_layernorm(x)[None])
        return x + moe_out[0]


class MixtralModel(nn.Module):
    def __init__(self, config, device):
        super().__init__()
        self.embed_tokens = nn.Embedding(config.vocab_size, config.hidden_size, dtype=torch.float16, device=device)
        self.layers = nn.ModuleList([DecoderLayer(config, device) for _ in range(config.num_hidden_layers)])
        self.norm = RMSNorm(config.hidden_size, config.rms_norm_eps, device)


class DecodeGraph:
    """One batch-1 decode step of the whole model as a replayable HIP graph.

    Usable when every expert of every layer is resident on the device: the router's choice then stays on the device
    (``hip_kernels.router_top2`` writes the two expert indices, ``expert_ffn_indexed`` reads them), the position is a
    device tensor, attention runs over the whole cache with the positions past the current one masked, and the next
    token is written back into the step's own input -- nothing in a step waits for the host.  The reference drives
    the same step from Python with one host synchronisation per MoE layer and two more per active expert
    (src/custom_layers.py:292-302)."""

    def __init__(self, model: "MixtralForCausalLM", max_len: int):
        from . import hip_kernels

        self.model, self.max_len = model, max_len
        cfg, dev = model.config, model.device
        # the attention kernel reads the rope tables at the device-side position, which only the cache length bounds
        if max_len > model.rotary.cos.shape[0]:
            raise ValueError(f"a cache of {max_len} positions exceeds the rope tables ({model.rotary.cos.shape[0]} "
                             "positions): build the model with a larger max_positions")
        self.tables = []
        for layer_id, layer in enumerate(model.model.layers):
            mods = layer.block_sparse_moe.experts.resident_group(layer_id)
            if mods is None:
                raise RuntimeError("the graph path needs every expert of every layer resident on the device")
            self.tables.append(hip_kernels.ExpertTable(
                [(m._expert[0].w1._desc(), m._expert[0].w2._desc(), m._expert[0].w3._desc()) for m in mods]))
        # the two active experts in two launches, q / k / v in one, where the shapes allow
        self.pair = all(hip_kernels.expert_pair_supported(t) for t in self.tables)
        self.routed = all(hip_kernels.moe_pair_routed_supported(t, cfg.hidden_size, cfg.num_local_experts) for t in self.tables)
        self.qkv = [hip_kernels.LinearGroup([p._desc() for p in (l.self_attn.q_proj, l.self_attn.k_proj, l.self_attn.v_proj)])
                    for l in model.model.layers]
        # norm + q/k/v, attention and o_proj as ONE launch (model.chain_attention = True).  Off by default here: in a
        # replayed graph the three launches follow each other without host gaps and the chained launch measured
        # 27 us per layer against their 25 (its two hand-overs through memory cost what two launch boundaries do, and
        # the heads run slower while the output projection's weights stream in beside them)
        self.chain = [hip_kernels.AttentionChain(g, l.self_attn.o_proj._desc()) for g, l in zip(self.qkv, model.model.layers)]
        self.cache = model.new_cache(max_len)
        mk = dict(device=dev)
        self.tok = torch.zeros(1, dtype=torch.int64, **mk)
        self.pos = torch.zeros(1, dtype=torch.int64, **mk)
        self.arange = torch.arange(max_len, **mk)
        self.x = torch.zeros((1, cfg.hidden_size), dtype=torch.float16, **mk)
        self.x2 = torch.zeros_like(self.x)
        self.xn = torch.zeros_like(self.x)
        self.moe = torch.zeros_like(self.x)
        self.att = torch.zeros((1, cfg.num_attention_heads * (cfg.hidden_size // cfg.num_attention_heads)), dtype=torch.float16, **mk)
        self.sel = torch.zeros(2, dtype=torch.int32, **mk)
        self.rw = torch.zeros(2, dtype=torch.float16, **mk)
        self.logits = torch.zeros((1, cfg.vocab_size), dtype=torch.float16, **mk)
        self.graph = None
        self._host_pos = 0  # host mirror of ``pos``: the cache capacity is checked without reading the device

    @torch.inference_mode()
    def _step(self):
        from . import hip_kernels

        m, cfg = self.model, self.model.config
        H, KV = cfg.num_attention_heads, cfg.num_key_value_heads
        hd = cfg.hidden_size // H
        g = H // KV
        eps = cfg.rms_norm_eps
        x, spare = self.x, self.x2  # the residual stream alternates between two buffers where the norm is fused
        x.copy_(m.model.embed_tokens(self.tok))
        delta = None
        chained = getattr(m, "chain_attention", False)
        for layer, (ck, cv), table, qkv, chain in zip(m.model.layers, self.cache, self.tables, self.qkv, self.chain):
            attn = layer.self_attn
            attn_out = None
            if chained and chain.supported:
                attn_out = chain(x, delta, layer.input_layernorm.weight, eps, spare, m.rotary.cos, m.rotary.sin, self.pos, ck, cv)
            if attn_out is not None:
                x, spare = spare, x
            else:
                if qkv.supported:
                    # residual add, input norm and the three projections in one launch
                    q, k, v = hip_kernels.matmul_group_norm(qkv, x, delta, layer.input_layernorm.weight, eps, spare)
                    x, spare = spare, x
                else:
                    hip_kernels.add_rmsnorm(x, delta, layer.input_layernorm.weight, eps, self.xn)
                    q, k, v = attn.q_proj(self.xn), attn.k_proj(self.xn), attn.v_proj(self.xn)
                out = hip_kernels.attention_decode(q, k, v, m.rotary.cos, m.rotary.sin, self.pos, ck, cv, self.att)
                attn_out = attn.o_proj(out)
            if self.routed:
                # post-attention norm, router and both experts in two launches
                hip_kernels.moe_pair_routed(table, x, attn_out, layer.post_attention_layernorm.weight, eps, spare,
                                            layer.block_sparse_moe.gate.weight, self.sel, self.rw, self.moe)
                x, spare = spare, x
                delta = self.moe
                continue
            hip_kernels.add_rmsnorm_router(x, attn_out, layer.post_attention_layernorm.weight, eps, self.xn,
                                           layer.block_sparse_moe.gate.weight, self.sel, self.rw)
            if self.pair:
                hip_kernels.expert_pair_ffn_indexed(table, self.sel, self.xn, self.moe, self.rw)
            else:
                hip_kernels.expert_ffn_indexed(table, self.sel[0:1], self.xn, self.moe, row_scale=self.rw[0:1])
                hip_kernels.expert_ffn_indexed(table, self.sel[1:2], self.xn, self.moe, row_scale=self.rw[1:2], accumulate=True)
            delta = self.moe
        hip_kernels.add_rmsnorm(x, delta, m.model.norm.weight, eps, self.xn)
        self.logits.copy_(m.lm_head(self.xn))
        self.tok.copy_(self.logits.argmax(-1))
        self.pos.add_(1)

    def capture(self):
        """Warm up on a side stream (workspaces and allocator pools get their final size), then record the step."""
        if self._host_pos + 3 > self.max_len:  # two warm-up steps and the recorded one each write one position further
            raise ValueError(f"capture at position {self._host_pos} needs a cache of {self._host_pos + 3} positions, "
                             f"this one holds {self.max_len}")
        keep = (self.tok.clone(), self.pos.clone())
        side = torch.cuda.Stream(device=self.model.device)
        side.wait_stream(torch.cuda.current_stream(self.model.device))
        with torch.cuda.stream(side):
            for _ in range(2):
                self._step()
        torch.cuda.current_stream(self.model.device).wait_stream(side)
        self.graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(self.graph):
            self._step()
        # the warm-up and the capture wrote cache entries at and after `pos`: every one is rewritten by the real
        # steps before a query can see it (positions past the current one are masked)
        self.tok.copy_(keep[0])
        self.pos.copy_(keep[1])

    @torch.inference_mode()
    def prefill(self, prompt_ids: torch.Tensor) -> torch.Tensor:
        """Runs the prompt through the eager path into this graph's cache; returns the first generated token."""
        if prompt_ids.numel() >= self.max_len:
            raise ValueError(f"a prompt of {prompt_ids.numel()} tokens does not fit a cache of {self.max_len} positions")
        logits = self.model.forward(prompt_ids, self.cache, 0)
        tok = logits[-1].argmax()
        self.tok.copy_(tok.view(1))
        self.pos.fill_(prompt_ids.numel())
        self._host_pos = prompt_ids.numel()
        return tok

    def step(self):
        """One decode step; afterwards ``self.tok`` holds the next token and ``self.logits`` its logits."""
        if self._host_pos >= self.max_len:
            raise ValueError(f"the cache of {self.max_len} positions is full")
        self._host_pos += 1
        if self.graph is None:
            self._step()
        else:
            self.graph.replay()


class MixtralForCausalLM(nn.Module):
    def __init__(self, config, device, max_positions: int = 4096):
        super().__init__()
        self.config = config
        self.model = MixtralModel(config, device)
        self.lm_head = nn.Linear(config.hidden_size, config.vocab_size, bias=False, dtype=torch.float16, device=device)
        head_dim = config.hidden_size // config.num_attention_heads
        self.rotary = Rotary(head_dim, max_positions, config.rope_theta, device)
        self.max_positions = max_positions
        self.device = device

    def new_cache(self, max_len: Optional[int] = None):
        cfg = self.config
        hd = cfg.hidden_size // cfg.num_attention_heads
        L = max_len or self.max_positions
        if L > self.rotary.cos.shape[0]:
            raise ValueError(f"a cache of {L} positions exceeds the rope tables ({self.rotary.cos.shape[0]} positions)")
        mk = dict(dtype=torch.float16, device=self.device)
        return [(torch.zeros((cfg.num_key_value_heads, L, hd), **mk), torch.zeros((cfg.num_key_value_heads, L, hd), **mk))
                for _ in range(cfg.num_hidden_layers)]

    def _token_state(self):
        """Buffers and grouped projections of the single-token step, made once."""
        st = getattr(self, "_token_bufs", None)
        if st is None:
            from . import hip_kernels

            cfg, mk = self.config, dict(device=self.device)
            row = lambda n: torch.zeros((1, n), dtype=torch.float16, **mk)  # noqa: E731
            st = dict(x=row(cfg.hidden_size), x2=row(cfg.hidden_size), xn=row(cfg.hidden_size), moe=row(cfg.hidden_size),
                      att=row(cfg.hidden_size), sel4=torch.zeros(4, dtype=torch.int32, **mk),
                      guess_w=torch.zeros(2, dtype=torch.float16, **mk),
                      rw=torch.zeros(2, dtype=torch.float16, **mk), pos=torch.zeros(1, dtype=torch.int64, **mk),
                      qkv=[hip_kernels.LinearGroup([p._desc() for p in (l.self_attn.q_proj, l.self_attn.k_proj, l.self_attn.v_proj)])
                           for l in self.model.layers])
            st["sel"], st["guess"] = st["sel4"][0:2], st["sel4"][2:4]  # one copy to the host brings both
            st["chain"] = [None] * len(self.model.layers)
            self._token_bufs = st
        return st

    @torch.inference_mode()
    def forward_token(self, token: torch.Tensor, cache, start: int) -> torch.Tensor:
        """One new token through the launches of the graph step (grouped q/k/v with the norm folded in, the attention
        kernel, norm + router in one launch, the fused expert FFN), but with the experts picked up from the expert cache
        by the host: one synchronisation per layer, which is what lets experts be offloaded.  Returns logits (1, vocab)."""
        from . import hip_kernels

        cfg, st = self.config, self._token_state()
        if cfg.num_experts_per_tok != 2 or not (0 <= start < min(cache[0][0].shape[1], self.rotary.cos.shape[0])):
            raise ValueError("the single-token step takes top-2 routing and a position inside the cache")
        eps = cfg.rms_norm_eps
        x, spare, xn, moe = st["x"], st["x2"], st["xn"], st["moe"]
        # speculative expert loads (self.speculate, off by default): the next layer's experts are guessed one layer ahead
        speculate = bool(getattr(self, "speculate", False))
        trace = getattr(self, "attention_trace", None)  # a list: (layer, start event, end event) around each attention
        # norm + q/k/v, attention and o_proj as one launch where it fits: on by default here, where every launch costs
        # host time (all experts resident: 197 -> 209 tok/s)
        chained = getattr(self, "chain_attention", True)
        st["pos"].fill_(start)
        x.copy_(self.model.embed_tokens(token.view(1)))
        delta = None
        for i, (layer, (ck, cv)) in enumerate(zip(self.model.layers, cache)):
            attn = layer.self_attn
            qkv = st["qkv"][i]
            if qkv.descs[0] is not attn.q_proj._desc():  # the layer's tensors were replaced since the group was made
                qkv = st["qkv"][i] = hip_kernels.LinearGroup([p._desc() for p in (attn.q_proj, attn.k_proj, attn.v_proj)])
                st["chain"][i] = None
            chain = st["chain"][i]
            if chain is None or chain.o is not attn.o_proj._desc():
                chain = st["chain"][i] = hip_kernels.AttentionChain(qkv, attn.o_proj._desc())
            if trace is not None:  # the interval of the layer's attention part (one launch when chained, else the kernel)
                trace.append((i, torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)))
            attn_out = None
            if chained and chain.supported:
                if trace is not None:
                    trace[-1][1].record()
                attn_out = chain(x, delta, layer.input_layernorm.weight, eps, spare, self.rotary.cos, self.rotary.sin,
                                 st["pos"], ck, cv)
            if attn_out is not None:
                x, spare = spare, x
                if trace is not None:
                    trace[-1][2].record()
            else:
                if qkv.supported:
                    q, k, v = hip_kernels.matmul_group_norm(qkv, x, delta, layer.input_layernorm.weight, eps, spare)
                    x, spare = spare, x
                else:
                    hip_kernels.add_rmsnorm(x, delta, layer.input_layernorm.weight, eps, xn)
                    q, k, v = attn.q_proj(xn), attn.k_proj(xn), attn.v_proj(xn)
                if trace is not None:
                    trace[-1][1].record()
                out = hip_kernels.attention_decode(q, k, v, self.rotary.cos, self.rotary.sin, st["pos"], ck, cv, st["att"])
                if trace is not None:
                    trace[-1][2].record()
                attn_out = attn.o_proj(out)
            moe_block = layer.block_sparse_moe
            hip_kernels.add_rmsnorm_router(x, attn_out, layer.post_attention_layernorm.weight, eps, xn,
                                           moe_block.gate.weight, st["sel"], st["rw"])
            nxt = self.model.layers[i + 1].block_sparse_moe if speculate and i + 1 < len(self.model.layers) else None
            if nxt is not None:
                # the guess for the next layer: its router applied to this layer's post-attention state
                hip_kernels.router_top2(xn, nxt.gate.weight, st["guess"], st["guess_w"])
                both = st["sel4"].cpu().tolist()  # the layer's one synchronisation
                moe_block.forward_routed(xn, st["sel"], st["rw"], moe, chosen=both[:2])
                # started now, before the host goes on to the next layer's attention: the copies overlap it
                nxt.experts.prefetch(*((nxt.layer_id, e) for e in sorted(set(both[2:]))))
            else:
                moe_block.forward_routed(xn, st["sel"], st["rw"], moe)
            delta = moe
        hip_kernels.add_rmsnorm(x, delta, self.model.norm.weight, eps, xn)
        return self.lm_head(xn)

    def _token_step_ok(self, cache) -> bool:
        cfg = self.config
        hd = cfg.hidden_size // cfg.num_attention_heads
        return (cfg.num_experts_per_tok == 2 and 2 <= cfg.num_local_experts <= 16 and hd in (64, 128)
                and cfg.hidden_size % 8 == 0 and hasattr(self.model.layers[0].block_sparse_moe, "forward_routed")
                and cache[0][0].is_contiguous() and cache[0][0].shape[1] <= 16000)

    @torch.inference_mode()
    def forward(self, input_ids: torch.Tensor, cache, start: int) -> torch.Tensor:
        """input_ids (T,), one sequence; returns logits (T, vocab)."""
        if input_ids.numel() == 1 and self._token_step_ok(cache):
            return self.forward_token(input_ids, cache, start)
        return self.forward_tokens(input_ids, cache, start)

    @torch.inference_mode()
    def forward_tokens(self, input_ids: torch.Tensor, cache, start: int) -> torch.Tensor:
        """Any number of tokens of one sequence, layer by layer with torch ops around the quantized linears."""
        x = self.model.embed_tokens(input_ids)  # a new tensor: the layers update it in place
        for layer, (ck, cv) in zip(self.model.layers, cache):
            x = layer(x, self.rotary, ck, cv, start, inplace=True)
        self.rotary.drop_causal_bias()
        return self.lm_head(self.model.norm(x))

    @torch.inference_mode()
    def generate_graph(self, prompt_ids: torch.Tensor, max_new_tokens: int, decode: Optional[DecodeGraph] = None):
        """Greedy decoding, batch 1, with the decode steps replayed from a HIP graph (all experts resident)."""
        total = prompt_ids.numel() + max_new_tokens + 2  # the warm-up of the capture writes two positions ahead
        if decode is None or decode.max_len < total:
            decode = DecodeGraph(self, total)
        out = [decode.prefill(prompt_ids).view(1)]
        if decode.graph is None:
            decode.capture()
        for _ in range(max_new_tokens - 1):
            decode.step()
            out.append(decode.tok.clone())
        return torch.cat(out), decode

    @torch.inference_mode()
    def generate(self, prompt_ids: torch.Tensor, max_new_tokens: int, cache=None):
        """Greedy decoding, batch 1; returns the generated ids (max_new_tokens,)."""
        from . import hip_kernels
        own_cache = cache is None
        cache = cache or self.new_cache(prompt_ids.numel() + max_new_tokens)
        logits = self.forward(prompt_ids, cache, 0)
        tok = logits[-1].argmax()
        out = [tok]
        pos = prompt_ids.numel()
        for _ in range(max_new_tokens - 1):
            logits = self.forward(tok.view(1), cache, pos)
            tok = logits[-1].argmax()
            out.append(tok)
            pos += 1
        ids = torch.stack(out)
        # The chained attention launch hands results from block to block inside one grid and assumes that workgroups
        # start in index order; a block whose bounded wait ran out sets an error word and carries on with whatever it
        # read.  That never happened in any run, but tokens and cache would be wrong if it did: check once per call,
        # and if the word is set, clear it, stop chaining for this model and decode again with the three launches.
        if getattr(self, "chain_attention", True) and hip_kernels.attention_chain_error(prompt_ids.device, clear=True):
            warnings.warn("a chained attention launch gave up a wait; decoding again without chaining")
            self.chain_attention = False
            return self.generate(prompt_ids, max_new_tokens, None if own_cache else cache)
        return ids
