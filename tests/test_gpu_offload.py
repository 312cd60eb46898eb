"""GPU tests of the expert slab, the expert cache with side-stream loads, the MoE block and the decoder harness."""
import numpy as np
import pytest
import torch

from oracle import hqq_oracle as o

pytestmark = pytest.mark.gpu


def _small_setup(layers=2, hidden=256, ffn=512, experts=8, vocab=128, offload_per_layer=6, main_per_layer=2,
                 buffers=2, seed=0, ffn_bits=2, heads=4, kv_heads=2):
    from mixtral_offloading_amd import build_model as bm
    from mixtral_offloading_amd.hqq_core import BaseQuantizeConfig
    cfg = bm.mixtral_config(hidden_size=hidden, intermediate_size=ffn, num_hidden_layers=layers, num_attention_heads=heads,
                            num_key_value_heads=kv_heads, vocab_size=vocab, num_local_experts=experts)
    off = bm.OffloadConfig(main_size=layers * main_per_layer, offload_size=layers * offload_per_layer,
                           buffer_size=buffers, offload_per_layer=offload_per_layer)
    qc = bm.default_quant_config()
    if ffn_bits != 2:
        qc = bm.QuantConfig(ffn_config=BaseQuantizeConfig(nbits=ffn_bits, group_size=64, quant_zero=True, quant_scale=True),
                            attn_config=qc.attn_config)
    model = bm.build_model(torch.device("cuda:0"), qc, off, model_config=cfg, seed=seed, max_positions=256)
    return model, cfg


def _layer_to_numpy(lin):
    m = lin.meta
    d = {"nbits": m["nbits"], "group_size": m["group_size"], "shape": (int(m["shape"][0]), int(m["shape"][1])),
         "quant_scale": True, "quant_zero": True,
         "W_q": torch.Tensor.as_subclass(lin.W_q, torch.Tensor).cpu().numpy(),
         "scale_q": m["scale_q"].cpu().numpy(), "zero_q": m["zero_q"].cpu().numpy(),
         "meta_scale": {"scale": m["meta_scale"]["scale"].cpu().numpy(), "zero": m["meta_scale"]["zero"].cpu().numpy()},
         "meta_zero": {"scale": m["meta_zero"]["scale"].cpu().numpy().reshape(()),
                       "zero": m["meta_zero"]["zero"].cpu().numpy().reshape(())}}
    return d


def test_slab_wrapper_keeps_results_and_aligns_tensors():
    from mixtral_offloading_amd import build_model as bm
    from mixtral_offloading_amd.expert_wrapper import MixtralExpertWrapper, SLAB_ALIGN
    cfg = bm.mixtral_config(hidden_size=256, intermediate_size=512, num_hidden_layers=1)
    qc = bm.default_quant_config()
    gen = torch.Generator(device="cuda").manual_seed(3)
    expert = bm.make_random_expert(cfg, qc, gen, torch.device("cuda:0"))
    x = torch.randn((3, 256), device="cuda", generator=gen).half()
    before = expert(x).clone()
    ptr_before = expert.w1.W_q.data_ptr()
    wrapped = MixtralExpertWrapper(expert, torch.device("cuda:0"))
    assert expert.w1.W_q.data_ptr() != ptr_before  # re-homed
    base = wrapped.storage.data_ptr()
    for lin in (expert.w1, expert.w2, expert.w3):
        for t in (lin.W_q, lin.meta["scale_q"], lin.meta["zero_q"], lin.meta["meta_scale"]["scale"],
                  lin.meta["meta_zero"]["zero"]):
            off = t.data_ptr() - base
            assert 0 <= off < len(wrapped.storage) and off % SLAB_ALIGN == 0
    # order of the reference: sorted keys -> w1.W_q first, then its meta tensors, then w2 ...
    assert expert.w1.W_q.data_ptr() == base
    assert expert.w1.W_q.data_ptr() < expert.w1.meta["meta_scale"]["scale"].data_ptr() < expert.w1.meta["scale_q"].data_ptr() \
        < expert.w1.meta["zero_q"].data_ptr() < expert.w2.W_q.data_ptr() < expert.w3.W_q.data_ptr()
    assert torch.equal(wrapped(x), before)
    # a slab copied into another wrapper gives the same expert
    expert2 = bm.make_random_expert(cfg, qc, gen, torch.device("cuda:0"))
    wrapped2 = MixtralExpertWrapper(expert2, torch.device("cuda:0"))
    assert not torch.equal(wrapped2(x), before)
    wrapped2.storage.copy_(wrapped.storage)
    assert torch.equal(wrapped2(x), before)
    sd = wrapped.state_dict()
    assert list(sd) == ["storage"] and sd["storage"].dtype == torch.uint8


def test_moe_block_against_oracle():
    model, cfg = _small_setup(layers=1, offload_per_layer=0, main_per_layer=8)
    moe = model.model.layers[0].block_sparse_moe
    gen = torch.Generator(device="cuda").manual_seed(5)
    x = torch.randn((1, 4, cfg.hidden_size), device="cuda", generator=gen).half()
    y, logits = moe(x)
    assert y.shape == x.shape and logits.shape == (4, 8)
    xn = x[0].cpu().numpy()
    gate = moe.gate.weight.detach().cpu().numpy()
    w, idx, _ = o.router(xn, gate)
    cache = model.expert_cache
    want = np.zeros((4, cfg.hidden_size), np.float32)
    for e in range(8):
        info = cache.registered_experts[(0, e)]
        slot = info._group.global_slot[info._group.slot_of(info.index)]
        ex = cache.slots[slot]._expert[0]
        l1, l2, l3 = (_layer_to_numpy(l) for l in (ex.w1, ex.w2, ex.w3))
        for t in range(4):
            for k in range(2):
                if idx[t, k] == e:
                    out = o.expert_ffn(xn[t:t + 1], l1, l2, l3)[0].astype(np.float32)
                    want[t] += (out.astype(np.float16) * w[t, k]).astype(np.float16).astype(np.float32)
    got = y[0].float().cpu().numpy()
    scale = np.abs(want).max()
    assert np.abs(got - want).max() <= 3e-2 * scale, np.abs(got - want).max() / scale
    # same tokens one at a time (the decode path) agree with the batched call
    for t in range(4):
        y1, _ = moe(x[:, t:t + 1])
        assert torch.allclose(y1[0, 0].float(), y[0, t].float(), atol=2e-2 * float(scale), rtol=2e-2)


def test_expert_cache_loads_match_resident_results_and_lru_counts():
    """Experts served through misses (pinned host -> side-stream copy -> spare slot) must give bit-identical
    results to the same experts kept resident, and hit / miss counts must follow the LRU model."""
    model_off, cfg = _small_setup(layers=1, offload_per_layer=6, main_per_layer=2, buffers=2, seed=7)
    model_res, _ = _small_setup(layers=1, offload_per_layer=0, main_per_layer=8, buffers=1, seed=7)
    c_off, c_res = model_off.expert_cache, model_res.expert_cache
    gen = torch.Generator(device="cuda").manual_seed(1)
    x = torch.randn((1, cfg.hidden_size), device="cuda", generator=gen).half()
    lru = o.LruModel(resident=[6, 7], offloaded=[0, 1, 2, 3, 4, 5])
    rng = np.random.default_rng(0)
    for step in range(40):
        n = int(rng.integers(1, 5))
        req = rng.choice(8, size=n, replace=False).tolist()
        order_model, _ = lru.load(req)
        got_order = []
        outs = {}
        for (layer, e), expert in c_off.load_experts(*[(0, e) for e in req], unordered=True):
            got_order.append(e)
            outs[e] = expert(x).clone()
        assert got_order == order_model
        for (layer, e), expert in c_res.load_experts(*[(0, e) for e in req], unordered=True):
            assert torch.equal(outs[e], expert(x)), (step, e)
        g = c_off.group_infos[0]
        assert (g.hits, g.misses) == (lru.hits, lru.misses)
        resident_now = sorted(i.index for i in g.members if not i.offloaded)
        assert resident_now == sorted(lru.main)
    assert c_off.stats()["bytes_copied"] == lru.misses * c_off.module_size
    torch.cuda.synchronize()


@pytest.mark.parametrize("buffers", [1, 2])
@pytest.mark.parametrize("unordered", [True, False])
def test_one_call_for_more_experts_than_the_group_has_slots(buffers, unordered):
    """A prompt routes tokens to every expert of a layer in one call while only two fit on the device: a slot must
    not be loaded over before the expert in it has been handed out and used, whatever the order.  Experts big
    enough (6 MB) that a copy takes longer than the kernels around it, over several rounds, against the same
    experts kept resident."""
    kw = dict(layers=1, hidden=1024, ffn=4096, seed=11, heads=8, kv_heads=2)
    model_off, cfg = _small_setup(offload_per_layer=6, main_per_layer=2, buffers=buffers, **kw)
    model_res, _ = _small_setup(offload_per_layer=0, main_per_layer=8, buffers=1, **kw)
    c_off, c_res = model_off.expert_cache, model_res.expert_cache
    gen = torch.Generator(device="cuda").manual_seed(2)
    x = torch.randn((3, cfg.hidden_size), device="cuda", generator=gen).half()
    want = {e: expert(x).clone() for (_, e), expert in c_res.load_experts(*[(0, e) for e in range(8)], unordered=True)}
    rng = np.random.default_rng(4)
    for rnd in range(6):
        req = rng.permutation(8).tolist()
        seen = []
        for (_, e), expert in c_off.load_experts(*[(0, e) for e in req], unordered=unordered):
            seen.append(e)
            y = expert(x)
            assert torch.equal(y, want[e]), (rnd, e, seen)
        assert sorted(seen) == list(range(8))
        if not unordered:
            assert seen == req
    torch.cuda.synchronize()


def test_cache_error_paths():
    model, cfg = _small_setup(layers=1, offload_per_layer=6, main_per_layer=2, buffers=1)
    c = model.expert_cache
    with pytest.raises(AssertionError):
        list(c.load_experts((0, 1), (0, 1)))  # duplicates
    with pytest.raises(KeyError):
        list(c.load_experts((0, 99)))
    it = c.load_experts((0, 6), (0, 7))
    next(it)
    with pytest.raises(AssertionError):  # "already loading experts; buffers are busy"
        list(c.load_experts((0, 6)))
    list(it)
    with pytest.raises(AssertionError):  # already registered
        c.add_expert((0, 0), c.slots[0])
    with pytest.raises(ValueError):  # Cache is full
        c.add_expert((0, 100), c.slots[0], eviction_group=0, offload=True)


@pytest.mark.parametrize("ffn_bits,hidden,ffn", [(2, 256, 512), (3, 256, 512), (3, 1024, 1280), (4, 256, 512)])
def test_generate_offloaded_equals_resident(ffn_bits, hidden, ffn):
    """Greedy decoding with a 2-expert cache per layer gives the same tokens as with every expert resident (2-, 3- and
    4-bit experts; 3-bit ones at a size the decode kernel does not take, which run on the general kernel, and at one
    it does)."""
    model_off, cfg = _small_setup(layers=2, hidden=hidden, ffn=ffn, offload_per_layer=6, main_per_layer=2, buffers=2, seed=11,
                                  ffn_bits=ffn_bits)
    model_res, _ = _small_setup(layers=2, hidden=hidden, ffn=ffn, offload_per_layer=0, main_per_layer=8, buffers=1, seed=11,
                                ffn_bits=ffn_bits)
    prompt = torch.randint(0, cfg.vocab_size, (9,), device="cuda", generator=torch.Generator(device="cuda").manual_seed(2))
    a = model_off.generate(prompt, 12)
    b = model_res.generate(prompt, 12)
    assert torch.equal(a, b)
    st = model_off.expert_cache.stats()
    assert st["misses"] > 0 and st["hits"] + st["misses"] >= 2 * 12
    # prefill of the same tokens in one call agrees with token-by-token decoding (KV cache + RoPE consistency)
    cache = model_res.new_cache(32)
    full = model_res.forward(prompt, cache, 0)
    cache2 = model_res.new_cache(32)
    step_logits = [model_res.forward(prompt[i:i + 1], cache2, i)[0] for i in range(prompt.numel())]
    got = torch.stack(step_logits).float()
    assert torch.allclose(got, full.float(), atol=3e-2 * float(full.float().abs().max()), rtol=3e-2)


@pytest.mark.parametrize("layout", ["hqq", "kernel"])
@pytest.mark.parametrize("ffn_bits,ffn_group", [(2, 16), (3, 64), (4, 64)])
def test_checkpoint_round_trip(tmp_path, layout, ffn_bits, ffn_group):
    """A model written as a checkpoint directory and built again from it is the same model, bit for bit: the flat
    state-dict keys, the safetensors index, and (``hqq`` layout) the step-layout codes of the reference's files,
    which ``repack`` turns into the kernel layout at load."""
    import json
    from safetensors.torch import load_file
    from mixtral_offloading_amd import build_model as bm
    from mixtral_offloading_amd.hqq_core import BaseQuantizeConfig
    cfg = bm.mixtral_config(hidden_size=256, intermediate_size=512, num_hidden_layers=2, num_attention_heads=4,
                            num_key_value_heads=2, vocab_size=128, num_local_experts=4)
    qc = bm.QuantConfig(ffn_config=BaseQuantizeConfig(nbits=ffn_bits, group_size=ffn_group, quant_zero=True, quant_scale=True),
                        attn_config=bm.default_quant_config().attn_config)
    off = bm.OffloadConfig(main_size=4, offload_size=4, buffer_size=2, offload_per_layer=2)
    dev = torch.device("cuda:0")
    model = bm.build_model(dev, qc, off, model_config=cfg, seed=5, max_positions=64)
    bm.save_quantized_checkpoint(model, str(tmp_path), layout=layout)

    index = json.load(open(tmp_path / "model.safetensors.index.json"))["weight_map"]
    w1_key = "model.layers.1.block_sparse_moe.experts.3.w1.W_q"
    assert index["model.embed_tokens.weight"] != index[w1_key]
    on_disk = load_file(str(tmp_path / index[w1_key]))["w1.W_q"]  # the file holds the expert module's own keys
    n, k = 512, 256
    if layout == "kernel":
        assert tuple(on_disk.shape) == ((n + 9) // 10 if ffn_bits == 3 else n * ffn_bits // 8, k)
    else:  # quantise-time shape: group_size code rows (70 for the padded 3-bit words) packed down the rows
        rows = {2: ffn_group // 4, 4: ffn_group // 2, 3: (ffn_group + 9) // 10}[ffn_bits]
        assert tuple(on_disk.shape) == (rows, n * k // ffn_group)

    again = bm.build_model(dev, qc, off, state_path=str(tmp_path), model_config=cfg, max_positions=64)
    a, b = model.state_dict(), again.state_dict()
    assert list(a) == list(b)
    for key in a:
        assert torch.equal(torch.Tensor.as_subclass(a[key], torch.Tensor), torch.Tensor.as_subclass(b[key], torch.Tensor)), key
    for (uid, ea), (uid_b, eb) in zip(bm.iterate_experts(model), bm.iterate_experts(again)):
        sa, sb = ea.state_dict(), eb.state_dict()
        assert uid == uid_b and list(sa) == list(sb) and len(sa) == 3 * 7
        for key in sa:
            assert torch.equal(torch.Tensor.as_subclass(sa[key], torch.Tensor), torch.Tensor.as_subclass(sb[key], torch.Tensor)), (uid, key)
    prompt = torch.randint(0, cfg.vocab_size, (7,), device="cuda", generator=torch.Generator(device="cuda").manual_seed(1))
    assert torch.equal(model.generate(prompt, 6), again.generate(prompt, 6))
    assert torch.equal(model.forward(prompt, model.new_cache(16), 0), again.forward(prompt, again.new_cache(16), 0))


@pytest.mark.parametrize("offload_per_layer", [0, 6])
def test_single_token_step_equals_the_layerwise_forward(offload_per_layer):
    """``forward`` of one token takes the fused launches of the decode step (experts still fetched through the cache
    by the host); it must give what the layer-by-layer path gives for the same token and cache."""
    model, cfg = _small_setup(layers=2, offload_per_layer=offload_per_layer, main_per_layer=8 - offload_per_layer, seed=4)
    g = torch.Generator(device="cuda").manual_seed(8)
    prompt = torch.randint(0, cfg.vocab_size, (11,), device="cuda", generator=g)
    cache_a, cache_b = model.new_cache(32), model.new_cache(32)
    model.forward(prompt, cache_a, 0)
    model.forward(prompt, cache_b, 0)
    tok = torch.randint(0, cfg.vocab_size, (1,), device="cuda", generator=g)
    for pos in range(11, 17):
        fused = model.forward_token(tok, cache_a, pos).float()
        plain = model.forward_tokens(tok, cache_b, pos).float()
        assert fused.shape == plain.shape == (1, cfg.vocab_size)
        assert float((fused - plain).abs().max()) <= 2e-2 * float(plain.abs().max()) + 1e-3
        tok = plain[-1].argmax().view(1)
    for (ka, va), (kb, vb) in zip(cache_a, cache_b):  # both paths appended the same keys and values
        assert float((ka.float() - kb.float()).abs().max()) <= 2e-2 and float((va.float() - vb.float()).abs().max()) <= 2e-2
    with pytest.raises(ValueError):
        model.forward_token(tok, cache_a, 32)  # past the cache


def test_speculative_prefetch_overlaps_attention_and_keeps_the_tokens():
    """Speculative expert loads (the reference lists them as not yet available, README.md:24-26): the next layer's
    router is applied to this layer's post-attention state and the guessed experts start loading before the next
    layer's attention is launched.  The router is made predictable by construction -- a residual stream so large that
    a layer barely changes it, so consecutive layers see nearly the same normed state -- and the test checks that the
    guesses are mostly right, that the guessed copies run while the next layer's attention does, and that the tokens
    are those of the run without speculation."""
    def run(speculate):
        # experts of 19 MB: a copy takes a few hundred microseconds, longer than the host needs to launch the next
        # layer's attention
        model, cfg = _small_setup(layers=4, hidden=2048, ffn=8192, offload_per_layer=6, main_per_layer=2, buffers=4, seed=21,
                                  heads=16, kv_heads=4)
        model.model.embed_tokens.weight.data.mul_(2000.0)  # hidden states of size 40 against layer outputs of size 1
        model.speculate = speculate
        cache = model.expert_cache
        # (with two places per layer nearly every request misses, so the link is hardly ever idle: let guesses queue
        # behind demand copies here, the overlap is what this test is about)
        cache.prefetch_backlog, cache.prefetch_busy_limit = 8, 1.0
        cache.copy_trace, model.attention_trace = [], []
        base = torch.cuda.Event(enable_timing=True)
        base.record()
        prompt = torch.randint(0, cfg.vocab_size, (5,), device="cuda", generator=torch.Generator(device="cuda").manual_seed(3))
        tokens = model.generate(prompt, 16)
        torch.cuda.synchronize()
        return model, tokens, base

    plain, want, _ = run(False)
    assert plain.expert_cache.stats()["prefetch_loads"] == 0
    spec, got, base = run(True)
    assert torch.equal(got, want)
    st, st_plain = spec.expert_cache.stats(), plain.expert_cache.stats()
    assert st["prefetch_loads"] > 10
    # predictable by construction: most guesses are asked for next
    assert st["prefetch_useful"] >= 0.7 * st["prefetch_loads"], st
    # experts that arrived on a guess are hits of the real requests: fewer real misses than without speculation
    assert st["misses"] < st_plain["misses"] and st["hits"] + st["misses"] == st_plain["hits"] + st_plain["misses"]
    assert st["bytes_copied"] == (st["misses"] + st["prefetch_loads"]) * spec.expert_cache.module_size
    # overlap: a copy started on a guess for layer L+1 is in flight while layer L+1's attention runs
    att = [(layer, base.elapsed_time(a), base.elapsed_time(b)) for layer, a, b in spec.attention_trace]
    copies = [(uid, base.elapsed_time(a), base.elapsed_time(b)) for uid, a, b, kind in spec.expert_cache.copy_trace if kind == "prefetch"]
    assert copies
    overlapping = 0
    for (layer, e), c0, c1 in copies:
        overlapping += any(l == layer and a0 < c1 and c0 < a1 for l, a0, a1 in att)
    assert overlapping >= 0.5 * len(copies), (overlapping, len(copies))


def test_prompt_in_two_passes_equals_one_pass_and_the_torch_op_layer():
    """The prompt pass through the row kernels (residual add + norm, router, rope + cache append of all tokens): a prompt
    fed as 10 + 6 tokens gives the logits and caches of the 16 tokens at once, and a layer gives what the same layer
    gives with torch ops for norm, rope, cache append and router (the path CPU tensors take, here forced)."""
    from mixtral_offloading_amd import hip_kernels
    model, cfg = _small_setup(layers=2, offload_per_layer=0, main_per_layer=8, seed=6)
    g = torch.Generator(device="cuda").manual_seed(3)
    prompt = torch.randint(0, cfg.vocab_size, (16,), device="cuda", generator=g)
    cache_a, cache_b = model.new_cache(20), model.new_cache(20)
    whole = model.forward(prompt, cache_a, 0).float()
    first = model.forward(prompt[:10], cache_b, 0).float()
    second = model.forward(prompt[10:], cache_b, 10).float()
    both = torch.cat((first, second))
    assert float((both - whole).abs().max()) <= 2e-2 * float(whole.abs().max()) + 1e-3
    for (ka, va), (kb, vb) in zip(cache_a, cache_b):
        assert float((ka.float() - kb.float()).abs().max()) <= 2e-2 and float((va.float() - vb.float()).abs().max()) <= 2e-2

    with torch.inference_mode():
        # one layer against itself with the torch ops: rows kernels switched off by handing the layer fp16 tensors through
        # the reference formulas
        layer = model.model.layers[0]
        x = torch.randn((12, cfg.hidden_size), device="cuda", generator=g).half()
        ck, cv = (t.clone() for t in model.new_cache(16)[0])
        got = layer(x, model.rotary, ck, cv, 2)
        ck2, cv2 = (t.clone() for t in model.new_cache(16)[0])

        def norm(mod, t):
            tf = t.float()
            return mod.weight * (tf * torch.rsqrt(tf.pow(2).mean(-1, keepdim=True) + mod.variance_epsilon)).half()

        att, hd = layer.self_attn, cfg.hidden_size // cfg.num_attention_heads
        h = norm(layer.input_layernorm, x)
        q = att.q_proj(h).view(12, att.num_heads, hd)
        k = att.k_proj(h).view(12, att.num_kv_heads, hd)
        v = att.v_proj(h).view(12, att.num_kv_heads, hd)
        q, k = model.rotary.apply(q, k, torch.arange(2, 14, device="cuda"))
        ck2[:, 2:14], cv2[:, 2:14] = k.transpose(0, 1), v.transpose(0, 1)
        assert torch.equal(ck[:, 2:14], ck2[:, 2:14]) and torch.equal(cv[:, 2:14], cv2[:, 2:14])
        grp = att.num_heads // att.num_kv_heads
        qh = q.transpose(0, 1).reshape(att.num_kv_heads, grp * 12, hd)
        scores = torch.bmm(qh, ck2[:, :14].transpose(1, 2)).float() / hd ** 0.5
        tok = torch.arange(12, device="cuda").repeat(grp)
        allowed = torch.arange(14, device="cuda")[None, :] <= (2 + tok)[:, None]
        probs = torch.softmax(scores.masked_fill(~allowed[None], float("-inf")), dim=-1).half()
        o_ = torch.bmm(probs, cv2[:, :14]).view(att.num_kv_heads, grp, 12, hd).permute(2, 0, 1, 3).reshape(12, -1)
        x1 = x + att.o_proj(o_)
        h2 = norm(layer.post_attention_layernorm, x1)
        moe = layer.block_sparse_moe
        logits = moe.gate(h2)
        pw, ps = torch.topk(torch.softmax(logits, dim=1, dtype=torch.float), 2, dim=-1)
        pw = (pw / pw.sum(dim=-1, keepdim=True)).half()
        want = x1.clone()
        for t in range(12):
            for slot in range(2):
                (_, _), expert = next(iter(moe.experts.load_experts((0, int(ps[t, slot])))))
                want[t] += (pw[t, slot] * expert(h2[t:t + 1]))[0]
        assert float((got.float() - want.float()).abs().max()) <= 2e-2 * float(want.float().abs().max()) + 1e-3
