"""GPU tests of the decode-step helpers: the device-side router, residual add + RMSNorm, the expert FFN whose expert
is chosen on the device, and the graph-captured decode step against the eager path."""
import numpy as np
import pytest
import torch

from helpers import desc_of, to_dev
from oracle import hqq_oracle as o

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("n_experts,hidden", [(8, 4096), (8, 256), (4, 1024), (16, 512)])
def test_router_top2_against_oracle(n_experts, hidden):
    from mixtral_offloading_amd import hip_kernels
    rng = np.random.default_rng(n_experts + hidden)
    for trial in range(4):
        x = rng.standard_normal((1, hidden)).astype(np.float16)
        w = (rng.standard_normal((n_experts, hidden)) * 0.05).astype(np.float16)
        want_w, want_e, want_logits = o.router(x, w, top_k=2)
        sel = torch.zeros(2, dtype=torch.int32, device="cuda")
        rw = torch.zeros(2, dtype=torch.float16, device="cuda")
        logits = torch.zeros(n_experts, dtype=torch.float16, device="cuda")
        hip_kernels.router_top2(to_dev(x), to_dev(w), sel, rw, logits)
        # fp32 accumulation order differs from the oracle's float64: logits agree to an fp16 ulp or two
        assert np.allclose(logits.cpu().numpy().astype(np.float32), want_logits[0].astype(np.float32), atol=4e-3, rtol=4e-3)
        order = np.argsort(-want_logits[0].astype(np.float64), kind="stable")
        gap = float(want_logits[0][order[1]]) - float(want_logits[0][order[2]])
        if gap > 0.02 and float(want_logits[0][order[0]]) - float(want_logits[0][order[1]]) > 0.02:  # no near-tie
            assert sel.cpu().tolist() == [int(order[0]), int(order[1])]
            assert sel.cpu().tolist() == [int(v) for v in want_e[0]]
            assert np.allclose(rw.cpu().numpy().astype(np.float32), want_w[0].astype(np.float32), atol=2e-3)
        assert abs(float(rw.float().sum()) - 1.0) < 2e-3


@pytest.mark.parametrize("hidden", [256, 4096, 5120])
@pytest.mark.parametrize("with_delta", [False, True])
def test_add_rmsnorm_against_torch(hidden, with_delta):
    from mixtral_offloading_amd import hip_kernels
    g = torch.Generator(device="cuda").manual_seed(hidden)
    x = torch.randn((1, hidden), device="cuda", generator=g).half()
    d = torch.randn((1, hidden), device="cuda", generator=g).half() if with_delta else None
    w = (1 + 0.1 * torch.randn(hidden, device="cuda", generator=g)).half()
    x_want = x + d if with_delta else x.clone()
    xf = x_want.float()
    want = w * (xf * torch.rsqrt(xf.pow(2).mean(-1, keepdim=True) + 1e-5)).half()
    y = torch.empty_like(x)
    xin = x.clone()
    hip_kernels.add_rmsnorm(xin, d, w, 1e-5, y)
    assert torch.equal(xin, x_want)
    # the mean of squares is summed in a different order: results agree to an fp16 ulp
    assert float((y.float() - want.float()).abs().max()) <= 2e-3 * float(want.float().abs().max())


@pytest.mark.parametrize("n_experts,hidden", [(8, 4096), (8, 256), (4, 1024), (16, 5120)])
def test_add_rmsnorm_router_equals_the_two_calls(n_experts, hidden):
    from mixtral_offloading_amd import hip_kernels
    g = torch.Generator(device="cuda").manual_seed(hidden + n_experts)
    for trial in range(3):
        x = torch.randn((1, hidden), device="cuda", generator=g).half()
        d = torch.randn((1, hidden), device="cuda", generator=g).half() if trial else None
        w = (1 + 0.1 * torch.randn(hidden, device="cuda", generator=g)).half()
        gw = (0.05 * torch.randn((n_experts, hidden), device="cuda", generator=g)).half()
        x1, y1 = x.clone(), torch.empty_like(x)
        sel1, rw1 = torch.zeros(2, dtype=torch.int32, device="cuda"), torch.zeros(2, dtype=torch.float16, device="cuda")
        lg1 = torch.zeros(n_experts, dtype=torch.float16, device="cuda")
        hip_kernels.add_rmsnorm(x1, d, w, 1e-5, y1)
        hip_kernels.router_top2(y1, gw, sel1, rw1, lg1)
        x2, y2 = x.clone(), torch.empty_like(x)
        sel2, rw2, lg2 = torch.zeros_like(sel1), torch.zeros_like(rw1), torch.zeros_like(lg1)
        hip_kernels.add_rmsnorm_router(x2, d, w, 1e-5, y2, gw, sel2, rw2, lg2)
        assert torch.equal(x1, x2) and torch.equal(y1, y2)
        assert float((lg1.float() - lg2.float()).abs().max()) <= 4e-3 * max(1.0, float(lg1.float().abs().max()))
        top = lg1.float().sort(descending=True).values
        if float(top[0] - top[1]) > 0.02 and float(top[1] - top[2]) > 0.02:  # no near-tie
            assert sel1.tolist() == sel2.tolist()
            assert float((rw1.float() - rw2.float()).abs().max()) <= 2e-3


@pytest.mark.parametrize("nbits,hidden,ffn,gs", [(2, 512, 1024, 16), (3, 768, 1280, 64)])
@pytest.mark.parametrize("m", [1, 2, 4])
def test_expert_ffn_indexed_equals_direct(m, nbits, hidden, ffn, gs):
    from mixtral_offloading_amd import hip_kernels
    rng = np.random.default_rng(17 + m)
    experts = []
    for e in range(4):
        w1, _ = o.random_layer(rng, ffn, hidden, nbits, gs)
        w3, _ = o.random_layer(rng, ffn, hidden, nbits, gs)
        w2, _ = o.random_layer(rng, hidden, ffn, nbits, gs)
        experts.append((desc_of(w1), desc_of(w2), desc_of(w3)))
    table = hip_kernels.ExpertTable(experts)
    x = to_dev(rng.standard_normal((m, hidden)).astype(np.float16))
    rw = to_dev(rng.uniform(0.2, 0.8, size=(m,)).astype(np.float16))
    for e in (2, 0, 3):
        idx = torch.tensor([e], dtype=torch.int32, device="cuda")
        base = to_dev(rng.standard_normal((m, hidden)).astype(np.float16))
        want = base.clone()
        hip_kernels.expert_ffn(*experts[e], x, out=want, row_scale=rw, accumulate=True)
        got = base.clone()
        hip_kernels.expert_ffn_indexed(table, idx, x, got, row_scale=rw, accumulate=True)
        assert torch.equal(got, want)
        plain = torch.empty_like(base)
        hip_kernels.expert_ffn_indexed(table, idx, x, plain)
        assert torch.equal(plain, hip_kernels.expert_ffn(*experts[e], x))


# (nbits, hidden, ffn, group size, quantised tables): K of the down projections split over one and several blocks
PAIR_SHAPES = [(2, 512, 1024, 16, True), (2, 1024, 3584, 16, True), (4, 512, 2048, 64, True), (2, 256, 768, 16, False),
               (2, 4096, 14336, 16, True), (3, 768, 1280, 64, True), (3, 1024, 2560, 32, False), (3, 4096, 14336, 64, True)]


@pytest.mark.parametrize("shape", PAIR_SHAPES, ids=lambda s: "w%d_h%d_f%d_g%d_%s" % (s[0], s[1], s[2], s[3], "q" if s[4] else "f16"))
def test_expert_pair_equals_two_indexed_calls(shape):
    """Both active experts of a token in two launches against one hqq_expert_ffn_indexed call per expert: the same
    fp16 rounding points for the projections, but K may be split over waves and blocks differently, so the fp32 sums
    can differ in the last bit and some outputs land on the neighbouring fp16 value."""
    from mixtral_offloading_amd import hip_kernels
    from test_gpu_matmul import _full_size_layer
    nbits, hidden, ffn, gs, qt = shape
    rng = np.random.default_rng(hidden + ffn)
    experts = []
    for e in range(3):
        if hidden >= 4096:  # built on the GPU: the numpy generator takes seconds per layer at this size
            experts.append((_full_size_layer(nbits, ffn, hidden, gs, seed=3 * e), _full_size_layer(nbits, hidden, ffn, gs, seed=3 * e + 1),
                            _full_size_layer(nbits, ffn, hidden, gs, seed=3 * e + 2)))
            continue
        w1, _ = o.random_layer(rng, ffn, hidden, nbits, gs, qt, qt)
        w3, _ = o.random_layer(rng, ffn, hidden, nbits, gs, qt, qt)
        w2, _ = o.random_layer(rng, hidden, ffn, nbits, gs, qt, qt)
        experts.append((desc_of(w1), desc_of(w2), desc_of(w3)))
    table = hip_kernels.ExpertTable(experts)
    assert hip_kernels.expert_pair_supported(table)
    x = to_dev(rng.standard_normal((1, hidden)).astype(np.float16))
    for pair in ((2, 0), (1, 2), (0, 1), (1, 1)):
        sel = torch.tensor(pair, dtype=torch.int32, device="cuda")
        rw = to_dev(rng.uniform(0.2, 0.8, size=(2,)).astype(np.float16))
        base = to_dev(rng.standard_normal((1, hidden)).astype(np.float16))
        for accumulate in (False, True):
            want = base.clone()
            hip_kernels.expert_ffn_indexed(table, sel[0:1], x, want, row_scale=rw[0:1], accumulate=accumulate)
            hip_kernels.expert_ffn_indexed(table, sel[1:2], x, want, row_scale=rw[1:2], accumulate=True)
            got = base.clone()
            hip_kernels.expert_pair_ffn_indexed(table, sel, x, got, rw, accumulate=accumulate)
            err = (got.float() - want.float()).abs()
            # h differs by an fp16 ulp in places, which the down projection carries through
            assert float(err.max()) <= 4e-3 * float(want.float().abs().max()), (pair, accumulate, float(err.max()))
            # where K is split over blocks the weighted sum of both experts is rounded to fp16 once, while the two
            # calls round each product and then the sum: about half of the outputs land on the neighbouring value
            assert float((err > 0).float().mean()) < 0.75


@pytest.mark.parametrize("shape", [(2, 512, 1024, 16, True), (2, 4096, 14336, 16, True), (4, 512, 2048, 64, True)],
                         ids=lambda s: "w%d_h%d_f%d" % s[:3])
def test_moe_pair_routed_equals_the_calls_it_replaces(shape):
    """Norm, router and both experts in two launches: the bits of hqq_add_rmsnorm_router followed by
    hqq_expert_pair_ffn_indexed."""
    from mixtral_offloading_amd import hip_kernels
    from test_gpu_matmul import _full_size_layer
    nbits, hidden, ffn, gs, qt = shape
    rng = np.random.default_rng(hidden + ffn + 1)
    experts = []
    for e in range(8):
        if hidden >= 4096:
            experts.append((_full_size_layer(nbits, ffn, hidden, gs, seed=3 * e), _full_size_layer(nbits, hidden, ffn, gs, seed=3 * e + 1),
                            _full_size_layer(nbits, ffn, hidden, gs, seed=3 * e + 2)))
            continue
        w1, _ = o.random_layer(rng, ffn, hidden, nbits, gs, qt, qt)
        w3, _ = o.random_layer(rng, ffn, hidden, nbits, gs, qt, qt)
        w2, _ = o.random_layer(rng, hidden, ffn, nbits, gs, qt, qt)
        experts.append((desc_of(w1), desc_of(w2), desc_of(w3)))
    table = hip_kernels.ExpertTable(experts)
    for trial in range(4):
        x = to_dev(rng.standard_normal((1, hidden)).astype(np.float16))
        d = to_dev(rng.standard_normal((1, hidden)).astype(np.float16)) if trial else None
        w = to_dev((1 + 0.1 * rng.standard_normal(hidden)).astype(np.float16))
        gw = to_dev((0.05 * rng.standard_normal((8, hidden))).astype(np.float16))
        base = to_dev(rng.standard_normal((1, hidden)).astype(np.float16))
        for accumulate in (False, True):
            x1, xn = x.clone(), torch.empty_like(x)
            sel1, rw1 = torch.zeros(2, dtype=torch.int32, device="cuda"), torch.zeros(2, dtype=torch.float16, device="cuda")
            hip_kernels.add_rmsnorm_router(x1, d, w, 1e-5, xn, gw, sel1, rw1)
            want = base.clone()
            hip_kernels.expert_pair_ffn_indexed(table, sel1, xn, want, rw1, accumulate=accumulate)
            x_sum = torch.full_like(x, float("nan"))
            sel2, rw2 = torch.full_like(sel1, -1), torch.zeros_like(rw1)
            got = base.clone()
            hip_kernels.moe_pair_routed(table, x, d, w, 1e-5, x_sum, gw, sel2, rw2, got, accumulate=accumulate)
            assert torch.equal(x_sum, x1)
            assert sel1.tolist() == sel2.tolist() and torch.equal(rw1, rw2)
            assert torch.equal(got, want), float((got.float() - want.float()).abs().max())


@pytest.mark.parametrize("nbits,gs,k,ns,bias", [(4, 64, 4096, (4096, 1024, 1024), False), (4, 64, 1024, (512, 128, 128), True),
                                                (2, 16, 512, (256, 64), False), (4, 32, 1024, (64, 64, 64, 128), True)])
def test_matmul_group_equals_single_calls(nbits, gs, k, ns, bias):
    """q, k and v projections in one launch against hqq_matmul_transpose on each layer: equal up to the order in which
    the fp32 partial sums over K are added (the split of K follows the size of the whole launch)."""
    from mixtral_offloading_amd import hip_kernels
    rng = np.random.default_rng(k + len(ns))
    descs = []
    for n in ns:
        w, _ = o.random_layer(rng, n, k, nbits, gs)
        b = rng.standard_normal((n,)).astype(np.float16) if bias else None
        descs.append(desc_of(w, bias=b))
    group = hip_kernels.LinearGroup(descs)
    assert group.supported
    for rep in range(3):
        x = to_dev(rng.standard_normal((1, k)).astype(np.float16))
        outs = group(x)
        for d, y in zip(descs, outs):
            want = hip_kernels.matmul(d, x)
            err = (y.float() - want.float()).abs()
            assert float(err.max()) <= 1e-3 * float(want.float().abs().max()), float(err.max())
            assert float((err > 0).float().mean()) < 0.2


@pytest.mark.parametrize("nbits,gs,k,ns", [(4, 64, 4096, (4096, 1024, 1024)), (4, 64, 1024, (512, 128, 128)),
                                           (2, 16, 512, (256, 64))])
@pytest.mark.parametrize("with_delta", [False, True])
def test_matmul_group_norm_equals_norm_then_group(nbits, gs, k, ns, with_delta):
    """Residual add and RMSNorm folded into the grouped launch: the bits of hqq_add_rmsnorm followed by
    hqq_matmul_group, and x + delta in the second buffer."""
    from mixtral_offloading_amd import hip_kernels
    rng = np.random.default_rng(k + len(ns) + with_delta)
    descs = [desc_of(o.random_layer(rng, n, k, nbits, gs)[0]) for n in ns]
    group = hip_kernels.LinearGroup(descs)
    assert group.supported
    for rep in range(3):
        x = to_dev(rng.standard_normal((1, k)).astype(np.float16))
        d = to_dev(rng.standard_normal((1, k)).astype(np.float16)) if with_delta else None
        w = to_dev((1 + 0.1 * rng.standard_normal(k)).astype(np.float16))
        x_ref, xn = x.clone(), torch.empty_like(x)
        hip_kernels.add_rmsnorm(x_ref, d, w, 1e-5, xn)
        want = group(xn)
        x_sum = torch.full_like(x, float("nan"))
        got = hip_kernels.matmul_group_norm(group, x, d, w, 1e-5, x_sum)
        assert torch.equal(x_sum, x_ref)
        for a, b in zip(got, want):
            assert torch.equal(a, b)


def test_matmul_group_refuses_mixed_layers():
    from mixtral_offloading_amd import hip_kernels
    rng = np.random.default_rng(3)
    a, _ = o.random_layer(rng, 256, 512, 4, 64)
    b, _ = o.random_layer(rng, 256, 512, 2, 16)
    assert not hip_kernels.LinearGroup([desc_of(a), desc_of(b)]).supported


@pytest.mark.parametrize("ffn_bits,wide", [(2, False), (3, False), (2, True)])
def test_graph_decode_matches_eager_logits(ffn_bits, wide):
    """Each replayed step must give the logits of the eager forward at the same position (same kernels for the
    quantized linears; attention over the masked full cache instead of the sliced one).  With 3-bit experts the
    step takes the norm + router launch and the three-launch expert pair instead of the routed pair."""
    from mixtral_offloading_amd import build_model as bm
    from mixtral_offloading_amd.hqq_core import BaseQuantizeConfig
    from mixtral_offloading_amd.mixtral_model import DecodeGraph
    qc = bm.default_quant_config()
    if wide:  # a row longer than the routed launch takes: norm + router in a launch of their own, then the pair
        cfg = bm.mixtral_config(hidden_size=5120, intermediate_size=1024, num_hidden_layers=2, num_attention_heads=40,
                                num_key_value_heads=8, vocab_size=128, num_local_experts=4)
    elif ffn_bits == 2:
        cfg = bm.mixtral_config(hidden_size=256, intermediate_size=512, num_hidden_layers=2, num_attention_heads=4,
                                num_key_value_heads=2, vocab_size=128, num_local_experts=8)
    else:
        cfg = bm.mixtral_config(hidden_size=1024, intermediate_size=1280, num_hidden_layers=2, num_attention_heads=8,
                                num_key_value_heads=2, vocab_size=128, num_local_experts=8)
        qc = bm.QuantConfig(ffn_config=BaseQuantizeConfig(nbits=3, group_size=64, quant_zero=True, quant_scale=True),
                            attn_config=qc.attn_config)
    off = bm.OffloadConfig(main_size=2 * cfg.num_local_experts, offload_size=0, buffer_size=1, offload_per_layer=0)
    model = bm.build_model(torch.device("cuda:0"), qc, off, model_config=cfg, seed=5, max_positions=64)
    prompt = torch.randint(0, 128, (9,), device="cuda", generator=torch.Generator(device="cuda").manual_seed(2))
    steps = 6
    dec = DecodeGraph(model, prompt.numel() + steps + 4)
    assert dec.pair and dec.routed == (ffn_bits == 2 and not wide)
    first = dec.prefill(prompt)
    dec.capture()
    # eager reference driven with the graph's own tokens
    cache = model.new_cache(prompt.numel() + steps + 4)
    logits = model.forward(prompt, cache, 0)
    assert int(logits[-1].argmax()) == int(first)
    tok, pos = first.view(1), prompt.numel()
    for _ in range(steps):
        want = model.forward(tok, cache, pos)[-1].float()
        dec.step()
        got = dec.logits[0].float()
        assert float((got - want).abs().max()) <= 2e-2 * float(want.abs().max()) + 1e-3
        tok, pos = dec.tok.clone(), pos + 1
    assert int(dec.pos) == pos


def test_graph_decode_guards_its_cache_capacity():
    """A prompt or a step past the cache raises on the host; the attention kernel itself leaves a position past the
    cache alone."""
    from mixtral_offloading_amd import build_model as bm, hip_kernels
    from mixtral_offloading_amd.mixtral_model import DecodeGraph, Rotary
    cfg = bm.mixtral_config(hidden_size=256, intermediate_size=512, num_hidden_layers=1, num_attention_heads=4,
                            num_key_value_heads=2, vocab_size=128, num_local_experts=8)
    off = bm.OffloadConfig(main_size=8, offload_size=0, buffer_size=1, offload_per_layer=0)
    model = bm.build_model(torch.device("cuda:0"), bm.default_quant_config(), off, model_config=cfg, seed=5,
                           max_positions=64)
    with pytest.raises(ValueError):
        DecodeGraph(model, 65)  # a cache longer than the rope tables: the device-side position could run past them
    with pytest.raises(ValueError):
        model.new_cache(65)
    dec = DecodeGraph(model, 12)
    with pytest.raises(ValueError):
        dec.prefill(torch.zeros(12, dtype=torch.int64, device="cuda"))
    dec.prefill(torch.arange(10, device="cuda"))
    with pytest.raises(ValueError):
        dec.capture()  # needs positions 10, 11 and 12
    dec.step()
    dec.step()
    with pytest.raises(ValueError):
        dec.step()
    hd, L = 64, 16
    rot = Rotary(hd, 64, 1e6, torch.device("cuda"))
    ck = torch.zeros((2, L, hd), dtype=torch.float16, device="cuda")
    cv = torch.zeros_like(ck)
    guard = torch.zeros((2, 4 * hd), dtype=torch.float16, device="cuda")  # would be hit by a write at position L
    q = torch.randn((1, 4 * hd), device="cuda").half()
    k = torch.randn((1, 2 * hd), device="cuda").half()
    out = torch.zeros((1, 4 * hd), dtype=torch.float16, device="cuda")
    hip_kernels.attention_decode(q, k, k, rot.cos, rot.sin, torch.tensor([L], device="cuda"), ck, cv, out)
    torch.cuda.synchronize()
    assert float(ck.abs().sum()) == 0 and float(cv.abs().sum()) == 0 and float(out.abs().sum()) == 0 and float(guard.abs().sum()) == 0


def test_graph_decode_refuses_offloaded_experts():
    from mixtral_offloading_amd import build_model as bm
    from mixtral_offloading_amd.mixtral_model import DecodeGraph
    cfg = bm.mixtral_config(hidden_size=256, intermediate_size=512, num_hidden_layers=1, num_attention_heads=4,
                            num_key_value_heads=2, vocab_size=128, num_local_experts=8)
    off = bm.OffloadConfig(main_size=4, offload_size=4, buffer_size=2, offload_per_layer=4)
    model = bm.build_model(torch.device("cuda:0"), bm.default_quant_config(), off, model_config=cfg, seed=5,
                           max_positions=64)
    with pytest.raises(RuntimeError):
        DecodeGraph(model, 32)


@pytest.mark.parametrize("heads,kv,hd,pos,L", [(32, 8, 128, 0, 512), (32, 8, 128, 37, 512), (32, 8, 128, 511, 512),
                                               (4, 2, 64, 5, 512), (8, 8, 64, 300, 512),
                                               # caches past 512 positions run the 1024-thread form of the kernel
                                               (32, 8, 128, 3, 2048), (32, 8, 128, 1500, 2048), (8, 8, 64, 1100, 1200)])
def test_attention_decode_against_torch_ops(heads, kv, hd, pos, L):
    """Same roundings as the harness's torch attention (rope terms, fp16 scores, fp32 softmax, fp16 probabilities)."""
    import math
    from mixtral_offloading_amd import hip_kernels
    from mixtral_offloading_amd.mixtral_model import Rotary
    g = torch.Generator(device="cuda").manual_seed(heads + pos)
    rot = Rotary(hd, L, 1e6, torch.device("cuda"))
    q = torch.randn((1, heads * hd), device="cuda", generator=g).half()
    k = torch.randn((1, kv * hd), device="cuda", generator=g).half()
    v = torch.randn((1, kv * hd), device="cuda", generator=g).half()
    ck = torch.randn((kv, L, hd), device="cuda", generator=g).half()
    cv = torch.randn((kv, L, hd), device="cuda", generator=g).half()
    ck2, cv2 = ck.clone(), cv.clone()
    # torch path (the harness's Attention.forward for T = 1)
    positions = torch.tensor([pos], device="cuda")
    qr, kr = rot.apply(q.view(1, heads, hd), k.view(1, kv, hd), positions)
    ck[:, pos:pos + 1] = kr.transpose(0, 1)
    cv[:, pos:pos + 1] = v.view(1, kv, hd).transpose(0, 1)
    grp = heads // kv
    qh = qr.transpose(0, 1).reshape(kv, grp, hd)
    scores = torch.bmm(qh, ck[:, :pos + 1].transpose(1, 2)).float() / math.sqrt(hd)
    probs = torch.softmax(scores, dim=-1).half()
    want = torch.bmm(probs, cv[:, :pos + 1]).view(kv, grp, 1, hd).permute(2, 0, 1, 3).reshape(1, -1)
    out = torch.empty((1, heads * hd), dtype=torch.float16, device="cuda")
    hip_kernels.attention_decode(q, k, v, rot.cos, rot.sin, torch.tensor([pos], device="cuda"), ck2, cv2, out)
    assert torch.equal(ck2, ck) and torch.equal(cv2, cv)  # the rotated key and the value landed in the cache, bit-exact
    err = (out.float() - want.float()).abs().max()
    assert float(err) <= 4e-3 * max(1.0, float(want.float().abs().max()))


@pytest.mark.parametrize("heads,kv,hd,pos,L", [(32, 8, 128, 0, 2048), (32, 8, 128, 1, 2048), (32, 8, 128, 1023, 2048), (32, 8, 128, 1024, 2048),
                                               (32, 8, 128, 2047, 2048), (32, 8, 128, 5, 4096), (32, 8, 128, 3000, 4096),
                                               (32, 8, 128, 4095, 4096), (8, 8, 64, 1100, 1200), (4, 2, 64, 2900, 3000), (8, 2, 128, 15999, 16000)])
def test_split_attention_against_the_one_block_kernel(heads, kv, hd, pos, L):
    """Caches past 512 positions: a head's positions over two to eight blocks, shares added up by the block that
    finishes last.  Against the one-block kernel (itself checked against the torch ops above) within fp16 rounding of
    the output -- its probabilities stay fp32 --, the cache bit for bit, and twice in a row (the counters in the
    workspace must be back at zero)."""
    from mixtral_offloading_amd import hip_kernels, _lib
    from mixtral_offloading_amd.mixtral_model import Rotary
    assert _lib.lib.hqq_attention_decode_workspace_bytes(L, heads, hd) > 0
    g = torch.Generator(device="cuda").manual_seed(heads + pos + L)
    rot = Rotary(hd, L, 1e6, torch.device("cuda"))
    ck = torch.randn((kv, L, hd), device="cuda", generator=g).half()
    cv = torch.randn((kv, L, hd), device="cuda", generator=g).half()
    for rep in range(2):
        q = torch.randn((1, heads * hd), device="cuda", generator=g).half()
        k = torch.randn((1, kv * hd), device="cuda", generator=g).half()
        v = torch.randn((1, kv * hd), device="cuda", generator=g).half()
        ck1, cv1, ck2, cv2 = ck.clone(), cv.clone(), ck.clone(), cv.clone()
        p = torch.tensor([pos], device="cuda")
        want = torch.empty((1, heads * hd), dtype=torch.float16, device="cuda")
        got = torch.empty_like(want)
        hip_kernels.attention_decode(q, k, v, rot.cos, rot.sin, p, ck1, cv1, want, split=False)
        hip_kernels.attention_decode(q, k, v, rot.cos, rot.sin, p, ck2, cv2, got)
        assert torch.equal(ck1, ck2) and torch.equal(cv1, cv2)
        err = (got.float() - want.float()).abs().max()
        assert float(err) <= 4e-3 * max(1.0, float(want.float().abs().max())), float(err)
    # a position outside the cache: nothing written, nothing counted
    before = ck.clone()
    hip_kernels.attention_decode(q, k, v, rot.cos, rot.sin, torch.tensor([L], device="cuda"), ck, cv, got)
    torch.cuda.synchronize()
    assert torch.equal(ck, before)


@pytest.mark.gpu
@pytest.mark.parametrize("rows,hidden", [(1, 256), (7, 1024), (128, 4096), (33, 5120)])
@pytest.mark.parametrize("with_delta", [False, True])
def test_add_rmsnorm_rows_equals_the_one_row_call(rows, hidden, with_delta):
    from mixtral_offloading_amd import hip_kernels
    g = torch.Generator(device="cuda").manual_seed(rows * hidden)
    x = torch.randn((rows, hidden), device="cuda", generator=g).half()
    d = torch.randn((rows, hidden), device="cuda", generator=g).half() if with_delta else None
    w = (1 + 0.1 * torch.randn(hidden, device="cuda", generator=g)).half()
    xs = x.clone()
    ys = hip_kernels.add_rmsnorm_rows(xs, d, w, 1e-5)
    for r in sorted({0, rows // 2, rows - 1}):
        x1, y1 = x[r:r + 1].clone(), torch.empty((1, hidden), dtype=torch.float16, device="cuda")
        hip_kernels.add_rmsnorm(x1, d[r:r + 1].clone() if with_delta else None, w, 1e-5, y1)
        assert torch.equal(xs[r:r + 1], x1) and torch.equal(ys[r:r + 1], y1)
    x_want = x + d if with_delta else x
    xf = x_want.float()
    want = w * (xf * torch.rsqrt(xf.pow(2).mean(-1, keepdim=True) + 1e-5)).half()
    assert torch.equal(xs, x_want)
    assert float((ys.float() - want.float()).abs().max()) <= 2e-3 * float(want.float().abs().max())


@pytest.mark.gpu
@pytest.mark.parametrize("rows,n_experts,hidden", [(1, 8, 256), (128, 8, 4096), (19, 4, 1024), (64, 16, 512)])
def test_router_top2_rows_equals_the_one_row_call_and_the_reference_lines(rows, n_experts, hidden):
    from mixtral_offloading_amd import hip_kernels
    g = torch.Generator(device="cuda").manual_seed(rows + hidden)
    x = torch.randn((rows, hidden), device="cuda", generator=g).half()
    gw = (0.05 * torch.randn((n_experts, hidden), device="cuda", generator=g)).half()
    sel, rw, lg = hip_kernels.router_top2_rows(x, gw)
    for r in sorted({0, rows // 2, rows - 1}):
        s1, w1 = torch.zeros(2, dtype=torch.int32, device="cuda"), torch.zeros(2, dtype=torch.float16, device="cuda")
        l1 = torch.zeros(n_experts, dtype=torch.float16, device="cuda")
        hip_kernels.router_top2(x[r:r + 1].clone(), gw, s1, w1, l1)
        assert torch.equal(sel[r], s1) and torch.equal(rw[r], w1) and torch.equal(lg[r], l1)
    # the reference's five lines (src/custom_layers.py:276-282) in torch
    logits = torch.nn.functional.linear(x, gw)
    p = torch.softmax(logits, dim=1, dtype=torch.float)
    pw, ps = torch.topk(p, 2, dim=-1)
    pw = (pw / pw.sum(dim=-1, keepdim=True)).half()
    assert float((lg.float() - logits.float()).abs().max()) <= 4e-3 * max(1.0, float(logits.float().abs().max()))
    top = logits.float().sort(dim=1, descending=True).values
    clear = ((top[:, 0] - top[:, 1]) > 0.02) & ((top[:, 1] - top[:, 2]) > 0.02)  # rows without a near-tie
    assert int(clear.sum()) >= rows // 2
    assert torch.equal(sel[clear].long(), ps[clear])
    assert float((rw[clear].float() - pw[clear].float()).abs().max()) <= 2e-3


@pytest.mark.gpu
@pytest.mark.parametrize("tokens,n_experts", [(1, 8), (2, 8), (128, 8), (129, 2), (1000, 16), (4096, 8)])
def test_moe_group_pairs_is_a_stable_sort_by_expert(tokens, n_experts):
    """The device-side grouping of a prompt pass's (token, slot) pairs equals the stable sort by expert the host would
    do (numpy), including experts that received no pair; index for index (integers: exact)."""
    import numpy as np
    from mixtral_offloading_amd import hip_kernels
    rng = np.random.default_rng(tokens + n_experts)
    first = rng.integers(0, n_experts, size=tokens)
    second = (first + rng.integers(1, n_experts, size=tokens)) % n_experts  # two different experts per token
    if n_experts > 2:
        first[first == 1] = 0  # expert 1 is chosen first by nobody ...
        second[second == 1] = np.where(first[second == 1] == 2, 0, 2)  # ... and second by nobody: an empty group
    sel = np.stack([first, second], axis=1).astype(np.int32)
    w = rng.uniform(0.0, 1.0, size=(tokens, 2)).astype(np.float16)
    counts, token_of_row, scale_of_row = hip_kernels.moe_group_pairs(torch.from_numpy(sel).cuda(), torch.from_numpy(w).cuda(),
                                                                     n_experts)
    flat = sel.reshape(-1)
    order = np.argsort(flat, kind="stable")
    assert np.array_equal(counts.cpu().numpy(), np.bincount(flat, minlength=n_experts))
    assert np.array_equal(token_of_row.cpu().numpy(), order // 2)
    assert np.array_equal(scale_of_row.cpu().numpy(), w.reshape(-1)[order])
    if n_experts > 2:
        assert int(counts[1]) == 0
    # an expert id out of range is left out; the rows that stay free name token 0 with weight zero
    bad = sel.copy()
    bad[0, 0] = n_experts + 3
    counts, token_of_row, scale_of_row = hip_kernels.moe_group_pairs(torch.from_numpy(bad).cuda(), torch.from_numpy(w).cuda(),
                                                                     n_experts)
    assert int(counts.sum()) == 2 * tokens - 1
    assert int(token_of_row[-1]) == 0 and float(scale_of_row[-1]) == 0.0


@pytest.mark.gpu
@pytest.mark.parametrize("T,heads,kv,hd,start,L", [(128, 32, 8, 128, 0, 130), (5, 32, 8, 128, 37, 64), (1, 4, 4, 64, 9, 10),
                                                   (17, 8, 2, 64, 0, 17)])
def test_rope_append_rows_equals_the_torch_ops(T, heads, kv, hd, start, L):
    from mixtral_offloading_amd import hip_kernels
    from mixtral_offloading_amd.mixtral_model import Rotary
    g = torch.Generator(device="cuda").manual_seed(T * hd + start)
    rot = Rotary(hd, L + 3, 1e6, torch.device("cuda"))
    q = torch.randn((T, heads, hd), device="cuda", generator=g).half()
    k = torch.randn((T, kv, hd), device="cuda", generator=g).half()
    v = torch.randn((T, kv, hd), device="cuda", generator=g).half()
    ck = torch.randn((kv, L, hd), device="cuda", generator=g).half()
    cv = torch.randn((kv, L, hd), device="cuda", generator=g).half()
    ck_want, cv_want = ck.clone(), cv.clone()
    q_want, k_want = rot.apply(q, k, torch.arange(start, start + T, device="cuda"))
    ck_want[:, start:start + T] = k_want.transpose(0, 1)
    cv_want[:, start:start + T] = v.transpose(0, 1)
    out = hip_kernels.rope_append_rows(q, k, v, rot.cos, rot.sin, start, ck, cv)
    assert out is q and torch.equal(q, q_want) and torch.equal(ck, ck_want) and torch.equal(cv, cv_want)
    with pytest.raises(Exception):  # past the end of the cache
        hip_kernels.rope_append_rows(q, k, v, rot.cos, rot.sin, L - T + 1, ck, cv)
