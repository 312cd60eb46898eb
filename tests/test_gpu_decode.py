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


@pytest.mark.parametrize("m", [1, 2, 4])
def test_expert_ffn_indexed_equals_direct(m):
    from mixtral_offloading_amd import hip_kernels
    rng = np.random.default_rng(17 + m)
    experts = []
    for e in range(4):
        w1, _ = o.random_layer(rng, 1024, 512, 2, 16)
        w3, _ = o.random_layer(rng, 1024, 512, 2, 16)
        w2, _ = o.random_layer(rng, 512, 1024, 2, 16)
        experts.append((desc_of(w1), desc_of(w2), desc_of(w3)))
    table = hip_kernels.ExpertTable(experts)
    x = to_dev(rng.standard_normal((m, 512)).astype(np.float16))
    rw = to_dev(rng.uniform(0.2, 0.8, size=(m,)).astype(np.float16))
    for e in (2, 0, 3):
        idx = torch.tensor([e], dtype=torch.int32, device="cuda")
        base = to_dev(rng.standard_normal((m, 512)).astype(np.float16))
        want = base.clone()
        hip_kernels.expert_ffn(*experts[e], x, out=want, row_scale=rw, accumulate=True)
        got = base.clone()
        hip_kernels.expert_ffn_indexed(table, idx, x, got, row_scale=rw, accumulate=True)
        assert torch.equal(got, want)
        plain = torch.empty_like(base)
        hip_kernels.expert_ffn_indexed(table, idx, x, plain)
        assert torch.equal(plain, hip_kernels.expert_ffn(*experts[e], x))


def test_graph_decode_matches_eager_logits():
    """Each replayed step must give the logits of the eager forward at the same position (same kernels for the
    quantized linears; attention over the masked full cache instead of the sliced one)."""
    from mixtral_offloading_amd import build_model as bm
    from mixtral_offloading_amd.mixtral_model import DecodeGraph
    cfg = bm.mixtral_config(hidden_size=256, intermediate_size=512, num_hidden_layers=2, num_attention_heads=4,
                            num_key_value_heads=2, vocab_size=128, num_local_experts=8)
    off = bm.OffloadConfig(main_size=16, offload_size=0, buffer_size=1, offload_per_layer=0)
    model = bm.build_model(torch.device("cuda:0"), bm.default_quant_config(), off, model_config=cfg, seed=5,
                           max_positions=64)
    prompt = torch.randint(0, 128, (9,), device="cuda", generator=torch.Generator(device="cuda").manual_seed(2))
    steps = 6
    dec = DecodeGraph(model, prompt.numel() + steps + 4)
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


@pytest.mark.parametrize("heads,kv,hd,pos", [(32, 8, 128, 0), (32, 8, 128, 37), (32, 8, 128, 511), (4, 2, 64, 5), (8, 8, 64, 300)])
def test_attention_decode_against_torch_ops(heads, kv, hd, pos):
    """Same roundings as the harness's torch attention (rope terms, fp16 scores, fp32 softmax, fp16 probabilities)."""
    import math
    from mixtral_offloading_amd import hip_kernels
    from mixtral_offloading_amd.mixtral_model import Rotary
    g = torch.Generator(device="cuda").manual_seed(heads + pos)
    L = 512
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
