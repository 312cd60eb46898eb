"""The attention part of a decoder layer at one token as one launch (hqq_attention_chain) against the three calls it
replaces (hqq_matmul_group_norm, hqq_attention_decode, hqq_matmul_transpose): the same bits in every output and in the
KV cache, at successive positions (the chain's counters must be back at zero after every launch), for both thread
counts of the attention part, and replayed from a HIP graph."""
import numpy as np
import pytest
import torch

from helpers import desc_of, to_dev
from oracle import hqq_oracle as o

pytestmark = pytest.mark.gpu

# (hidden, heads, kv heads, cache length, 8-bit tables)
SHAPES = [
    (4096, 32, 8, 1024, True),    # Mixtral-8x7B, the longest cache the chain takes (longer ones are split over blocks)
    (4096, 32, 8, 96, True),      # the 256-thread attention part
    (4096, 32, 8, 384, False),    # fp16 tables
    (4096, 32, 4, 200, False),
]


def _setup(hidden, heads, kv, L, q8, seed):
    from mixtral_offloading_amd import hip_kernels
    from mixtral_offloading_amd.mixtral_model import Rotary
    hd = 128
    rng = np.random.default_rng(seed)
    mk = lambda n, k: desc_of(o.random_layer(rng, n, k, 4, 64, q8, q8)[0])  # noqa: E731
    dq, dk, dv, do = mk(heads * hd, hidden), mk(kv * hd, hidden), mk(kv * hd, hidden), mk(hidden, heads * hd)
    group = hip_kernels.LinearGroup([dq, dk, dv])
    assert group.supported
    rot = Rotary(hd, L, 1e6, torch.device("cuda"))
    g = torch.Generator(device="cuda").manual_seed(seed)
    ck = torch.randn((kv, L, hd), device="cuda", generator=g).half()
    cv = torch.randn((kv, L, hd), device="cuda", generator=g).half()
    w = to_dev((1 + 0.1 * rng.standard_normal(hidden)).astype(np.float16))
    return rng, group, do, rot, ck, cv, w


def _three_calls(group, do, rot, x, d, w, pos, ck, cv):
    from mixtral_offloading_amd import hip_kernels
    x_sum = torch.empty_like(x)
    q, k, v = hip_kernels.matmul_group_norm(group, x, d, w, 1e-5, x_sum)
    att = torch.empty((1, q.numel()), dtype=torch.float16, device="cuda")
    hip_kernels.attention_decode(q, k, v, rot.cos, rot.sin, pos, ck, cv, att)
    return hip_kernels.matmul(do, att), x_sum


@pytest.mark.parametrize("shape", SHAPES, ids=lambda s: "h%d_%dx%d_L%d_%s" % (s[0], s[1], s[2], s[3], "q" if s[4] else "f16"))
def test_chain_equals_the_three_calls(shape):
    from mixtral_offloading_amd import hip_kernels
    hidden, heads, kv, L, q8 = shape
    rng, group, do, rot, ck, cv, w = _setup(hidden, heads, kv, L, q8, seed=hidden + L)
    chain = hip_kernels.AttentionChain(group, do)
    ck2, cv2 = ck.clone(), cv.clone()
    for step, p in enumerate([0, 1, 2, 37, L // 2, L - 2, L - 1]):
        x = to_dev(rng.standard_normal((1, hidden)).astype(np.float16))
        d = to_dev(rng.standard_normal((1, hidden)).astype(np.float16)) if step % 2 else None
        pos = torch.tensor([p], device="cuda")
        want, want_sum = _three_calls(group, do, rot, x, d, w, pos, ck, cv)
        x_sum = torch.full_like(x, float("nan"))
        got = chain(x, d, w, 1e-5, x_sum, rot.cos, rot.sin, pos, ck2, cv2)
        assert got is not None and chain.supported, "the chain refused a shape it is meant for"
        torch.cuda.synchronize()
        assert torch.equal(x_sum, want_sum)
        assert torch.equal(ck2, ck) and torch.equal(cv2, cv)
        assert torch.equal(got, want), f"position {p}: {int((got != want).sum())} of {got.numel()} outputs differ"
    assert not hip_kernels.attention_chain_error(torch.device("cuda", torch.cuda.current_device()))


def test_chain_with_a_position_outside_the_cache_writes_nothing_and_ends():
    """pos lives in device memory: a step past the cache must leave the cache alone, and the blocks that wait for the
    heads must still be released."""
    from mixtral_offloading_amd import hip_kernels
    hidden, heads, kv, L = 4096, 32, 8, 256
    rng, group, do, rot, ck, cv, w = _setup(hidden, heads, kv, L, True, seed=5)
    chain = hip_kernels.AttentionChain(group, do)
    x = to_dev(rng.standard_normal((1, hidden)).astype(np.float16))
    before_k, before_v = ck.clone(), cv.clone()
    for p in (L, -1):
        got = chain(x, None, w, 1e-5, torch.empty_like(x), rot.cos, rot.sin, torch.tensor([p], device="cuda"), ck, cv)
        torch.cuda.synchronize()
        assert got is not None
        assert torch.equal(ck, before_k) and torch.equal(cv, before_v)
    # and the next launch in range is right: the counters were left at zero
    pos = torch.tensor([3], device="cuda")
    ck2, cv2 = ck.clone(), cv.clone()
    want, _ = _three_calls(group, do, rot, x, None, w, pos, ck, cv)
    got = chain(x, None, w, 1e-5, torch.empty_like(x), rot.cos, rot.sin, pos, ck2, cv2)
    assert torch.equal(got, want) and torch.equal(ck2, ck)
    assert not hip_kernels.attention_chain_error(torch.device("cuda", torch.cuda.current_device()))


def test_chain_refuses_what_it_does_not_take():
    from mixtral_offloading_amd import hip_kernels
    from mixtral_offloading_amd.mixtral_model import Rotary
    rng = np.random.default_rng(9)
    # heads of 64, and a hidden size whose projections do not run as 16 waves of one slab each: the three calls take
    # them, the chain does not
    for hidden, heads, kv, hd, L in [(512, 8, 8, 64, 128), (1024, 8, 2, 128, 128), (4096, 32, 8, 128, 1025)]:
        mk = lambda n, k: desc_of(o.random_layer(rng, n, k, 4, 64)[0])  # noqa: E731
        group = hip_kernels.LinearGroup([mk(heads * hd, hidden), mk(kv * hd, hidden), mk(kv * hd, hidden)])
        chain = hip_kernels.AttentionChain(group, mk(hidden, heads * hd))
        rot = Rotary(hd, L, 1e6, torch.device("cuda"))
        x = to_dev(rng.standard_normal((1, hidden)).astype(np.float16))
        w = to_dev(np.ones(hidden, dtype=np.float16))
        ck = torch.zeros((kv, L, hd), dtype=torch.float16, device="cuda")
        got = chain(x, None, w, 1e-5, torch.empty_like(x), rot.cos, rot.sin, torch.tensor([0], device="cuda"), ck, ck.clone())
        assert got is None and not chain.supported


def test_chain_replayed_from_a_graph():
    """Replays with the program's own eager work between them; every replay against the eager three calls."""
    from mixtral_offloading_amd import hip_kernels
    hidden, heads, kv, L = 4096, 32, 8, 512
    rng, group, do, rot, ck, cv, w = _setup(hidden, heads, kv, L, True, seed=77)
    chain = hip_kernels.AttentionChain(group, do)
    x = to_dev(rng.standard_normal((1, hidden)).astype(np.float16))
    d = to_dev(rng.standard_normal((1, hidden)).astype(np.float16))
    pos = torch.tensor([10], device="cuda")
    x_sum = torch.empty_like(x)
    ck2, cv2 = ck.clone(), cv.clone()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        for _ in range(2):
            chain(x, d, w, 1e-5, x_sum, rot.cos, rot.sin, pos, ck2, cv2)
    torch.cuda.current_stream().wait_stream(side)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        y = chain(x, d, w, 1e-5, x_sum, rot.cos, rot.sin, pos, ck2, cv2)
    ck.copy_(ck2), cv.copy_(cv2)  # the warm-up wrote position 10
    for p in (11, 12, 200, 511):
        pos.fill_(p)
        x.copy_(to_dev(rng.standard_normal((1, hidden)).astype(np.float16)))
        want, want_sum = _three_calls(group, do, rot, x, d, w, pos, ck, cv)
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(y, want) and torch.equal(x_sum, want_sum)
        assert torch.equal(ck2[:, p], ck[:, p]) and torch.equal(cv2[:, p], cv[:, p])
    assert not hip_kernels.attention_chain_error(torch.device("cuda", torch.cuda.current_device()))


def test_generate_notices_a_chain_that_gave_up_and_decodes_again_without_it():
    """The error word of the chained launch is forced from the host (no kernel ever gives up a wait in a test):
    generate() must notice it, clear it, stop chaining for the model and return the tokens of the three-launch path."""
    import warnings
    from mixtral_offloading_amd import _lib, build_model as bm, hip_kernels
    cfg = bm.mixtral_config(hidden_size=256, intermediate_size=512, num_hidden_layers=2, num_attention_heads=4,
                            num_key_value_heads=2, vocab_size=128, num_local_experts=8)
    off = bm.OffloadConfig(main_size=16, offload_size=0, buffer_size=1, offload_per_layer=0)
    dev = torch.device("cuda:0")
    model = bm.build_model(dev, bm.default_quant_config(), off, model_config=cfg, seed=5, max_positions=64)
    prompt = torch.arange(7, device="cuda")
    model.chain_attention = True
    want = model.generate(prompt, 6)
    assert not hip_kernels.attention_chain_error(dev)
    word_at = int(_lib.lib.hqq_attention_chain_error_offset())
    ws = hip_kernels.workspace(dev, word_at + 4)
    ws[word_at:word_at + 4].view(torch.int32).fill_(1)
    assert hip_kernels.attention_chain_error(dev)
    with warnings.catch_warnings(record=True) as caught:
        warnings.simplefilter("always")
        got = model.generate(prompt, 6)
    assert any("chained attention" in str(w.message) for w in caught)
    assert torch.equal(got, want)
    assert model.chain_attention is False and not hip_kernels.attention_chain_error(dev)
    torch.cuda.synchronize()
    assert not bool(ws[: 576 * 1024].any())  # the workspace head is at zero again for the launches that rely on it
