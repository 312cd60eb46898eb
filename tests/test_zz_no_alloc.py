"""GPU test of hqq_expert_ffn_static, the expert FFN on the library's built-in scratch (for callers that cannot
allocate): its output must equal hqq_expert_ffn's bit for bit, on two calls in a row, the second with a smaller
input, from two streams, and replayed from a graph; it must allocate nothing, and sizes beyond the built-in scratch
must be rejected."""
import numpy as np
import pytest
import torch

from helpers import desc_of, to_dev
from oracle import hqq_oracle as o

pytestmark = pytest.mark.gpu


def _experts(rng, nbits, hidden, ffn, gs):
    w1, _ = o.random_layer(rng, ffn, hidden, nbits, gs, True, True)
    w3, _ = o.random_layer(rng, ffn, hidden, nbits, gs, True, True)
    w2, _ = o.random_layer(rng, hidden, ffn, nbits, gs, True, True)
    return desc_of(w1), desc_of(w2), desc_of(w3)


@pytest.mark.parametrize("nbits,gs", [(2, 16), (3, 64), (4, 64)])
def test_static_scratch_ffn_equals_workspace_ffn(nbits, gs):
    from mixtral_offloading_amd import hip_kernels
    rng = np.random.default_rng(100 + nbits)
    # first call: four rows, the down projection's K split over blocks (accumulation slots in the scratch head);
    # second call: one row of a smaller expert
    for m, hidden, ffn in ((4, 1024, 3584), (1, 512, 1792)):
        d1, d2, d3 = _experts(rng, nbits, hidden, ffn, gs)
        x = to_dev(rng.standard_normal((m, hidden)).astype(np.float16))
        rw = to_dev(rng.uniform(0.1, 0.9, size=(m,)).astype(np.float16))
        base = to_dev(rng.standard_normal((m, hidden)).astype(np.float16))
        want = hip_kernels.expert_ffn(d1, d2, d3, x)
        got = torch.full_like(want, float("nan"))
        hip_kernels.expert_ffn_static(d1, d2, d3, x, got)
        assert torch.equal(got, want)
        want_acc = hip_kernels.expert_ffn(d1, d2, d3, x, out=base.clone(), row_scale=rw, accumulate=True)
        got_acc = hip_kernels.expert_ffn_static(d1, d2, d3, x, base.clone(), row_scale=rw, accumulate=True)
        assert torch.equal(got_acc, want_acc)


def test_static_scratch_ffn_at_mixtral_size_and_its_limit():
    """Four rows, then one row, at Mixtral-8x7B expert size; then a batch whose workspace exceeds the built-in scratch."""
    from mixtral_offloading_amd import _lib, hip_kernels
    from test_gpu_matmul import _full_size_layer
    d1 = _full_size_layer(2, 14336, 4096, 16, seed=1)
    d3 = _full_size_layer(2, 14336, 4096, 16, seed=2)
    d2 = _full_size_layer(2, 4096, 14336, 16, seed=3)
    for m in (4, 1):
        x = torch.randn((m, 4096), device="cuda").half()
        want = hip_kernels.expert_ffn(d1, d2, d3, x)
        got = torch.empty_like(want)
        hip_kernels.expert_ffn_static(d1, d2, d3, x, got)
        assert torch.equal(got, want)
    m = 128
    assert _lib.lib.hqq_expert_ffn_workspace_bytes(d1.ref, d2.ref, d3.ref, m) > hip_kernels.STATIC_SCRATCH_BYTES
    x = torch.randn((m, 4096), device="cuda").half()
    with pytest.raises(_lib.HqqError) as err:
        hip_kernels.expert_ffn_static(d1, d2, d3, x, torch.empty((m, 4096), device="cuda", dtype=torch.float16))
    assert err.value.code == -5


def test_static_scratch_ffn_from_two_streams_one_after_the_other():
    """Calls that do not overlap may come from different streams: nothing the entry point does is tied to the
    stream of the first call on a device."""
    from mixtral_offloading_amd import hip_kernels
    rng = np.random.default_rng(7)
    d1, d2, d3 = _experts(rng, 2, 1024, 3584, 16)
    x = to_dev(rng.standard_normal((4, 1024)).astype(np.float16))
    want = hip_kernels.expert_ffn(d1, d2, d3, x)
    torch.cuda.synchronize()
    for _ in range(3):
        for stream in (torch.cuda.Stream(), torch.cuda.Stream()):
            got = torch.full_like(want, float("nan"))
            with torch.cuda.stream(stream):
                hip_kernels.expert_ffn_static(d1, d2, d3, x, got)
            stream.synchronize()
            assert torch.equal(got, want)


def test_static_scratch_ffn_allocates_nothing_and_replays_from_a_graph():
    """Device memory in use does not change across calls, and a captured call gives the eager result on every replay,
    with eager calls of the same entry point and synchronisations between the replays."""
    from mixtral_offloading_amd import hip_kernels
    rng = np.random.default_rng(8)
    d1, d2, d3 = _experts(rng, 2, 1024, 3584, 16)
    xs = [to_dev(rng.standard_normal((m, 1024)).astype(np.float16)) for m in (4, 1)]
    wants = [hip_kernels.expert_ffn(d1, d2, d3, x) for x in xs]
    outs = [torch.empty_like(w) for w in wants]
    hip_kernels.expert_ffn_static(d1, d2, d3, xs[0], outs[0])  # the first call on the device is not captured
    torch.cuda.synchronize()
    free_before, _ = torch.cuda.mem_get_info()
    for x, out in zip(xs, outs):
        hip_kernels.expert_ffn_static(d1, d2, d3, x, out)
    torch.cuda.synchronize()
    free_after, _ = torch.cuda.mem_get_info()
    assert free_after == free_before
    for out, want in zip(outs, wants):
        assert torch.equal(out, want)
    side = torch.cuda.Stream()
    graph = torch.cuda.CUDAGraph()
    captured = [torch.empty_like(w) for w in wants]
    with torch.cuda.stream(side):
        with torch.cuda.graph(graph, stream=side):
            for x, out in zip(xs, captured):
                hip_kernels.expert_ffn_static(d1, d2, d3, x, out)
    for rep in range(4):
        for out in captured:
            out.fill_(float("nan"))
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        for out, want in zip(captured, wants):
            assert torch.equal(out, want), rep
        eager = torch.empty_like(wants[1])
        hip_kernels.expert_ffn_static(d1, d2, d3, xs[1], eager)  # eager work on the same scratch between replays
        torch.cuda.synchronize()
        assert torch.equal(eager, wants[1])
