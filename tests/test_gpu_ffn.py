"""GPU parity tests of the expert FFN entry point (reference src/custom_layers.py:253-256, :308-312) against the
numpy oracle at small sizes, and against de-quantise-then-matmul on the GPU at Mixtral size."""
import numpy as np
import pytest
import torch

from helpers import assert_matmul_close, desc_of, to_dev
from oracle import hqq_oracle as o

pytestmark = pytest.mark.gpu

# (nbits, hidden, ffn, group_size, quant tables)
SHAPES = [
    (2, 256, 1024, 16, True),    # one slab in phase 1, four in phase 2
    (2, 1024, 3584, 16, True),   # G of the gate projections = 224 (table meta period that does not divide K)
    (2, 4096, 512, 16, True),    # sixteen slabs in phase 1: every wave busy
    (2, 512, 8192, 16, True),    # phase 2 split over two blocks per tile
    (4, 512, 1024, 64, True),    # four row blocks per tile
    (4, 256, 512, 32, False),    # fp16 tables
    (2, 768, 1280, 16, False),
    (3, 768, 1280, 64, True),    # 3-bit: both gate projections in one launch, silu(a) * b applied by the down projection
    (3, 1024, 2560, 32, True),   # K of the down projection split over blocks
    (3, 1280, 768, 64, False),   # fp16 tables
]


def _ffn_case(rng, nbits, hidden, ffn, gs, qt):
    w1, _ = o.random_layer(rng, ffn, hidden, nbits, gs, qt, qt)
    w3, _ = o.random_layer(rng, ffn, hidden, nbits, gs, qt, qt)
    w2, _ = o.random_layer(rng, hidden, ffn, nbits, gs, qt, qt)
    return w1, w2, w3


def _tolerance(x, w1, w2, w3):
    a = o.matmul_transpose(x, w1)
    b = o.matmul_transpose(x, w3)
    h = (o.silu_f16(a).astype(np.float32) * b.astype(np.float32)).astype(np.float16)
    # the intermediate h carries the tolerance of two matmuls already: allow 4x the single-matmul bound
    return 4 * o.matmul_tolerance(h, w2)


@pytest.mark.parametrize("shape", SHAPES, ids=lambda s: "w%d_h%d_f%d_g%d_%s" % (s[0], s[1], s[2], s[3], "q" if s[4] else "f16"))
@pytest.mark.parametrize("m", [1, 2, 3, 4, 7, 16, 40])
def test_expert_ffn_against_oracle(shape, m):
    from mixtral_offloading_amd import hip_kernels
    nbits, hidden, ffn, gs, qt = shape
    rng = np.random.default_rng(hidden + ffn + m)
    w1, w2, w3 = _ffn_case(rng, nbits, hidden, ffn, gs, qt)
    x = rng.standard_normal((m, hidden)).astype(np.float16)
    d1, d2, d3 = desc_of(w1), desc_of(w2), desc_of(w3)
    ref = o.expert_ffn(x, w1, w2, w3)
    atol = _tolerance(x, w1, w2, w3)
    for rep in range(3):  # the arrival counters must be left ready for the next call
        y = hip_kernels.expert_ffn(d1, d2, d3, to_dev(x)).cpu().numpy()
        assert_matmul_close(y, ref, atol, rtol=2e-2)


@pytest.mark.parametrize("nbits,hidden,ffn,gs", [(2, 512, 1792, 16), (3, 768, 1280, 64)])
@pytest.mark.parametrize("m", [1, 2, 3, 4, 8, 40, 130])
def test_expert_ffn_row_scale_and_accumulate(m, nbits, hidden, ffn, gs):
    """Routing weight and the index_add_ of the reference (src/custom_layers.py:308-312) as the FFN's epilogue."""
    from mixtral_offloading_amd import hip_kernels
    rng = np.random.default_rng(7 + m)
    w1, w2, w3 = _ffn_case(rng, nbits, hidden, ffn, gs, True)
    x = rng.standard_normal((m, hidden)).astype(np.float16)
    rw = rng.uniform(0.1, 0.9, size=(m,)).astype(np.float16)
    base = rng.standard_normal((m, hidden)).astype(np.float16)
    d1, d2, d3 = desc_of(w1), desc_of(w2), desc_of(w3)
    plain = hip_kernels.expert_ffn(d1, d2, d3, to_dev(x))
    out = to_dev(base.copy())
    hip_kernels.expert_ffn(d1, d2, d3, to_dev(x), out=out, row_scale=to_dev(rw), accumulate=True)
    # fp16 multiply by the routing weight, then fp16 add, exactly as the reference's ops would on the plain result
    want = to_dev(base) + plain * to_dev(rw)[:, None]
    assert torch.equal(out, want)


@pytest.mark.parametrize("nbits,gs", [(2, 16), (3, 64)])
@pytest.mark.parametrize("m", [1, 2, 4, 8])
def test_ffn_entry_point_equals_its_three_steps(m, nbits, gs):
    """hqq_expert_ffn rounds where the reference's three layers do (fp16 after each matmul, fp16 silu * up): it gives
    the bits that two hqq_matmul_transpose calls, torch's silu * up and a third call give, whatever kernels it picks."""
    from mixtral_offloading_amd import hip_kernels
    rng = np.random.default_rng(11 + m)
    w1, w2, w3 = _ffn_case(rng, nbits, 1024, 3584 if nbits == 2 else 2560, gs, True)
    x = to_dev(rng.standard_normal((m, 1024)).astype(np.float16))
    d1, d2, d3 = desc_of(w1), desc_of(w2), desc_of(w3)
    whole = hip_kernels.expert_ffn(d1, d2, d3, x)
    a, b = hip_kernels.matmul(d1, x), hip_kernels.matmul(d3, x)
    steps = hip_kernels.matmul(d2, torch.nn.functional.silu(a.float()).half() * b)
    err = (whole.float() - steps.float()).abs().max().item()
    # the gate kernel and the two single launches split K alike; silu is rounded once in both
    assert err <= 2e-3 * steps.float().abs().max().item() + 1e-3, err


@pytest.mark.parametrize("m", [1, 2, 3, 4, 8, 16, 128])
def test_full_size_ffn_against_dequantize_then_matmul(m):
    """Mixtral shapes (2-bit g16, 4096 -> 14336 -> 4096): the library's bit-exact de-quantiser followed by torch
    matmuls with the reference's fp16 roundings."""
    from mixtral_offloading_amd import hip_kernels
    from test_gpu_matmul import _full_size_layer
    d1 = _full_size_layer(2, 14336, 4096, 16, seed=1)
    d2 = _full_size_layer(2, 4096, 14336, 16, seed=2)
    d3 = _full_size_layer(2, 14336, 4096, 16, seed=3)
    g = torch.Generator(device="cuda").manual_seed(m)
    x = torch.randn((m, 4096), device="cuda", generator=g).half()
    wa, wb, wc = (hip_kernels.dequantize(d).float() for d in (d1, d3, d2))
    a = (x.float() @ wa.t()).half()
    b = (x.float() @ wb.t()).half()
    h = torch.nn.functional.silu(a) * b
    ref = h.float() @ wc.t()
    for rep in range(2):
        y = hip_kernels.expert_ffn(d1, d2, d3, x)
        err = (y.float() - ref).abs()
        atol = 4e-3 * h.float().norm(dim=1)[:, None] * wc.norm(dim=1)[None, :]
        bound = 2e-2 * ref.abs() + atol
        assert bool((err <= bound).all()), float((err / bound).max())


@pytest.mark.parametrize("shape", SHAPES, ids=lambda s: "w%d_h%d_f%d_g%d_%s" % (s[0], s[1], s[2], s[3], "q" if s[4] else "f16"))
@pytest.mark.parametrize("m", [1, 2, 4, 7, 16, 40])
def test_gate_up_entry_point(shape, m):
    """hqq_gate_up against the numpy oracle's silu(x w1^T) * (x w3^T) (reference src/custom_layers.py:254), and
    against the two projections done one by one on the GPU followed by torch's silu * up: the fused kernels round where
    those three steps round, so the two agree to an fp16 ulp of the larger values."""
    from mixtral_offloading_amd import hip_kernels
    nbits, hidden, ffn, gs, qt = shape
    rng = np.random.default_rng(3 * hidden + ffn + m)
    w1, _, w3 = _ffn_case(rng, nbits, hidden, ffn, gs, qt)
    x = rng.standard_normal((m, hidden)).astype(np.float16)
    d1, d3 = desc_of(w1), desc_of(w3)
    a = o.matmul_transpose(x, w1)
    b = o.matmul_transpose(x, w3)
    want = (o.silu_f16(a).astype(np.float32) * b.astype(np.float32)).astype(np.float16)
    ta, tb = o.matmul_tolerance(x, w1), o.matmul_tolerance(x, w3)
    # |d(silu(a) b)| <= |b| |da| * max|silu'| + |silu(a)| |db|, max|silu'| < 1.1
    atol = 1.1 * np.abs(b.astype(np.float32)) * ta + np.abs(o.silu_f16(a).astype(np.float32)) * tb + 1e-3
    xd = to_dev(x)
    for rep in range(2):
        got = hip_kernels.gate_up(d1, d3, xd)
        assert_matmul_close(got.cpu().numpy(), want, atol, rtol=2e-2)
    steps = torch.nn.functional.silu(hip_kernels.matmul(d1, xd).float()).half() * hip_kernels.matmul(d3, xd)
    err = (got.float() - steps.float()).abs().max().item()
    assert err <= 4e-3 * steps.float().abs().max().item() + 1e-3, err


def test_gate_up_refuses_bias_and_mismatched_layers():
    from mixtral_offloading_amd import _lib, hip_kernels
    rng = np.random.default_rng(5)
    w1, _ = o.random_layer(rng, 512, 256, 2, 16)
    w3, _ = o.random_layer(rng, 512, 256, 2, 16)
    other, _ = o.random_layer(rng, 768, 256, 2, 16)
    x = to_dev(rng.standard_normal((2, 256)).astype(np.float16))
    with pytest.raises(_lib.HqqError):
        hip_kernels.gate_up(desc_of(w1, bias=np.zeros(512, np.float16)), desc_of(w3), x)
    with pytest.raises(AssertionError):
        hip_kernels.gate_up(desc_of(w1), desc_of(other), x)
    assert hip_kernels.gate_up(desc_of(w1), desc_of(w3), x[:0]).shape == (0, 512)


@pytest.mark.parametrize("nbits,hidden,ffn,gs", [(2, 512, 1792, 16), (3, 768, 1280, 64), (4, 512, 1024, 64)])
def test_expert_groups_entry_point_equals_one_call_per_expert(nbits, hidden, ffn, gs):
    """The expert loop of a MoE layer as one call (reference src/custom_layers.py:298-312): rows grouped by expert,
    ragged groups (an empty one, one row, a decode batch, a prefill batch), every row scaled by its routing weight.
    The result is that of one hqq_expert_ffn call per expert, bit for bit, and agrees with the oracle."""
    from mixtral_offloading_amd import hip_kernels
    rng = np.random.default_rng(nbits + hidden)
    counts = [5, 0, 1, 40, 16, 3]
    experts = [_ffn_case(rng, nbits, hidden, ffn, gs, True) for _ in counts]
    descs = [tuple(desc_of(l) for l in e) for e in experts]
    group = hip_kernels.ExpertGroup(descs)
    starts = np.concatenate(([0], np.cumsum(counts)))
    rows = int(starts[-1])
    x = rng.standard_normal((rows, hidden)).astype(np.float16)
    scale = rng.uniform(0.2, 0.8, size=rows).astype(np.float16)
    xd, sd = to_dev(x), to_dev(scale)
    out = torch.full((rows, hidden), 7.0, dtype=torch.float16, device="cuda")
    hip_kernels.expert_groups_ffn(group, xd, starts, sd, out)
    each = torch.empty_like(out)
    for g, (w1, w2, w3) in enumerate(descs):
        lo, hi = int(starts[g]), int(starts[g + 1])
        if hi > lo:
            hip_kernels.expert_ffn(w1, w2, w3, xd[lo:hi], out=each[lo:hi], row_scale=sd[lo:hi])
    assert torch.equal(out, each)
    # without routing weights: against the oracle as well
    hip_kernels.expert_groups_ffn(group, xd, starts, None, out)
    got = out.cpu().numpy()
    for g, (w1, w2, w3) in enumerate(experts):
        lo, hi = int(starts[g]), int(starts[g + 1])
        if hi == lo:
            continue
        hip_kernels.expert_ffn(descs[g][0], descs[g][1], descs[g][2], xd[lo:hi], out=each[lo:hi])
        assert_matmul_close(got[lo:hi], o.expert_ffn(x[lo:hi], w1, w2, w3), _tolerance(x[lo:hi], w1, w2, w3), rtol=2e-2)
    assert torch.equal(out, each)
    # a row_start that does not begin at zero is refused
    with pytest.raises(AssertionError):
        hip_kernels.expert_groups_ffn(group, xd, starts + 1, None, out)


def test_expert_groups_at_full_size_leave_the_finishing_passes_to_the_end():
    """Mixtral-sized 2-bit experts with 17 to 64 rows each: their down projections split K, write their partial sums
    to places of their own and are finished by one launch at the end of the call.  Bit for bit what one call per
    expert gives, twice over (the second call finds the workspace as the first left it), and a decode-sized call in
    between on the same workspace."""
    from mixtral_offloading_amd import hip_kernels
    from test_gpu_matmul import _full_size_layer
    counts = [33, 20, 0, 64, 7, 40]
    descs = [(_full_size_layer(2, 14336, 4096, 16, seed=3 * e), _full_size_layer(2, 4096, 14336, 16, seed=3 * e + 1),
              _full_size_layer(2, 14336, 4096, 16, seed=3 * e + 2)) for e in range(len(counts))]
    group = hip_kernels.ExpertGroup(descs)
    starts = np.concatenate(([0], np.cumsum(counts)))
    rows = int(starts[-1])
    g = torch.Generator(device="cuda").manual_seed(11)
    x = torch.randn((rows, 4096), device="cuda", generator=g).half()
    scale = (torch.rand((rows,), device="cuda", generator=g) * 0.6 + 0.2).half()
    each = torch.empty((rows, 4096), dtype=torch.float16, device="cuda")
    for e, (w1, w2, w3) in enumerate(descs):
        lo, hi = int(starts[e]), int(starts[e + 1])
        if hi > lo:
            hip_kernels.expert_ffn(w1, w2, w3, x[lo:hi], out=each[lo:hi], row_scale=scale[lo:hi])
    assert bool(torch.isfinite(each).all()) and float(each.float().abs().max()) > 0
    for rep in range(2):
        out = torch.full((rows, 4096), 3.0, dtype=torch.float16, device="cuda")
        hip_kernels.expert_groups_ffn(group, x, starts, scale, out)
        assert torch.equal(out, each)
        one = hip_kernels.expert_ffn(descs[0][0], descs[0][1], descs[0][2], x[:1].contiguous())
        assert bool(torch.isfinite(one).all())
