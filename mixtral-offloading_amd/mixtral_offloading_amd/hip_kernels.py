"""Host side of the unpack-dequantise-matmul kernels.

Keeps the call signatures of the reference's ``src/triton_kernels.py``
wrappers (``triton_matmul4_transpose`` at :133, ``triton_matmul2_transpose``
at :321, ``triton_matmul3_transpose`` at :511) and adds the fused entry the
module layer uses, where the 8-bit scale / zero tables are de-quantised inside
the kernel instead of being expanded to fp16 first
(src/custom_layers.py:62-66)."""
from __future__ import annotations

import ctypes
from typing import Optional

import torch

from . import _lib
from ._lib import HqqLinear, HqqTable

_workspaces = {}


class _Stay:
    def __enter__(self):
        return self

    def __exit__(self, *exc):
        return False


_STAY = _Stay()


def _on(device: torch.device):
    """Context that makes ``device`` current for the launches inside; free when it already is."""
    if device.index is None or torch.cuda.current_device() == device.index:
        return _STAY
    return torch.cuda.device(device)


kHeadReserve = 1 << 20  # the head of a workspace belongs to the kernels' counters and slots: other scratch goes past it


def workspace(device: torch.device, nbytes: int) -> torch.Tensor:
    """Per (device, stream) scratch for split-K partial sums; grows on demand.
    Calls on one stream are ordered, so sharing it between them is safe."""
    key = (device.index, torch.cuda.current_stream(device).cuda_stream)
    buf = _workspaces.get(key)
    if buf is None or buf.numel() < nbytes:
        # zero-filled: the head of a workspace holds arrival counters that must start at zero
        buf = torch.zeros(max(int(nbytes), 1 << 20), dtype=torch.uint8, device=device)
        _workspaces[key] = buf
    return buf


def _table(values: torch.Tensor, meta: Optional[dict]) -> tuple:
    """(HqqTable, keep-alive) for a scale or zero table: fp16 values, or uint8
    codes plus the fp16 meta pair of ``Quantizer.quantize``."""
    t = HqqTable()
    if meta is None:
        assert values.dtype == torch.float16, "scale/zero tables must be fp16"
        v = values.contiguous()
        t.data, t.kind, t.meta_cols = v.data_ptr(), _lib.HQQ_TABLE_F16, 0
        return t, (v,)
    assert values.dtype == torch.uint8, "8-bit scale/zero codes must be uint8"
    v = values.contiguous()
    ms = meta["scale"].to(torch.float16).contiguous()
    mz = meta["zero"].to(torch.float16).contiguous()
    assert ms.numel() == mz.numel()
    t.data, t.kind = v.data_ptr(), _lib.HQQ_TABLE_U8
    t.meta_scale, t.meta_zero, t.meta_cols = ms.data_ptr(), mz.data_ptr(), ms.numel()
    return t, (v, ms, mz)


class LinearDesc:
    """``hqq_linear`` descriptor of one layer plus the tensors it points into."""

    def __init__(self, W_q: torch.Tensor, meta: dict, bias: Optional[torch.Tensor] = None,
                 scale: Optional[torch.Tensor] = None, zero: Optional[torch.Tensor] = None):
        N, K = int(meta["shape"][0]), int(meta["shape"][1])
        nbits = int(meta["nbits"])
        codes = W_q.contiguous()
        if nbits == 3:
            assert codes.dtype == torch.int32
            assert 0 <= codes.numel() // K * 10 - N < 10  # reference src/triton_kernels.py:536
        else:
            assert codes.dtype == torch.uint8
            assert codes.numel() == N * K * nbits // 8, "codes are not in the kernel layout (call repack)"
        if scale is None:
            scale_t, keep_s = (_table(meta["scale_q"], meta["meta_scale"]) if meta.get("quant_scale")
                               else _table(meta["scale"], None))
        else:
            scale_t, keep_s = _table(scale, None)
        if zero is None:
            zero_t, keep_z = (_table(meta["zero_q"], meta["meta_zero"]) if meta.get("quant_zero")
                              else _table(meta["zero"], None))
        else:
            zero_t, keep_z = _table(zero, None)
        s_cnt = N * K // int(meta["group_size"])
        for kp in (keep_s, keep_z):
            assert kp[0].numel() == s_cnt, "scale/zero table does not have N*K/group_size entries"
        d = HqqLinear()
        d.nbits, d.group_size, d.N, d.K = nbits, int(meta["group_size"]), N, K
        d.codes, d.scale, d.zero = codes.data_ptr(), scale_t, zero_t
        b = None
        if bias is not None:
            b = bias.to(torch.float16).contiguous().view(-1)
            assert b.numel() == N
            d.bias = b.data_ptr()
        self.c = d
        self.N, self.K, self.nbits = N, K, nbits
        self.device = codes.device
        self._keep = (codes, keep_s, keep_z, b)

    @property
    def ref(self):
        return ctypes.byref(self.c)


def matmul(desc: LinearDesc, a: torch.Tensor, family: int = -1) -> torch.Tensor:
    """C = a @ dequant(W).T (+ bias) on the GPU; fp16 in, fp16 out."""
    assert a.shape[-1] == desc.K  # reference src/triton_kernels.py:150
    assert a.is_contiguous(), "A must be contiguous"  # :151
    assert a.dtype == torch.float16 and a.is_cuda and a.device == desc.device
    x = a.view(-1, desc.K)
    M = x.shape[0]
    c = torch.empty((M, desc.N), device=a.device, dtype=torch.float16)
    if M > 0:
        with _on(a.device):
            need = _lib.lib.hqq_matmul_workspace_bytes(desc.ref, M)
            if family == _lib.FAM_DQGEMM:  # forced below the batch size it is chosen from: room for the fp16 weights
                need = max(need, 2 * desc.N * desc.K + (1 << 20))
            ws = workspace(a.device, need)
            _lib.check(_lib.lib.hqq_matmul_transpose_ex(desc.ref, x.data_ptr(), M, c.data_ptr(), ws.data_ptr(),
                                                        ws.numel(), family, _lib.current_stream_ptr(a.device)),
                       "hqq_matmul_transpose")
    return c.view(a.shape[:-1] + (desc.N,))


def kernel_family(desc: LinearDesc, M: int) -> int:
    return _lib.lib.hqq_matmul_kernel_family(desc.ref, M)


def _matmul_fp16_tables(nbits, groupsize, a, qweight, scales, zeros, N, bias):
    assert scales.shape[1] == zeros.shape[1]  # reference src/triton_kernels.py:152
    assert scales.shape[1] == qweight.shape[1]  # :153
    K = qweight.shape[1]
    meta = {"nbits": nbits, "group_size": groupsize, "shape": (N, K)}
    desc = LinearDesc(qweight, meta, None, scale=scales, zero=zeros)
    c = matmul(desc, a)
    if bias is not None:
        c = c + bias  # reference :188-189
    return c


def hip_matmul4_transpose(groupsize: int, a, qweight, scales, zeros, bias=None):
    """Drop-in for ``triton_matmul4_transpose`` (reference src/triton_kernels.py:133-191):
    ``a`` (..., K) fp16, ``qweight`` (N//2, K) uint8, ``scales`` / ``zeros`` (G, K) fp16."""
    return _matmul_fp16_tables(4, groupsize, a, qweight, scales, zeros, qweight.shape[0] * 2, bias)


def hip_matmul2_transpose(groupsize: int, a, qweight, scales, zeros, bias=None):
    """Drop-in for ``triton_matmul2_transpose`` (reference src/triton_kernels.py:321-380)."""
    return _matmul_fp16_tables(2, groupsize, a, qweight, scales, zeros, qweight.shape[0] * 4, bias)


def hip_matmul3_transpose(groupsize: int, a, qweight, scales, zeros, N: int, bias=None):
    """Drop-in for ``triton_matmul3_transpose`` (reference src/triton_kernels.py:511-564)."""
    assert 0 <= (qweight.shape[0] * 10 - N) < 10  # :536
    return _matmul_fp16_tables(3, groupsize, a, qweight, scales, zeros, N, bias)


# the reference's names, so call sites need no edit
triton_matmul4_transpose = hip_matmul4_transpose
triton_matmul2_transpose = hip_matmul2_transpose
triton_matmul3_transpose = hip_matmul3_transpose


def dequantize(desc: LinearDesc) -> torch.Tensor:
    w = torch.empty((desc.N, desc.K), dtype=torch.float16, device=desc.device)
    with _on(desc.device):
        _lib.check(_lib.lib.hqq_dequantize(desc.ref, w.data_ptr(), _lib.current_stream_ptr(desc.device)),
                   "hqq_dequantize")
    return w


def table_to_f16(values: torch.Tensor, meta: dict) -> torch.Tensor:
    """``Quantizer.dequantize`` of an 8-bit scale / zero table (reference src/custom_layers.py:63-66)."""
    t, keep = _table(values, meta)
    out = torch.empty(meta["shape"] if "shape" in meta else values.shape, dtype=torch.float16, device=values.device)
    with _on(values.device):
        _lib.check(_lib.lib.hqq_table_to_f16(ctypes.byref(t), values.numel(), out.data_ptr(),
                                             _lib.current_stream_ptr(values.device)), "hqq_table_to_f16")
    del keep
    return out


def expert_ffn(w1: LinearDesc, w2: LinearDesc, w3: LinearDesc, x: torch.Tensor, out: Optional[torch.Tensor] = None,
               row_scale: Optional[torch.Tensor] = None, accumulate: bool = False) -> torch.Tensor:
    """w2(silu(w1 x) * w3 x), optionally scaled per row and accumulated into ``out``
    (reference src/custom_layers.py:253-256, :308-312)."""
    assert x.dtype == torch.float16 and x.is_contiguous() and x.shape[-1] == w1.K
    xv = x.view(-1, w1.K)
    M = xv.shape[0]
    if out is None:
        assert not accumulate
        out = torch.empty((M, w2.N), dtype=torch.float16, device=x.device)
    assert out.is_contiguous() and out.numel() == M * w2.N
    if M == 0:
        return out
    if row_scale is not None:
        row_scale = row_scale.to(torch.float16).contiguous()
        assert row_scale.numel() == M
    with _on(x.device):
        need = _lib.lib.hqq_expert_ffn_workspace_bytes(w1.ref, w2.ref, w3.ref, M)
        ws = workspace(x.device, need)
        _lib.check(_lib.lib.hqq_expert_ffn(w1.ref, w2.ref, w3.ref, xv.data_ptr(), M, out.data_ptr(),
                                           row_scale.data_ptr() if row_scale is not None else None,
                                           int(accumulate), ws.data_ptr(), ws.numel(),
                                           _lib.current_stream_ptr(x.device)), "hqq_expert_ffn")
    return out


class ExpertGroup:
    """The layers of a MoE layer's experts as the pointer arrays ``expert_groups_ffn`` takes (built once per layer;
    the descriptors are kept alive here)."""

    def __init__(self, experts):
        self.descs = [tuple(e) for e in experts]  # (w1, w2, w3) LinearDesc per expert
        n = len(self.descs)
        arr = ctypes.c_void_p * n
        self.w1 = arr(*[ctypes.addressof(d[0].c) for d in self.descs])
        self.w2 = arr(*[ctypes.addressof(d[1].c) for d in self.descs])
        self.w3 = arr(*[ctypes.addressof(d[2].c) for d in self.descs])
        self.n = n
        self.K, self.N = self.descs[0][0].K, self.descs[0][1].N


def expert_groups_ffn(group: ExpertGroup, x: torch.Tensor, row_start, row_scale: Optional[torch.Tensor],
                      out: torch.Tensor) -> torch.Tensor:
    """Rows ``row_start[g] .. row_start[g + 1] - 1`` of ``x`` through expert ``g``, scaled per row, into ``out``: the
    expert loop of the reference's ``SparseMoeWrapper.forward`` (src/custom_layers.py:298-312) as one library call."""
    assert x.dtype == torch.float16 and x.is_contiguous() and x.shape[-1] == group.K
    rows = x.numel() // group.K
    assert out.dtype == torch.float16 and out.is_contiguous() and out.numel() == rows * group.N
    assert len(row_start) == group.n + 1 and int(row_start[0]) == 0 and int(row_start[-1]) == rows
    assert row_scale is None or (row_scale.dtype == torch.float16 and row_scale.is_contiguous() and row_scale.numel() == rows)
    starts = (ctypes.c_int64 * (group.n + 1))(*[int(v) for v in row_start])
    with _on(x.device):
        need = _lib.lib.hqq_expert_groups_ffn_workspace_bytes(group.w1, group.w2, group.w3, group.n, starts)
        if rows and need == 0:
            raise _lib.HqqError(-6, "hqq_expert_groups_ffn_workspace_bytes")
        ws = workspace(x.device, max(need, 1))
        _lib.check(_lib.lib.hqq_expert_groups_ffn(group.w1, group.w2, group.w3, group.n, starts, x.data_ptr(), out.data_ptr(),
                                                  row_scale.data_ptr() if row_scale is not None else None,
                                                  ws.data_ptr(), ws.numel(), _lib.current_stream_ptr(x.device)),
                   "hqq_expert_groups_ffn")
    return out


STATIC_SCRATCH_BYTES = 16 << 20  # HQQ_STATIC_SCRATCH_BYTES of include/hqq_mi355x.h


def expert_ffn_static(w1: LinearDesc, w2: LinearDesc, w3: LinearDesc, x: torch.Tensor, out: torch.Tensor,
                      row_scale: Optional[torch.Tensor] = None, accumulate: bool = False) -> torch.Tensor:
    """``expert_ffn`` on the library's built-in scratch: nothing is allocated, here or in the library, so ``out`` is
    the caller's.  Raises ``HqqError`` (workspace) when the batch needs more than ``STATIC_SCRATCH_BYTES``."""
    assert x.dtype == torch.float16 and x.is_contiguous() and x.shape[-1] == w1.K
    M = x.numel() // w1.K
    assert out.is_contiguous() and out.numel() == M * w2.N and out.dtype == torch.float16
    assert row_scale is None or (row_scale.dtype == torch.float16 and row_scale.is_contiguous() and row_scale.numel() == M)
    with _on(x.device):
        _lib.check(_lib.lib.hqq_expert_ffn_static(w1.ref, w2.ref, w3.ref, x.data_ptr(), M, out.data_ptr(),
                                                  row_scale.data_ptr() if row_scale is not None else None,
                                                  int(accumulate), _lib.current_stream_ptr(x.device)),
                   "hqq_expert_ffn_static")
    return out


def gate_up(w1: LinearDesc, w3: LinearDesc, x: torch.Tensor) -> torch.Tensor:
    """``silu(w1 x) * (w3 x)``, the first half of the expert FFN (reference src/custom_layers.py:254)."""
    assert x.dtype == torch.float16 and x.is_contiguous() and x.shape[-1] == w1.K == w3.K and w1.N == w3.N
    xv = x.view(-1, w1.K)
    M = xv.shape[0]
    out = torch.empty((M, w1.N), dtype=torch.float16, device=x.device)
    if M == 0:
        return out
    with _on(x.device):
        ws = workspace(x.device, _lib.lib.hqq_gate_up_workspace_bytes(w1.ref, w3.ref, M))
        _lib.check(_lib.lib.hqq_gate_up(w1.ref, w3.ref, xv.data_ptr(), M, out.data_ptr(), ws.data_ptr(), ws.numel(),
                                        _lib.current_stream_ptr(x.device)), "hqq_gate_up")
    return out


class ExpertTable:
    """Device-resident table of the experts of one MoE layer for ``expert_ffn_indexed``: three records per expert
    (w1, w3, w2).  ``experts`` is a list of (w1, w2, w3) ``LinearDesc`` triples that all share one shape."""

    def __init__(self, experts):
        rec = _lib.lib.hqq_expert_record_bytes()
        host = (ctypes.c_uint8 * (rec * 3 * len(experts)))()
        base = ctypes.addressof(host)
        for e, (w1, w2, w3) in enumerate(experts):
            for j, d in enumerate((w1, w3, w2)):
                _lib.check(_lib.lib.hqq_expert_record_fill(d.ref, base + (3 * e + j) * rec), "hqq_expert_record_fill")
        self.shape = experts[0]
        self.device = experts[0][0].device
        self.table = torch.frombuffer(host, dtype=torch.uint8).clone().to(self.device)
        self._keep = list(experts)


def expert_ffn_indexed(table: ExpertTable, expert_index: torch.Tensor, x: torch.Tensor, out: torch.Tensor,
                       row_scale: Optional[torch.Tensor] = None, accumulate: bool = False) -> torch.Tensor:
    """``expert_ffn`` of expert ``expert_index[0]`` (an int32 device tensor) of the table: no host synchronisation."""
    w1, w2, w3 = table.shape
    assert x.dtype == torch.float16 and x.is_contiguous() and x.shape[-1] == w1.K
    assert expert_index.dtype == torch.int32 and expert_index.is_cuda
    M = x.numel() // w1.K
    assert out.is_contiguous() and out.numel() == M * w2.N and out.dtype == torch.float16
    with _on(x.device):
        need = _lib.lib.hqq_expert_ffn_workspace_bytes(w1.ref, w2.ref, w3.ref, M)
        ws = workspace(x.device, need)
        _lib.check(_lib.lib.hqq_expert_ffn_indexed(w1.ref, w2.ref, w3.ref, table.table.data_ptr(),
                                                   expert_index.data_ptr(), x.data_ptr(), M, out.data_ptr(),
                                                   row_scale.data_ptr() if row_scale is not None else None,
                                                   int(accumulate), ws.data_ptr(), ws.numel(),
                                                   _lib.current_stream_ptr(x.device)), "hqq_expert_ffn_indexed")
    return out


def expert_pair_supported(table: ExpertTable) -> bool:
    """Whether ``expert_pair_ffn_indexed`` takes the experts of this table."""
    w1, w2, w3 = table.shape
    return _lib.lib.hqq_expert_pair_ffn_workspace_bytes(w1.ref, w2.ref, w3.ref) > 0


def moe_pair_routed_supported(table: ExpertTable, hidden: int, n_experts: int) -> bool:
    """Whether ``moe_pair_routed`` takes this layer: the two-launch pair, 2- or 4-bit experts, a row of at most 4096."""
    return (expert_pair_supported(table) and table.shape[0].nbits != 3 and hidden <= 4096 and hidden % 8 == 0
            and 2 <= n_experts <= 8)


def expert_pair_ffn_indexed(table: ExpertTable, expert_index: torch.Tensor, x: torch.Tensor, out: torch.Tensor,
                            row_scale: torch.Tensor, accumulate: bool = False) -> torch.Tensor:
    """``out (+)= sum_e expert_ffn_{expert_index[e]}(x) * row_scale[e]`` over the two active experts of one token
    (reference src/custom_layers.py:298-312) in two launches; ``expert_index`` int32[2] and ``row_scale`` fp16[2] are
    device tensors, as ``router_top2`` writes them."""
    w1, w2, w3 = table.shape
    assert x.dtype == torch.float16 and x.is_contiguous() and x.numel() == w1.K
    assert expert_index.dtype == torch.int32 and expert_index.is_cuda and expert_index.numel() >= 2
    assert row_scale.dtype == torch.float16 and row_scale.is_cuda and row_scale.numel() >= 2
    assert out.is_contiguous() and out.numel() == w2.N and out.dtype == torch.float16
    with _on(x.device):
        need = _lib.lib.hqq_expert_pair_ffn_workspace_bytes(w1.ref, w2.ref, w3.ref)
        ws = workspace(x.device, need)
        _lib.check(_lib.lib.hqq_expert_pair_ffn_indexed(w1.ref, w2.ref, w3.ref, table.table.data_ptr(),
                                                        expert_index.data_ptr(), x.data_ptr(), out.data_ptr(),
                                                        row_scale.data_ptr(), int(accumulate), ws.data_ptr(), ws.numel(),
                                                        _lib.current_stream_ptr(x.device)), "hqq_expert_pair_ffn_indexed")
    return out


def moe_pair_routed(table: ExpertTable, x: torch.Tensor, delta: Optional[torch.Tensor], weight: torch.Tensor, eps: float,
                    x_sum: torch.Tensor, gate_weight: torch.Tensor, sel: torch.Tensor, weights: torch.Tensor,
                    out: torch.Tensor, accumulate: bool = False) -> torch.Tensor:
    """``add_rmsnorm_router`` and ``expert_pair_ffn_indexed`` in two launches: the norm of ``x + delta`` and the router
    run in front of the gates of the two experts they choose.  ``x + delta`` goes to ``x_sum`` (not ``x`` itself)."""
    w1, w2, w3 = table.shape
    n_experts, hidden = gate_weight.shape
    assert x.dtype == torch.float16 and x.is_contiguous() and x.numel() == w1.K == hidden
    assert x_sum.dtype == torch.float16 and x_sum.numel() == hidden and x_sum.data_ptr() != x.data_ptr()
    assert weight.dtype == torch.float16 and weight.numel() == hidden and gate_weight.dtype == torch.float16
    assert gate_weight.is_contiguous() and sel.dtype == torch.int32 and sel.numel() >= 2
    assert weights.dtype == torch.float16 and weights.numel() >= 2
    assert out.is_contiguous() and out.numel() == w2.N and out.dtype == torch.float16
    with _on(x.device):
        need = _lib.lib.hqq_expert_pair_ffn_workspace_bytes(w1.ref, w2.ref, w3.ref)
        ws = workspace(x.device, need)
        _lib.check(_lib.lib.hqq_moe_pair_routed(w1.ref, w2.ref, w3.ref, table.table.data_ptr(), x.data_ptr(),
                                                delta.data_ptr() if delta is not None else None, weight.data_ptr(),
                                                float(eps), x_sum.data_ptr(), gate_weight.data_ptr(), n_experts,
                                                sel.data_ptr(), weights.data_ptr(), out.data_ptr(), int(accumulate),
                                                ws.data_ptr(), ws.numel(), _lib.current_stream_ptr(x.device)),
                   "hqq_moe_pair_routed")
    return out


class LinearGroup:
    """Up to four layers applied to the same single row in one launch (``hqq_matmul_group``): the q, k and v
    projections of an attention block.  ``supported`` is False when the layers do not fit one launch."""

    def __init__(self, descs):
        self.descs = list(descs)
        n = len(self.descs)
        self._ptrs = (ctypes.POINTER(_lib.HqqLinear) * n)(*[ctypes.pointer(d.c) for d in self.descs])
        self.need = int(_lib.lib.hqq_matmul_group_workspace_bytes(self._ptrs, n)) if 1 <= n <= 4 else 0
        self.supported = self.need > 0

    def __call__(self, x: torch.Tensor):
        d0 = self.descs[0]
        assert x.dtype == torch.float16 and x.is_contiguous() and x.numel() == d0.K and x.device == d0.device
        outs = [torch.empty((1, d.N), device=x.device, dtype=torch.float16) for d in self.descs]
        ys = (ctypes.c_void_p * len(outs))(*[o.data_ptr() for o in outs])
        with _on(x.device):
            ws = workspace(x.device, self.need)
            _lib.check(_lib.lib.hqq_matmul_group(self._ptrs, len(outs), x.data_ptr(), ys, ws.data_ptr(), ws.numel(),
                                                 _lib.current_stream_ptr(x.device)), "hqq_matmul_group")
        return outs


def matmul_group_norm(group: LinearGroup, x: torch.Tensor, delta: Optional[torch.Tensor], weight: torch.Tensor,
                      eps: float, x_sum: torch.Tensor):
    """``add_rmsnorm`` folded into the grouped launch: returns the group's outputs for the row
    ``weight * rmsnorm(x + delta)`` and writes ``x + delta`` to ``x_sum`` (which must not be ``x``)."""
    d0 = group.descs[0]
    assert x.dtype == torch.float16 and x.is_contiguous() and x.numel() == d0.K and x.device == d0.device
    assert x_sum.dtype == torch.float16 and x_sum.numel() == d0.K and x_sum.data_ptr() != x.data_ptr()
    assert weight.dtype == torch.float16 and weight.numel() == d0.K
    outs = [torch.empty((1, d.N), device=x.device, dtype=torch.float16) for d in group.descs]
    ys = (ctypes.c_void_p * len(outs))(*[o.data_ptr() for o in outs])
    with _on(x.device):
        ws = workspace(x.device, group.need)
        _lib.check(_lib.lib.hqq_matmul_group_norm(group._ptrs, len(outs), x.data_ptr(),
                                                  delta.data_ptr() if delta is not None else None, weight.data_ptr(),
                                                  float(eps), x_sum.data_ptr(), ys, ws.data_ptr(), ws.numel(),
                                                  _lib.current_stream_ptr(x.device)), "hqq_matmul_group_norm")
    return outs


QUANTIZE_GROUP_SIZES = (8, 16, 32, 64, 128)


def quantize_groups(w: torch.Tensor, group_size: int, nbits: int, round_zero: bool = False, iters: int = 0,
                    lp_norm: float = 0.7, beta: float = 10.0, kappa: float = 1.01):
    """hqq's ``Quantizer.quantize`` for ``axis=0`` grouping on the GPU (``hqq_quantize_groups``): ``w`` (fp16 or fp32,
    contiguous, any shape) is read as ``(group_size, numel / group_size)`` whose columns are the groups.  ``iters`` > 0
    runs hqq's solver for the zero point.  Returns ``(codes uint8 (group_size, cols), scale fp32 (1, cols), zero fp32
    (1, cols))`` with ``scale`` already inverted, as hqq's meta holds it."""
    assert w.is_cuda and w.is_contiguous() and w.dtype in (torch.float16, torch.float32)
    assert group_size in QUANTIZE_GROUP_SIZES and w.numel() % group_size == 0 and w.numel() > 0
    cols = w.numel() // group_size
    codes = torch.empty((group_size, cols), dtype=torch.uint8, device=w.device)
    scale = torch.empty((1, cols), dtype=torch.float32, device=w.device)
    zero = torch.empty((1, cols), dtype=torch.float32, device=w.device)
    with _on(w.device):
        ws = workspace(w.device, int(_lib.lib.hqq_quantize_workspace_bytes()) + kHeadReserve)
        # past the head of the shared workspace (counters that must stay zero between launches)
        base = ws.data_ptr() + kHeadReserve
        _lib.check(_lib.lib.hqq_quantize_groups(w.data_ptr(), int(w.dtype == torch.float32), group_size, cols, nbits,
                                                int(bool(round_zero)), int(iters), float(lp_norm), float(beta), float(kappa),
                                                codes.data_ptr(), scale.data_ptr(), zero.data_ptr(), base,
                                                ws.numel() - kHeadReserve, _lib.current_stream_ptr(w.device)),
                   "hqq_quantize_groups")
    return codes, scale, zero


def quantize_whole(x: torch.Tensor, nbits: int):
    """``Quantizer.quantize(channel_wise=False)`` on the GPU: one scale and zero for the whole fp32 tensor.
    Returns ``(codes uint8 of x's shape, scale fp32 scalar tensor (inverted), zero fp32 scalar tensor)``."""
    assert x.is_cuda and x.is_contiguous() and x.dtype == torch.float32 and x.numel() > 0
    codes = torch.empty(x.shape, dtype=torch.uint8, device=x.device)
    sz = torch.empty(2, dtype=torch.float32, device=x.device)
    with _on(x.device):
        ws = workspace(x.device, int(_lib.lib.hqq_quantize_workspace_bytes()) + kHeadReserve)
        _lib.check(_lib.lib.hqq_quantize_whole(x.data_ptr(), x.numel(), nbits, codes.data_ptr(), sz[0:1].data_ptr(),
                                               sz[1:2].data_ptr(), ws.data_ptr() + kHeadReserve, ws.numel() - kHeadReserve,
                                               _lib.current_stream_ptr(x.device)), "hqq_quantize_whole")
    return codes, sz[0], sz[1]


class AttentionChain:
    """The attention part of a decoder layer at one token as one launch (``hqq_attention_chain``): input norm + q/k/v,
    rope + cache append + attention, output projection.  ``supported`` turns False at the first call the library
    refuses (shapes outside the chained kernel); the caller then makes the three calls."""

    def __init__(self, qkv: LinearGroup, o_desc):
        self.qkv, self.o = qkv, o_desc
        self.supported = qkv.supported and len(qkv.descs) == 3
        self._scratch = None

    def __call__(self, x: torch.Tensor, delta: Optional[torch.Tensor], weight: torch.Tensor, eps: float,
                 x_sum: torch.Tensor, cos: torch.Tensor, sin: torch.Tensor, pos: torch.Tensor, cache_k: torch.Tensor,
                 cache_v: torch.Tensor) -> Optional[torch.Tensor]:
        """Returns the output projection's result (1, hidden), or None when the shapes are not taken."""
        q, k, v = self.qkv.descs
        n_kv, max_len, hd = cache_k.shape
        n_heads = q.N // hd
        assert x.dtype == torch.float16 and x.is_contiguous() and x.numel() == q.K and x.device == q.device
        assert x_sum.dtype == torch.float16 and x_sum.numel() == q.K and x_sum.data_ptr() != x.data_ptr()
        assert weight.dtype == torch.float16 and weight.numel() == q.K
        assert cache_k.is_contiguous() and cache_v.is_contiguous() and k.N == n_kv * hd == v.N and n_heads * hd == q.N
        assert pos.dtype == torch.int64 and pos.is_cuda and cos.shape[-1] == hd and cos.is_contiguous() and sin.is_contiguous()
        assert cos.shape[0] >= max_len and sin.shape[0] >= max_len, "rope tables shorter than the KV cache"
        if self._scratch is None or self._scratch.device != x.device:
            self._scratch = torch.zeros(2 * q.N + 2 * k.N, device=x.device, dtype=torch.float16)
        sc = self._scratch
        qs, ks, vs, atts = sc[:q.N], sc[q.N:q.N + k.N], sc[q.N + k.N:q.N + 2 * k.N], sc[q.N + 2 * k.N:]
        y = torch.empty((1, self.o.N), device=x.device, dtype=torch.float16)
        with _on(x.device):
            ws = workspace(x.device, int(_lib.lib.hqq_attention_chain_workspace_bytes()))
            rc = _lib.lib.hqq_attention_chain(q.ref, k.ref, v.ref, self.o.ref, x.data_ptr(),
                                              delta.data_ptr() if delta is not None else None, weight.data_ptr(), float(eps),
                                              x_sum.data_ptr(), qs.data_ptr(), ks.data_ptr(), vs.data_ptr(), atts.data_ptr(),
                                              cos.data_ptr(), sin.data_ptr(), pos.data_ptr(), cache_k.data_ptr(),
                                              cache_v.data_ptr(), max_len, n_heads, n_kv, hd, y.data_ptr(), ws.data_ptr(),
                                              ws.numel(), _lib.current_stream_ptr(x.device))
        if rc == _lib.HQQ_E_UNSUPPORTED:
            self.supported = False
            return None
        _lib.check(rc, "hqq_attention_chain")
        return y


def attention_chain_error(device, clear: bool = False) -> bool:
    """Whether a chained launch on one of this device's workspaces has ever given up a wait (it never should): reads
    a word per workspace back from the device, so call it outside the decode loop.  ``clear`` resets the words."""
    off = int(_lib.lib.hqq_attention_chain_error_offset())
    bad = False
    for (index, _stream), ws in list(_workspaces.items()):
        if index == device.index and ws.numel() >= off + 4:
            word = ws[off:off + 4].view(torch.int32)
            if bool(word.item()):
                bad = True
                if clear:
                    word.zero_()
    return bad


def router_top2(x: torch.Tensor, gate_weight: torch.Tensor, sel: torch.Tensor, weights: torch.Tensor,
                logits: Optional[torch.Tensor] = None) -> None:
    """Router of one token into device tensors ``sel`` (int32[2]) and ``weights`` (fp16[2])
    (reference src/custom_layers.py:276-282)."""
    n_experts, hidden = gate_weight.shape
    assert x.dtype == torch.float16 and gate_weight.dtype == torch.float16 and x.numel() == hidden
    assert sel.dtype == torch.int32 and sel.numel() >= 2 and weights.dtype == torch.float16 and weights.numel() >= 2
    with _on(x.device):
        _lib.check(_lib.lib.hqq_router_top2(x.data_ptr(), gate_weight.data_ptr(), n_experts, hidden, sel.data_ptr(),
                                            weights.data_ptr(), logits.data_ptr() if logits is not None else None,
                                            _lib.current_stream_ptr(x.device)), "hqq_router_top2")


def add_rmsnorm(x: torch.Tensor, delta: Optional[torch.Tensor], weight: torch.Tensor, eps: float,
                out: torch.Tensor) -> torch.Tensor:
    """``x += delta`` (when given) then ``out = weight * rmsnorm(x)`` for one token."""
    assert x.dtype == torch.float16 and x.is_contiguous() and out.dtype == torch.float16 and x.numel() == weight.numel()
    with _on(x.device):
        _lib.check(_lib.lib.hqq_add_rmsnorm(x.data_ptr(), delta.data_ptr() if delta is not None else None,
                                            weight.data_ptr(), float(eps), out.data_ptr(), x.numel(),
                                            _lib.current_stream_ptr(x.device)), "hqq_add_rmsnorm")
    return out


def add_rmsnorm_router(x: torch.Tensor, delta: Optional[torch.Tensor], weight: torch.Tensor, eps: float,
                       out: torch.Tensor, gate_weight: torch.Tensor, sel: torch.Tensor, weights: torch.Tensor,
                       logits: Optional[torch.Tensor] = None) -> torch.Tensor:
    """``add_rmsnorm`` followed by ``router_top2`` on its output, in one launch."""
    n_experts, hidden = gate_weight.shape
    assert x.dtype == torch.float16 and x.is_contiguous() and out.dtype == torch.float16 and x.numel() == weight.numel()
    assert gate_weight.dtype == torch.float16 and gate_weight.is_contiguous() and x.numel() == hidden
    assert sel.dtype == torch.int32 and sel.numel() >= 2 and weights.dtype == torch.float16 and weights.numel() >= 2
    with _on(x.device):
        _lib.check(_lib.lib.hqq_add_rmsnorm_router(x.data_ptr(), delta.data_ptr() if delta is not None else None,
                                                   weight.data_ptr(), float(eps), out.data_ptr(), hidden,
                                                   gate_weight.data_ptr(), n_experts, sel.data_ptr(), weights.data_ptr(),
                                                   logits.data_ptr() if logits is not None else None,
                                                   _lib.current_stream_ptr(x.device)), "hqq_add_rmsnorm_router")
    return out


def add_rmsnorm_rows(x: torch.Tensor, delta: Optional[torch.Tensor], weight: torch.Tensor, eps: float,
                     out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """``add_rmsnorm`` over the rows of ``x`` (tokens, hidden): ``x += delta`` in place (when given), returns
    ``weight * rmsnorm(x)`` row by row."""
    assert x.dtype == torch.float16 and x.dim() == 2 and x.is_contiguous() and x.shape[1] == weight.numel()
    assert delta is None or (delta.dtype == torch.float16 and delta.shape == x.shape and delta.is_contiguous())
    if out is None:
        out = torch.empty_like(x)
    assert out.dtype == torch.float16 and out.shape == x.shape and out.is_contiguous()
    with _on(x.device):
        _lib.check(_lib.lib.hqq_add_rmsnorm_rows(x.data_ptr(), delta.data_ptr() if delta is not None else None,
                                                 weight.data_ptr(), float(eps), out.data_ptr(), x.shape[0], x.shape[1],
                                                 _lib.current_stream_ptr(x.device)), "hqq_add_rmsnorm_rows")
    return out


def router_top2_rows(x: torch.Tensor, gate_weight: torch.Tensor):
    """Router of every row of ``x`` (tokens, hidden) (reference src/custom_layers.py:276-282): returns ``sel``
    int32 (tokens, 2), ``weights`` fp16 (tokens, 2), ``logits`` fp16 (tokens, n_experts)."""
    n_experts, hidden = gate_weight.shape
    assert x.dtype == torch.float16 and x.dim() == 2 and x.is_contiguous() and x.shape[1] == hidden
    assert gate_weight.dtype == torch.float16 and gate_weight.is_contiguous()
    rows = x.shape[0]
    sel = torch.empty((rows, 2), dtype=torch.int32, device=x.device)
    weights = torch.empty((rows, 2), dtype=torch.float16, device=x.device)
    logits = torch.empty((rows, n_experts), dtype=torch.float16, device=x.device)
    with _on(x.device):
        _lib.check(_lib.lib.hqq_router_top2_rows(x.data_ptr(), gate_weight.data_ptr(), n_experts, rows, hidden,
                                                 sel.data_ptr(), weights.data_ptr(), logits.data_ptr(),
                                                 _lib.current_stream_ptr(x.device)), "hqq_router_top2_rows")
    return sel, weights, logits


def moe_group_pairs(sel: torch.Tensor, weights: torch.Tensor, n_experts: int):
    """The (token, slot) pairs of ``router_top2_rows`` grouped by expert on the device (reference
    src/custom_layers.py:288-301): returns ``counts`` int32 (n_experts,), and per row of the grouped order the token
    it came from (int64) and its routing weight (fp16).  Nothing here waits for the device."""
    assert sel.dtype == torch.int32 and sel.dim() == 2 and sel.shape[1] == 2 and sel.is_contiguous()
    assert weights.dtype == torch.float16 and weights.shape == sel.shape and weights.is_contiguous()
    tokens = sel.shape[0]
    counts = torch.empty((n_experts,), dtype=torch.int32, device=sel.device)
    token_of_row = torch.empty((2 * tokens,), dtype=torch.int64, device=sel.device)
    scale_of_row = torch.empty((2 * tokens,), dtype=torch.float16, device=sel.device)
    with _on(sel.device):
        _lib.check(_lib.lib.hqq_moe_group_pairs(sel.data_ptr(), weights.data_ptr(), tokens, n_experts, counts.data_ptr(),
                                                token_of_row.data_ptr(), scale_of_row.data_ptr(),
                                                _lib.current_stream_ptr(sel.device)), "hqq_moe_group_pairs")
    return counts, token_of_row, scale_of_row


def rope_append_rows(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, cos: torch.Tensor, sin: torch.Tensor, start: int,
                     cache_k: torch.Tensor, cache_v: torch.Tensor) -> torch.Tensor:
    """Rotary embedding of ``q`` (tokens, heads, hd; in place) and ``k`` (tokens, kv_heads, hd) at positions ``start``
    onwards; the rotated keys and ``v`` are written to the caches (kv_heads, max_len, hd).  Returns ``q``."""
    T, n_heads, hd = q.shape
    n_kv, max_len = cache_k.shape[0], cache_k.shape[1]
    for t in (q, k, v, cos, sin, cache_k, cache_v):
        assert t.dtype == torch.float16 and t.is_contiguous()
    assert k.shape == (T, n_kv, hd) and v.shape == (T, n_kv, hd) and cache_v.shape == cache_k.shape
    assert cos.shape[1] == hd and cos.shape[0] >= start + T and sin.shape == cos.shape and start + T <= max_len
    with _on(q.device):
        _lib.check(_lib.lib.hqq_rope_append_rows(q.data_ptr(), k.data_ptr(), v.data_ptr(), cos.data_ptr(), sin.data_ptr(),
                                                 int(start), T, cache_k.data_ptr(), cache_v.data_ptr(), max_len, n_heads,
                                                 n_kv, hd, _lib.current_stream_ptr(q.device)), "hqq_rope_append_rows")
    return q


_attention_workspaces = {}  # (device, stream) -> zero-filled bytes for the split attention launch


def attention_decode(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, cos: torch.Tensor, sin: torch.Tensor,
                     pos: torch.Tensor, cache_k: torch.Tensor, cache_v: torch.Tensor, out: torch.Tensor,
                     split: bool = True) -> torch.Tensor:
    """Rope, cache append and attention of one new token; ``pos`` is an int64 device tensor with the position.
    Caches longer than 1024 positions are split over several blocks per head unless ``split`` is False."""
    n_kv, max_len, hd = cache_k.shape
    n_heads = q.numel() // hd
    assert q.is_contiguous() and k.is_contiguous() and v.is_contiguous() and cache_k.is_contiguous() and cache_v.is_contiguous()
    assert pos.dtype == torch.int64 and pos.is_cuda and cos.shape[-1] == hd and cos.is_contiguous() and sin.is_contiguous()
    assert out.numel() == n_heads * hd and k.numel() == n_kv * hd == v.numel()
    # the kernel bounds the device-side position by the cache length only: the rope tables must cover the cache
    assert cos.shape[0] >= max_len and sin.shape[0] >= max_len, "rope tables shorter than the KV cache"
    with _on(q.device):
        need = int(_lib.lib.hqq_attention_decode_workspace_bytes(max_len, n_heads, hd))
        if need and split:
            # long caches: a head's positions over several blocks, their shares added up through a workspace of the
            # launch's own (its counters must stay zero between launches, so nothing else may write there)
            key = (q.device.index, torch.cuda.current_stream(q.device).cuda_stream)
            ws = _attention_workspaces.get(key)
            if ws is None or ws.numel() < need:
                ws = _attention_workspaces[key] = torch.zeros(need, dtype=torch.uint8, device=q.device)
            _lib.check(_lib.lib.hqq_attention_decode_ws(q.data_ptr(), k.data_ptr(), v.data_ptr(), cos.data_ptr(), sin.data_ptr(),
                                                        pos.data_ptr(), cache_k.data_ptr(), cache_v.data_ptr(), max_len, n_heads,
                                                        n_kv, hd, out.data_ptr(), ws.data_ptr(), ws.numel(),
                                                        _lib.current_stream_ptr(q.device)), "hqq_attention_decode_ws")
            return out
        _lib.check(_lib.lib.hqq_attention_decode(q.data_ptr(), k.data_ptr(), v.data_ptr(), cos.data_ptr(), sin.data_ptr(),
                                                 pos.data_ptr(), cache_k.data_ptr(), cache_v.data_ptr(), max_len, n_heads,
                                                 n_kv, hd, out.data_ptr(), _lib.current_stream_ptr(q.device)),
                   "hqq_attention_decode")
    return out
