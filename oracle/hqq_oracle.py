"""CPU restatement (numpy) of the reference's HQQ quantized-linear path.

TEST INFRASTRUCTURE ONLY.  Nothing under ``oracle/`` is part of the product:
only ``tests/``, ``__graft_entry__.smoke()`` and the ``cpu_baseline`` leg of
``bench.py`` may import it, and only as the checker.  The product path calls
the HIP library through its C ABI and fails loudly when that is missing.

Every function cites the reference lines it restates (paths are relative to
the reference tree, ``src/...``).  The reference's arithmetic lives partly in
the third-party ``hqq`` package (git commit 37502bea), which is not available
offline; for those functions the published algorithm is restated and the
reference's own call sites anchor the behaviour.

Pinning status (what independent evidence fixes each function; the tests
named here live in ``tests/test_oracle_*.py``):

* pack/unpack 4, 2, 3 bit ......... pinned: hand-computed known answers,
  exhaustive byte values, every code in every 3-bit lane, tail heights,
  cross-check against the shift formulas of the reference's matmul kernels
  (``src/triton_kernels.py:91,279,469``), round trips, and the C restatement.
* group index / dequantize ........ pinned: brute-force scalar loop with the
  index identity ``col = (n % G) * K + k`` on tiny shapes, IEEE fp16 rounding
  cross-checked against an integer-only software rounding in the C oracle.
* meta_dequant .................... pinned: same scalar brute force.
* matmul_transpose / forward ...... pinned: fp64 brute force on tiny shapes,
  linearity, and the dequantize-then-matmul path.
* expert_ffn, router .............. pinned: scalar restatement with math.exp.
* slab_layout ..................... pinned: closed-form byte totals
  (66,404,364 B for a 2-bit g16 Mixtral expert).
* LruModel ........................ pinned: hand-traced access sequences.
* hqq_quantize (quantise side) .... PARITY UNPINNED: restated from memory of
  hqq @37502bea; the reference holds no test or fixture at that boundary.
  It only manufactures inputs; kernels and oracle consume the same tensors.
"""
from __future__ import annotations

import math
from collections import OrderedDict

import numpy as np

F16 = np.float16


# --------------------------------------------------------------------------
# Bit packers  (src/packing.py)
# --------------------------------------------------------------------------
def pack_4bit_u8(q: np.ndarray) -> np.ndarray:
    """src/packing.py:10-17 -- byte[p] = (q[2p] << 4) | q[2p+1] along axis 0.

    The shift happens in uint8, so bits above the low nibble of q[2p] fall
    off and q[2p+1] is OR-ed in unmasked (the reference does not mask)."""
    q = np.asarray(q)
    if q.shape[0] % 2 != 0:
        raise AssertionError("height must be even")  # src/packing.py:12
    q = q.astype(np.uint8)
    return ((q[0::2] << np.uint8(4)) | q[1::2]).astype(np.uint8)


def unpack_4bit_u8(p: np.ndarray) -> np.ndarray:
    """src/packing.py:19-27 -- rows 2p = high nibble, rows 2p+1 = low nibble."""
    p = np.asarray(p).astype(np.uint8)
    out = np.empty((2 * p.shape[0],) + p.shape[1:], dtype=np.uint8)
    out[0::2] = p >> np.uint8(4)
    out[1::2] = p & np.uint8(0x0F)
    return out


def pack_2bit_u8(q: np.ndarray) -> np.ndarray:
    """src/packing.py:36-41 -- byte[p] = q[4p]<<6 | q[4p+1]<<4 | q[4p+2]<<2 | q[4p+3]."""
    q = np.asarray(q).astype(np.uint8)
    if q.shape[0] % 4 != 0:
        # the reference would fail on the mismatched strided slices
        raise AssertionError("height must be a multiple of 4")
    return ((q[0::4] << np.uint8(6)) | (q[1::4] << np.uint8(4))
            | (q[2::4] << np.uint8(2)) | q[3::4]).astype(np.uint8)


def unpack_2bit_u8(p: np.ndarray) -> np.ndarray:
    """src/packing.py:43-53."""
    p = np.asarray(p).astype(np.uint8)
    out = np.empty((4 * p.shape[0],) + p.shape[1:], dtype=np.uint8)
    out[0::4] = (p >> np.uint8(6)) & np.uint8(3)
    out[1::4] = (p >> np.uint8(4)) & np.uint8(3)
    out[2::4] = (p >> np.uint8(2)) & np.uint8(3)
    out[3::4] = p & np.uint8(3)
    return out


def pack_3bit_i32(q: np.ndarray) -> np.ndarray:
    """src/packing.py:62-81 -- ten codes per int32, code i at bit 3*(9-i).

    The last word holds ``H mod 10`` (or 10) codes; its missing lanes stay 0.
    Codes are widened to int32 and shifted unmasked, as the reference does."""
    q = np.asarray(q)
    h = q.shape[0]
    words = (h + 9) // 10
    out = np.zeros((words,) + q.shape[1:], dtype=np.int32)
    for i in range(10):
        rows = q[i::10].astype(np.int32)
        out[: rows.shape[0]] |= rows << np.int32(3 * (9 - i))
    return out


def unpack_3bit_i32(p: np.ndarray) -> np.ndarray:
    """src/packing.py:83-97 -- always yields 10*words rows (spare rows are 0)."""
    p = np.asarray(p)
    if p.dtype != np.int32:
        raise AssertionError("3-bit codes are packed in int32")  # :88
    out = np.empty((10 * p.shape[0],) + p.shape[1:], dtype=np.uint8)
    for i in range(10):
        out[i::10] = ((p >> np.int32(3 * (9 - i))) & np.int32(7)).astype(np.uint8)
    return out


PACK = {4: pack_4bit_u8, 2: pack_2bit_u8, 3: pack_3bit_i32}
UNPACK = {4: unpack_4bit_u8, 2: unpack_2bit_u8, 3: unpack_3bit_i32}
CODES_PER_WORD = {4: 2, 2: 4, 3: 10}


def kernel_code(packed: np.ndarray, nbits: int, n: int, k: int) -> int:
    """The code the reference matmul kernels read for weight (n, k).

    src/triton_kernels.py:84,91 (4 bit), :272,279 (2 bit), :462,469 (3 bit).
    This is an independent statement of the layout and pins the packers."""
    if nbits == 4:
        return (int(packed[n // 2, k]) >> (((n + 1) % 2) * 4)) & 0xF
    if nbits == 2:
        return (int(packed[n // 4, k]) >> ((3 - n % 4) * 2)) & 0x3
    if nbits == 3:
        return (int(packed[n // 10, k]) >> ((9 - n % 10) * 3)) & 0x7
    raise ValueError(nbits)


# --------------------------------------------------------------------------
# Quantise-time layout -> kernel layout  (src/custom_layers.py:41-47)
# --------------------------------------------------------------------------
def repack(unpacked_quant_layout: np.ndarray, shape, nbits: int) -> np.ndarray:
    """src/custom_layers.py:41-47.  ``unpacked_quant_layout`` holds the codes
    as the quantiser produced them, (gs_padded, N*K/gs); flat order equals the
    row-major order of W, so reshape to (-1, K), keep N rows, pack."""
    n, k = shape
    q = np.asarray(unpacked_quant_layout).reshape(-1, k)[:n]
    return PACK[nbits](q)


# --------------------------------------------------------------------------
# Meta de-quantisation and weight de-quantisation
# --------------------------------------------------------------------------
def meta_dequant(q_u8: np.ndarray, meta_scale, meta_zero, out_shape) -> np.ndarray:
    """src/custom_layers.py:63-66 call hqq ``Quantizer.dequantize`` whose formula
    the reference restates at src/custom_layers.py:111:
    ``((W_r - zero) * scale).reshape(shape)`` with every operand fp16, i.e. two
    fp16 roundings.  ``q_u8`` is (mgs, S/mgs) for the scale table and (1, S)
    for the zero table; ``meta_scale``/``meta_zero`` broadcast against it."""
    w = np.asarray(q_u8).astype(F16)
    t = (w - np.asarray(meta_zero, dtype=F16)).astype(F16)
    return (t * np.asarray(meta_scale, dtype=F16)).astype(F16).reshape(out_shape)


def expand_tables(layer: dict):
    """fp16 (G, K) scale and zero tables of a layer, meta-dequantised when the
    layer stores them as 8-bit (src/custom_layers.py:62-66, 80-84 ``view(-1,K)``)."""
    n, k = layer["shape"]
    gs = layer["group_size"]
    s_cnt = n * k // gs
    if layer.get("quant_scale"):
        scale = meta_dequant(layer["scale_q"], layer["meta_scale"]["scale"],
                             layer["meta_scale"]["zero"], (1, s_cnt))
    else:
        scale = np.asarray(layer["scale"], dtype=F16)
    if layer.get("quant_zero"):
        zero = meta_dequant(layer["zero_q"], layer["meta_zero"]["scale"],
                            layer["meta_zero"]["zero"], (1, s_cnt))
    else:
        zero = np.asarray(layer["zero"], dtype=F16)
    return scale.reshape(-1, k), zero.reshape(-1, k)


def dequantize(layer: dict) -> np.ndarray:
    """src/custom_layers.py:95-116 -- unpack, half, first N rows, reshape
    (gs, -1), ``(W - zero) * scale`` in fp16, reshape to (N, K)."""
    n, k = layer["shape"]
    gs = layer["group_size"]
    scale, zero = expand_tables(layer)
    w = UNPACK[layer["nbits"]](layer["W_q"]).astype(F16)[:n]
    w = w.reshape(gs, -1)
    t = (w - zero.reshape(1, -1)).astype(F16)
    return (t * scale.reshape(1, -1)).astype(F16).reshape(n, k)


def dequantize_scalar(layer: dict) -> np.ndarray:
    """Element-by-element statement of what the reference matmul kernels compute
    for B (src/triton_kernels.py:86-88,109-118): group row ``n % G``, two fp16
    roundings.  Slow; for tiny shapes, to pin ``dequantize``."""
    n_rows, k_cols = layer["shape"]
    gs = layer["group_size"]
    g = n_rows // gs
    scale, zero = expand_tables(layer)
    out = np.empty((n_rows, k_cols), dtype=F16)
    for n in range(n_rows):
        for k in range(k_cols):
            q = F16(kernel_code(layer["W_q"], layer["nbits"], n, k))
            t = F16(np.float32(q) - np.float32(zero[n % g, k]))
            out[n, k] = F16(np.float32(t) * np.float32(scale[n % g, k]))
    return out


# --------------------------------------------------------------------------
# Matmul  (src/triton_kernels.py:103-131 and wrappers :133-191 etc.)
# --------------------------------------------------------------------------
def matmul_transpose(x: np.ndarray, layer: dict, bias=None) -> np.ndarray:
    """C = x @ dequant(B).T (+ bias): fp16 operands, wide accumulation, fp16
    result (src/triton_kernels.py:103-131; bias added in fp16 at :188-189).
    Accumulates in fp64, so it is the exact value the fp32-accumulating
    kernels approximate."""
    w = dequantize(layer).astype(np.float64)
    xf = np.asarray(x, dtype=F16).astype(np.float64)
    y = (xf.reshape(-1, xf.shape[-1]) @ w.T).astype(F16)
    y = y.reshape(x.shape[:-1] + (w.shape[0],))
    if bias is not None:
        y = (y + np.asarray(bias, dtype=F16)).astype(F16)
    return y


def matmul_tolerance(x: np.ndarray, layer: dict) -> np.ndarray:
    """Absolute tolerance 1e-3 * ||x_m|| * ||w_n|| per output element."""
    w = dequantize(layer).astype(np.float64)
    xf = np.asarray(x, dtype=np.float64).reshape(-1, x.shape[-1])
    return 1e-3 * np.linalg.norm(xf, axis=1)[:, None] * np.linalg.norm(w, axis=1)[None, :]


def silu_f16(x: np.ndarray) -> np.ndarray:
    """torch's half SiLU computes in fp32 and rounds once."""
    xf = np.asarray(x, dtype=F16).astype(np.float32)
    return (xf / (np.float32(1.0) + np.exp(-xf))).astype(F16)


def expert_ffn(x: np.ndarray, w1: dict, w2: dict, w3: dict) -> np.ndarray:
    """src/custom_layers.py:253-256 -- w2(silu(w1 x) * w3 x), fp16 intermediates."""
    a = matmul_transpose(x, w1)
    b = matmul_transpose(x, w3)
    h = (silu_f16(a).astype(np.float32) * b.astype(np.float32)).astype(F16)
    return matmul_transpose(h, w2)


def router(hidden: np.ndarray, gate_w: np.ndarray, top_k: int = 2):
    """src/custom_layers.py:276-282 -- fp16 logits, fp32 softmax, top-k,
    renormalise, cast back to fp16.  Returns (weights fp16, experts, logits)."""
    h = np.asarray(hidden, dtype=F16).astype(np.float64)
    logits = (h @ np.asarray(gate_w, dtype=F16).astype(np.float64).T).astype(F16)
    z = logits.astype(np.float32)
    z = z - z.max(axis=1, keepdims=True)
    p = np.exp(z)
    p = (p / p.sum(axis=1, keepdims=True)).astype(np.float32)
    idx = np.argsort(-p, axis=1, kind="stable")[:, :top_k]
    w = np.take_along_axis(p, idx, axis=1)
    w = (w / w.sum(axis=1, keepdims=True)).astype(np.float32)
    return w.astype(F16), idx, logits


# --------------------------------------------------------------------------
# Expert slab layout  (src/expert_wrapper.py:41-57, src/utils.py:34-45)
# --------------------------------------------------------------------------
def layer_tensor_order(layer: dict):
    """Tensors of one linear in the reference's flatten order: dict keys sorted
    at every level (src/utils.py:42): W_q, bias, meta{meta_scale{scale,zero},
    meta_zero{scale,zero}, scale_q, zero_q} (or scale / zero when not
    meta-quantised).  Non-tensor leaves and ``None`` are skipped
    (src/expert_wrapper.py:52-54)."""
    out = [("W_q", layer["W_q"])]
    if layer.get("bias") is not None:
        out.append(("bias", layer["bias"]))
    meta = {}
    if layer.get("quant_scale"):
        meta["meta_scale.scale"] = layer["meta_scale"]["scale"]
        meta["meta_scale.zero"] = layer["meta_scale"]["zero"]
        meta["scale_q"] = layer["scale_q"]
    else:
        meta["scale"] = layer["scale"]
    if layer.get("quant_zero"):
        meta["meta_zero.scale"] = layer["meta_zero"]["scale"]
        meta["meta_zero.zero"] = layer["meta_zero"]["zero"]
        meta["zero_q"] = layer["zero_q"]
    else:
        meta["zero"] = layer["zero"]

    def key(name):  # sorted at each nesting level
        return name.split(".")

    for name in sorted(meta, key=key):
        out.append(("meta." + name, meta[name]))
    return out


def slab_layout(w1: dict, w2: dict, w3: dict):
    """Byte offsets of every tensor of an expert in the reference's single
    storage: cumulative ``nbytes`` in flatten order, no padding
    (src/expert_wrapper.py:47-57).  Returns ([(name, offset, nbytes)], total)."""
    entries, off = [], 0
    for lname, layer in (("w1", w1), ("w2", w2), ("w3", w3)):
        for tname, t in layer_tensor_order(layer):
            nb = int(np.asarray(t).nbytes)
            entries.append((f"{lname}.{tname}", off, nb))
            off += nb
    return entries, off


# --------------------------------------------------------------------------
# LRU model  (src/expert_cache.py:20-52, 120-201)
# --------------------------------------------------------------------------
class LruModel:
    """Plain model of one eviction group: which experts are device-resident,
    in least-recently-used order, plus hit / miss counters.

    ``load(uids)`` restates ``ExpertCache.load_experts(..., unordered=True)``:
    resident experts first (src/expert_cache.py:136-137), every requested
    expert is marked used before any swap (:141-143), each miss evicts the
    least recently used resident (:33-36, :160-162) and enters as most recent
    (:38-42).  The sliding window of in-flight copies (:155-175) changes when
    copies start, not which expert is evicted, as long as enough device
    buffers exist; the yield order is resident-first then misses in request
    order."""

    def __init__(self, resident, offloaded):
        self.main = OrderedDict((u, None) for u in resident)
        self.off = OrderedDict((u, None) for u in offloaded)
        self.hits = 0
        self.misses = 0

    def load(self, uids):
        uids = list(uids)
        assert len(set(uids)) == len(uids)
        order = sorted(uids, key=lambda u: u in self.off)  # stable
        for u in order:
            if u in self.main:
                self.main.move_to_end(u)
                self.hits += 1
            elif u in self.off:
                self.off.move_to_end(u)
                self.misses += 1
            else:
                raise ValueError(f"expert {u} not in group")
        evicted = []
        for u in order:
            if u in self.off:
                victim = next(iter(self.main))
                del self.main[victim]
                del self.off[u]
                self.main[u] = None
                self.off[victim] = None
                evicted.append((u, victim))
        return order, evicted


# --------------------------------------------------------------------------
# Quantise side (hqq @37502bea, restated from memory) -- PARITY UNPINNED
# --------------------------------------------------------------------------
def _shrink_lp(x, beta, p):
    return np.sign(x) * np.maximum(np.abs(x) - (1.0 / beta) * np.power(np.abs(x) + 1e-8, p - 1), 0)


def hqq_quantize_tensor(w, nbits, group_size, channel_wise=True, optimize=False,
                        round_zero=False, iters=20):
    """hqq ``Quantizer.quantize`` with axis 0 (call sites:
    src/custom_layers.py:36, 120).  Returns (codes uint8 unpacked in the
    quantise layout, scale fp32, zero fp32).  PARITY UNPINNED."""
    w = np.asarray(w, dtype=np.float32)
    if group_size is not None and channel_wise:
        w = w.reshape(group_size, -1)
    if channel_wise:
        mn = w.min(axis=0, keepdims=True)
        mx = w.max(axis=0, keepdims=True)
    else:
        mn, mx = w.min(), w.max()
        optimize = False
    max_v = float(2 ** nbits - 1)
    with np.errstate(divide="ignore"):
        scale = np.minimum(max_v / (mx - mn), np.float32(2e4)).astype(np.float32)
    zero = (-mn * scale).astype(np.float32)
    if round_zero:
        zero = np.round(zero)
    if optimize:
        beta, kappa, best = 10.0, 1.01, 1e4
        for _ in range(iters):
            wq = np.clip(np.round(w * scale + zero), 0, max_v)
            wr = (wq - zero) / scale
            we = _shrink_lp(w - wr, beta, 0.7)
            zero = np.mean(wq - (w - we) * scale, axis=0, keepdims=True).astype(np.float32)
            beta *= kappa
            err = float(np.abs(w - wr).mean())
            if err < best:
                best = err
            else:
                break
    q = np.clip(np.round(w * scale + zero), 0, max_v).astype(np.uint8)
    return q, (np.float32(1.0) / scale).astype(np.float32), np.asarray(zero, dtype=np.float32)


def hqq_quantize_layer(w, nbits, group_size, quant_scale=True, quant_zero=True,
                       meta_group_size=128, optimize=False):
    """hqq ``HQQLinear.quantize`` followed by the reference's ``repack``
    (src/custom_layers.py:35-47): weight codes in the kernel layout plus 8-bit
    scale (channel-wise, group ``meta_group_size``) and 8-bit zero (one group
    for the whole tensor) with fp16 meta tables.  PARITY UNPINNED."""
    w = np.asarray(w, dtype=F16)
    n, k = w.shape
    q, scale, zero = hqq_quantize_tensor(w, nbits, group_size, optimize=optimize,
                                         round_zero=(nbits == 4))
    s_cnt = n * k // group_size
    layer = {"nbits": nbits, "group_size": group_size, "shape": (n, k), "axis": 0,
             "quant_scale": bool(quant_scale), "quant_zero": bool(quant_zero),
             "W_q": repack(q, (n, k), nbits)}
    if quant_scale:
        sq, ms, mz = hqq_quantize_tensor(scale.reshape(1, s_cnt), 8, meta_group_size)
        layer["scale_q"] = sq.reshape(meta_group_size, -1)
        layer["meta_scale"] = {"scale": ms.astype(F16), "zero": mz.astype(F16)}
    else:
        layer["scale"] = scale.reshape(1, s_cnt).astype(F16)
    if quant_zero:
        zq, ms, mz = hqq_quantize_tensor(zero.reshape(1, s_cnt), 8, None, channel_wise=False)
        layer["zero_q"] = zq.reshape(1, s_cnt)
        layer["meta_zero"] = {"scale": np.asarray(ms, dtype=F16).reshape(()),
                              "zero": np.asarray(mz, dtype=F16).reshape(())}
    else:
        layer["zero"] = zero.reshape(1, s_cnt).astype(F16)
    return layer


def random_layer(rng, n, k, nbits, group_size, quant_scale=True, quant_zero=True,
                 meta_group_size=128, std=0.02):
    """Seeded synthetic layer: W ~ N(0, std) fp16, quantised as above."""
    w = (rng.standard_normal((n, k)) * std).astype(F16)
    return hqq_quantize_layer(w, nbits, group_size, quant_scale, quant_zero, meta_group_size), w
