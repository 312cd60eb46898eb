#!/usr/bin/env python3
"""Headline benchmark: HQQ dequant-GEMV throughput on one MI355X.

A "step" is one pass of the hot path over one batch of synthetic input: the
2-bit expert FFN of Mixtral-8x7B at batch 1 (w1, w3: 14336x4096, w2: 4096x14336,
group 16, 8-bit meta-quantised scale/zero), y = w2(silu(w1 x) * w3 x).  Steps
rotate over several distinct experts (more than the 256 MB Infinity Cache holds)
so that every weight byte really comes from HBM.  Inputs are resident in HBM
before the timed region.

Prints ONE JSON line.  ``value`` is algorithmic bytes per step / time per step.
``roofline`` is the dominant kernel alone (the fused w1/w3 pass), timed with HIP
events on the stream it is launched on.  ``cpu_baseline`` times the reference's
PyTorch dequantise-then-matmul path (restated in oracle/torch_path.py) on the
host cores for a bounded sample of the same steps.  ``decode`` is the second half
of the metric: greedy batch-1 decoding of the 32-layer random-init Mixtral-8x7B
(attention 4-bit g64, experts 2-bit g16) from a 64-token random prompt, with every
expert resident (graph-replayed and eager) and with a per-layer expert cache of 4
and 2 slots fed by pinned host-to-device copies on a side stream."""
from __future__ import annotations

import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
for _p in (ROOT, os.path.join(ROOT, "mixtral-offloading_amd")):
    if _p not in sys.path:
        sys.path.insert(0, _p)

HIDDEN, FFN = 4096, 14336
NBITS, GROUP, META_GROUP = 2, 16, 128
HBM_PEAK_GBS = 8000.0


def layer_bytes(n, k):
    s_cnt = n * k // GROUP
    return n * k * NBITS // 8 + 2 * s_cnt + 2 * 2 * (s_cnt // META_GROUP) + 4


def ffn_step_bytes(m):
    """Algorithmic bytes of one expert FFN: weight-side bytes of the three layers plus fp16 activations in and out."""
    weights = 2 * layer_bytes(FFN, HIDDEN) + layer_bytes(HIDDEN, FFN)
    acts = 2 * m * HIDDEN + 2 * m * FFN + 2 * m * FFN + 2 * m * HIDDEN  # x, h written, h read, y
    return weights + acts


def gate_up_bytes(m):
    return 2 * layer_bytes(FFN, HIDDEN) + 2 * m * HIDDEN + 2 * m * FFN


def make_expert(seed, device):
    """Random-init expert, quantised on the GPU by the package's own HQQ quantiser (W ~ N(0, 0.02))."""
    import torch
    from torch import nn

    from mixtral_offloading_amd.custom_layers import HQQLinearTritonSavable
    from mixtral_offloading_amd.hqq_core import BaseQuantizeConfig

    cfg = BaseQuantizeConfig(nbits=NBITS, group_size=GROUP, quant_zero=True, quant_scale=True)
    cfg["weight_quant_params"]["optimize"] = False  # min/max quantisation: the speed of the path does not depend on it
    g = torch.Generator(device=device).manual_seed(seed)
    layers = []
    for n, k in ((FFN, HIDDEN), (HIDDEN, FFN), (FFN, HIDDEN)):
        lin = nn.Linear(k, n, bias=False, device=device, dtype=torch.float16)
        lin.weight.data = (torch.randn((n, k), device=device, generator=g) * 0.02).half()
        layers.append(HQQLinearTritonSavable(lin, cfg))
        del lin
    return layers


def make_attention(device):
    """The four 4-bit g64 projections of one decoder layer (q, k, v, o), random-init, for the CPU decode figure."""
    import torch
    from torch import nn

    from mixtral_offloading_amd.custom_layers import HQQLinearTritonSavable
    from mixtral_offloading_amd.hqq_core import BaseQuantizeConfig

    cfg = BaseQuantizeConfig(nbits=4, group_size=64, quant_zero=True, quant_scale=True)
    cfg["weight_quant_params"]["optimize"] = False
    g = torch.Generator(device=device).manual_seed(77)
    layers = []
    for n in (HIDDEN, 1024, 1024, HIDDEN):
        lin = nn.Linear(HIDDEN, n, bias=False, device=device, dtype=torch.float16)
        lin.weight.data = (torch.randn((n, HIDDEN), device=device, generator=g) * 0.02).half()
        layers.append(HQQLinearTritonSavable(lin, cfg))
    return layers


def _cpu_layer(lin):
    """A quantised layer of the GPU leg as the CPU path's layer dict (the same tensors, copied to the host)."""
    import torch

    meta = lin.meta
    out = {"nbits": int(meta["nbits"]), "group_size": int(meta["group_size"]), "shape": tuple(int(v) for v in meta["shape"]),
           "quant_scale": bool(meta.get("quant_scale")), "quant_zero": bool(meta.get("quant_zero")),
           "W_q": torch.Tensor.as_subclass(lin.W_q, torch.Tensor).cpu()}
    for q, m in (("scale_q", "meta_scale"), ("zero_q", "meta_zero")):
        if q in meta:
            out[q] = meta[q].cpu()
            out[m] = {"scale": meta[m]["scale"].cpu().half(), "zero": meta[m]["zero"].cpu().half()}
    for key in ("scale", "zero"):
        if key in meta and key + "_q" not in meta:
            out[key] = meta[key].cpu()
    return out


def cpu_baseline(expert, x, attention=None, budget_s=12.0):
    """The reference's PyTorch path (meta expansion + dequantize + matmul per call, src/custom_layers.py:95-116) on the
    host cores, on the tensors the GPU leg runs on: expert 0 and the same x.  With `attention` (the four 4-bit
    projections of one decoder layer) it also times one decoder layer's quantised linears, from which a CPU decode
    rate follows: a token is 32 layers of 4 attention projections and 2 expert FFNs (the fp16 head, the norms, the
    router and the attention itself are left out, which flatters the CPU)."""
    import torch

    from oracle import torch_path as tp

    w1, w2, w3 = (_cpu_layer(l) for l in expert)
    xc = x.cpu()
    with torch.inference_mode():
        tp.expert_ffn(xc, w1, w2, w3)  # warm up
        t0 = time.perf_counter()
        n = 0
        while n < 3 or (time.perf_counter() - t0 < budget_s and n < 200):
            tp.expert_ffn(xc, w1, w2, w3)
            n += 1
        dt = (time.perf_counter() - t0) / n
        out = {"value": round(ffn_step_bytes(xc.shape[0]) / dt / 1e9, 3), "unit": "GB/s", "cores": torch.get_num_threads(),
               "os_cpu_count": os.cpu_count(), "kind": "port", "ms_per_step": round(dt * 1e3, 2),
               "sample": f"{n} steps of the same batch-{xc.shape[0]} 2-bit expert FFN on the GPU leg's own tensors (expert 0 "
                         f"and x copied to the host), torch CPU half ops, meta expansion + dequantize + matmul per call "
                         f"as the reference does"}
        if attention is not None:
            att = [_cpu_layer(l) for l in attention]
            xa = torch.randn((1, HIDDEN), generator=torch.Generator().manual_seed(5)).half()
            for l in att:
                tp.forward(xa, l)
            t0 = time.perf_counter()
            reps = 3
            for _ in range(reps):
                for l in att:
                    tp.forward(xa, l)
            dt_att = (time.perf_counter() - t0) / reps
            layer_ms = (dt_att + 2 * dt) * 1e3
            out["decode_layer_ms"] = round(layer_ms, 1)
            out["decode_tok_s"] = round(1e3 / (32 * layer_ms), 4)
            out["decode_sample"] = (f"one decoder layer's quantised linears at batch 1 (q, k, v, o 4-bit g64: {dt_att * 1e3:.1f} ms, "
                                    f"measured {reps} times; 2 expert FFNs at the rate above) x 32 layers")
    return out


def random_desc(nbits, n, k, gs, seed, dev):
    """Random codes and 8-bit tables of one layer in the kernel layout, built on the GPU (their values do not
    change the speed of any kernel)."""
    import torch

    from mixtral_offloading_amd import hip_kernels, packing

    g = torch.Generator(device=dev).manual_seed(seed)
    s_cnt = n * k // gs
    q = torch.randint(0, 2 ** nbits, (n, k), dtype=torch.uint8, device=dev, generator=g)
    pack = {4: packing.pack_4bit_u8_common, 2: packing.pack_2bit_u8_common, 3: packing.pack_3bit_i32_common}[nbits]
    step = 0.07 / (2 ** nbits - 1)
    meta = {"nbits": nbits, "group_size": gs, "shape": (n, k), "quant_scale": True, "quant_zero": True,
            "scale_q": torch.randint(0, 256, (128, s_cnt // 128), dtype=torch.uint8, device=dev, generator=g),
            "meta_scale": {"scale": torch.full((1, s_cnt // 128), step / 255, device=dev).half(),
                           "zero": torch.full((1, s_cnt // 128), -128.0, device=dev).half()},
            "zero_q": torch.randint(0, 256, (1, s_cnt), dtype=torch.uint8, device=dev, generator=g),
            "meta_zero": {"scale": torch.tensor([(2 ** nbits - 1) / 255.0], device=dev).half(),
                          "zero": torch.tensor([0.0], device=dev).half()}}
    return hip_kernels.LinearDesc(pack(q), meta), q


PROFILE = os.path.join(ROOT, "profiles", "gemv_strip_kernel_ffn_2bit_g16_m1.txt")


KERNEL_SOURCES = ("gemv_strip.hip", "gemv_parts.hpp")


def kernel_source_hash():
    """sha256 over the sources of the dominant kernel: the counter profile records the hash it was taken with."""
    import hashlib

    h = hashlib.sha256()
    for name in KERNEL_SOURCES:
        with open(os.path.join(ROOT, "mixtral-offloading_amd", "csrc", name), "rb") as f:
            h.update(f.read())
    return h.hexdigest()[:16]


def profiled_traffic():
    """HBM bytes per launch of the dominant kernel as the tracked counter profile records them (a line
    `traffic_bytes_per_launch: <int>`, from rocprofv3 FETCH_SIZE / WRITE_SIZE runs of this command scaled by a copy of
    known size).  The figure is a recorded one, not measured by this run: it is reported only when the profile's
    `kernel_source_sha256:` line names the kernel sources as they are now, else None with the reason."""
    traffic, taken_with = None, None
    try:
        with open(PROFILE) as f:
            for line in f:
                if line.startswith("traffic_bytes_per_launch:"):
                    traffic = int(line.split(":")[1].split()[0].replace(",", ""))
                if line.startswith("kernel_source_sha256:"):
                    taken_with = line.split(":")[1].strip()
    except OSError:
        return None, "no profile"
    if traffic is None:
        return None, "the profile has no traffic line"
    try:
        now = kernel_source_hash()
    except OSError:
        return None, "kernel sources not found"
    if taken_with != now:
        return None, f"the kernel sources changed since the profile was taken ({taken_with} -> {now})"
    return traffic, f"recorded in the profile for kernel sources {now}"


def load_probe():
    """The streaming-read probe (csrc/probe/stream_read.hip), a library of its own beside the product's."""
    import ctypes

    path = os.path.join(ROOT, "mixtral-offloading_amd", "lib", "libhqq_probe.so")
    lib = ctypes.CDLL(path)
    lib.hqq_probe_stream_read.restype = ctypes.c_int
    lib.hqq_probe_stream_read.argtypes = [ctypes.c_void_p, ctypes.c_size_t, ctypes.c_void_p, ctypes.c_void_p]
    return lib


def survey_section(dev):
    """Every kernel of the path at the Mixtral-8x7B shapes: microseconds per launch by HIP events (cache-cold: each
    timing rotates over more than 256 MB of distinct inputs) and the rate that follows from its algorithmic bytes."""
    import torch

    from mixtral_offloading_amd import _lib, hip_kernels, packing

    lib = _lib.lib
    probe = load_probe()
    stream = torch.cuda.Stream(device=dev)
    rows = []

    def timed(fn, iters):
        with torch.cuda.stream(stream):
            for i in range(max(4, iters // 4)):
                fn(i)
            stream.synchronize()
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record(stream)
            for i in range(iters):
                fn(i)
            e1.record(stream)
            stream.synchronize()
        return e0.elapsed_time(e1) * 1e3 / iters

    # the ceiling of a launch of a given size: a plain 128-bit streaming read of that many bytes, timed the same way
    # (rotating over more than 256 MB), cached per size
    pool = torch.empty(768 << 20, dtype=torch.uint8, device=dev).fill_(3)
    sink = torch.zeros(4, dtype=torch.int32, device=dev)
    ceilings = {}

    def stream_us(nbytes):
        key = (int(nbytes) + (1 << 20) - 1) >> 20  # per MiB
        if key not in ceilings:
            span = (int(nbytes) + 4095) // 4096 * 4096
            slots = max(1, pool.numel() // span)

            def f(i):
                rc = probe.hqq_probe_stream_read(pool.data_ptr() + (i % slots) * span, int(nbytes), sink.data_ptr(), stream.cuda_stream)
                if rc != 0:
                    raise RuntimeError(f"hqq_probe_stream_read: {rc}")

            ceilings[key] = timed(f, 48)
        return ceilings[key]

    def add(name, us, nbytes, flops=None, ceiling=False):
        r = {"kernel": name, "us": round(us, 2), "GB_s": round(nbytes / us / 1e3, 0), "frac_hbm": round(nbytes / us / 1e3 / HBM_PEAK_GBS, 3)}
        if ceiling:
            c = stream_us(nbytes)
            r["stream_read_same_bytes_us"] = round(c, 2)
            r["frac_of_stream_read"] = round(c / us, 3)
        if flops:
            r["TFLOP_s"] = round(flops / us / 1e6, 1)
            r["frac_mfma_f16"] = round(flops / us / 1e6 / 2500.0, 3)
        rows.append(r)
        print(f"{name:58s} {us:9.2f} us {r['GB_s']:8.0f} GB/s" + (f" {r['TFLOP_s']:8.1f} TFLOP/s" if flops else "")
              + (f"  stream read of the same bytes {r['stream_read_same_bytes_us']:.2f} us ({r['frac_of_stream_read']:.2f})" if ceiling else ""),
              file=sys.stderr, flush=True)

    shapes = [(4, 4096, 4096, 64, (1, 4, 16, 128, 512, 4096)), (4, 1024, 4096, 64, (1,)), (2, 14336, 4096, 16, (1, 4, 16, 128, 512, 4096)),
              (2, 4096, 14336, 16, (1, 4, 16, 128, 512, 4096)), (3, 14336, 4096, 64, (1, 8, 128, 4096)), (3, 4096, 14336, 64, (1, 8, 128))]
    for nbits, n, k, gs, batches in shapes:
        wbytes = (n * k * nbits // 8 if nbits != 3 else ((n + 9) // 10) * k * 4) + 2 * (n * k // gs) + 4 * (n * k // gs // META_GROUP) + 4
        nl = max(2, min(16, (320 << 20) // wbytes + 1))
        layers, codes = [], []
        for i in range(nl):
            d, q = random_desc(nbits, n, k, gs, 100 * nbits + i, dev)
            layers.append(d)
            if i < 4:
                codes.append(q)
        tag = f"w{nbits} {n}x{k} g{gs}"
        with torch.cuda.stream(stream):
            # packers and the de-quantiser (one-time work at load, streaming kernels)
            pk = {4: (packing.pack_4bit_u8_common, packing.unpack_4bit_u8_common), 2: (packing.pack_2bit_u8_common, packing.unpack_2bit_u8_common),
                  3: (packing.pack_3bit_i32_common, packing.unpack_3bit_i32_common)}[nbits]
            packed = [pk[0](c) for c in codes]
        cbytes = packed[0].numel() * packed[0].element_size()
        add(f"pack   {tag}", timed(lambda i: pk[0](codes[i % 4]), 12), n * k + cbytes)
        add(f"unpack {tag}", timed(lambda i: pk[1](packed[i % 4]), 12), n * k + cbytes)
        add(f"dequantize {tag}", timed(lambda i: hip_kernels.dequantize(layers[i % nl]), 12), wbytes + 2 * n * k)
        if gs in hip_kernels.QUANTIZE_GROUP_SIZES and n == 14336:
            # the quantiser on fp16 weights of the shape: reads 2 bytes and writes one unpacked code per weight
            wsrc = [torch.randn((n, k), device=dev).half() * 0.02 for _ in range(3)]
            with torch.cuda.stream(stream):
                add(f"quantize (min-max) {tag}", timed(lambda i: hip_kernels.quantize_groups(wsrc[i % 3], gs, nbits), 9), 3 * n * k)
                add(f"quantize (solver, 20 iterations at most) {tag}",
                    timed(lambda i: hip_kernels.quantize_groups(wsrc[i % 3], gs, nbits, iters=20), 6), 5 * n * k)
            del wsrc
        del codes, packed
        for m in batches:
            x = torch.randn((m, k), device=dev).half()
            y = torch.empty((m, n), device=dev, dtype=torch.float16)
            need = lib.hqq_matmul_workspace_bytes(layers[0].ref, m)
            ws = torch.zeros(max(int(need), 256), dtype=torch.uint8, device=dev)

            def f(i):
                rc = lib.hqq_matmul_transpose(layers[i % nl].ref, x.data_ptr(), m, y.data_ptr(), ws.data_ptr(), ws.numel(), stream.cuda_stream)
                if rc != 0:
                    raise _lib.HqqError(rc, "hqq_matmul_transpose")

            fam = lib.hqq_matmul_kernel_family(layers[0].ref, m)
            add(f"matmul {tag} M={m} (family {fam})", timed(f, 48 if m <= 16 else 16), wbytes + 2 * m * (n + k), 2.0 * m * n * k,
                ceiling=m <= 16)
            if fam == _lib.FAM_DQGEMM:
                # the matrix-core tile kernel, forced, beside the de-quantise + library GEMM form chosen for wide batches

                def t(i):
                    rc = lib.hqq_matmul_transpose_ex(layers[i % nl].ref, x.data_ptr(), m, y.data_ptr(), ws.data_ptr(), ws.numel(),
                                                     _lib.FAM_TILE, stream.cuda_stream)
                    if rc != 0:
                        raise _lib.HqqError(rc, "hqq_matmul_transpose_ex")

                add(f"matmul {tag} M={m} (family {_lib.FAM_TILE}, forced)", timed(t, 8), wbytes + 2 * m * (n + k), 2.0 * m * n * k)
            if (nbits, n, m) in ((2, 14336, 128), (2, 14336, 512)) and fam != _lib.FAM_LDS:
                # the other prefill kernel (weights de-quantised into LDS), forced, beside the one the library picks

                def g(i):
                    rc = lib.hqq_matmul_transpose_ex(layers[i % nl].ref, x.data_ptr(), m, y.data_ptr(), ws.data_ptr(), ws.numel(),
                                                     _lib.FAM_LDS, stream.cuda_stream)
                    if rc != 0:
                        raise _lib.HqqError(rc, "hqq_matmul_transpose_ex")

                add(f"matmul {tag} M={m} (family {_lib.FAM_LDS}, forced)", timed(g, 16), wbytes + 2 * m * (n + k), 2.0 * m * n * k)
        del layers
        torch.cuda.empty_cache()
    return rows


def prefill_section(dev, tokens=128, repeats=3):
    """The prompt pass alone (all experts resident): milliseconds for `tokens` tokens through the 32 layers."""
    import torch

    from mixtral_offloading_amd import build_model as bm

    cfg = bm.mixtral_config()
    off = bm.OffloadConfig(main_size=32 * 8, offload_size=0, buffer_size=4, offload_per_layer=0)
    model = bm.build_model(dev, bm.default_quant_config(), off, model_config=cfg, seed=0, max_positions=max(1024, tokens + 2))
    gen = torch.Generator(device=dev).manual_seed(1)
    prompt = torch.randint(0, cfg.vocab_size, (tokens,), device=dev, generator=gen)
    cache = model.new_cache(tokens + 2)
    model.forward(prompt, cache, 0)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(repeats):
        model.forward(prompt, cache, 0)
    torch.cuda.synchronize()
    return {"prefill_tokens": tokens, "prefill_ms": round((time.perf_counter() - t0) / repeats * 1e3, 2),
            "model": "Mixtral-8x7B architecture, 32 layers, random-init, attention 4-bit g64, experts 2-bit g16"}


def decode_section(dev, tokens_resident=256, tokens_offload=256):
    """Tokens per second of the whole model; every figure is measured between synchronisations
    around the decode loop, prompt processing excluded."""
    import gc

    import torch

    from mixtral_offloading_amd import build_model as bm
    from mixtral_offloading_amd.mixtral_model import DecodeGraph

    out = {"model": "Mixtral-8x7B architecture, 32 layers, random-init, attention 4-bit g64, experts 2-bit g16, "
                    "64-token prompt, greedy, batch 1"}
    cfg = bm.mixtral_config()
    gen = torch.Generator(device=dev).manual_seed(1)
    prompt = torch.randint(0, cfg.vocab_size, (64,), device=dev, generator=gen)

    def timed_eager(model, n):
        cache = model.new_cache(64 + n + 1)
        tok = model.forward(prompt, cache, 0)[-1].argmax()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for i in range(n):
            tok = model.forward(tok.view(1), cache, 64 + i)[-1].argmax()
        torch.cuda.synchronize()
        return n / (time.perf_counter() - t0)

    for per_layer in (8, 4, 2):
        off = bm.OffloadConfig(main_size=32 * per_layer, offload_size=32 * (8 - per_layer), buffer_size=4,
                               offload_per_layer=8 - per_layer)
        model = bm.build_model(dev, bm.default_quant_config(), off, model_config=cfg, seed=0, max_positions=1024)
        model.generate(prompt, 2)  # workspaces, allocator pools
        if per_layer == 8:
            dec = DecodeGraph(model, 64 + tokens_resident + 4)
            dec.prefill(prompt)
            dec.capture()
            dec.prefill(prompt)
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            for _ in range(tokens_resident):
                dec.step()
            torch.cuda.synchronize()
            out["all_experts_resident_graph_tok_s"] = round(tokens_resident / (time.perf_counter() - t0), 1)
            out["all_experts_resident_graph_tokens"] = tokens_resident
            del dec
            # the same step with a 512-token KV cache: 64 tokens after a 512-token prompt
            ctx = torch.randint(0, cfg.vocab_size, (512,), device=dev, generator=gen)
            dec = DecodeGraph(model, 512 + 64 + 4)
            dec.prefill(ctx)
            dec.capture()
            dec.prefill(ctx)
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            for _ in range(64):
                dec.step()
            torch.cuda.synchronize()
            out["all_experts_resident_graph_tok_s_kv512"] = round(64 / (time.perf_counter() - t0), 1)
            del dec, ctx
            out["all_experts_resident_eager_tok_s"] = round(timed_eager(model, 48), 1)
            # prompt processing (the multi-token kernels): a 128-token prompt through all 32 layers
            long_prompt = torch.randint(0, cfg.vocab_size, (128,), device=dev, generator=gen)
            cache = model.new_cache(130)
            model.forward(long_prompt, cache, 0)
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            for _ in range(3):
                model.forward(long_prompt, cache, 0)
            torch.cuda.synchronize()
            out["prefill_128_tokens_ms"] = round((time.perf_counter() - t0) / 3 * 1e3, 2)
            del cache
        else:
            before = model.expert_cache.stats()
            out[f"expert_cache_{per_layer}_per_layer_tok_s"] = round(timed_eager(model, tokens_offload), 2)
            st = model.expert_cache.stats()
            out[f"expert_cache_{per_layer}_per_layer_detail"] = {
                "tokens": tokens_offload, "hits": st["hits"] - before["hits"], "misses": st["misses"] - before["misses"],
                "GB_copied_host_to_device": round((st["bytes_copied"] - before["bytes_copied"]) / 1e9, 2)}
            # the same with speculative loads: the next layer's router applied one layer early picks what to prefetch
            # (a guess is only acted on while the host link is idle and never evicts the latest request's experts
            # before guesses have proved the better bet: with this random router the link is busy all the time)
            model.speculate = True
            before = model.expert_cache.stats()
            out[f"expert_cache_{per_layer}_per_layer_speculative_tok_s"] = round(timed_eager(model, tokens_offload), 2)
            st = model.expert_cache.stats()
            loads = st["prefetch_loads"] - before["prefetch_loads"]
            out[f"expert_cache_{per_layer}_per_layer_speculative_detail"] = {
                "tokens": tokens_offload, "prefetch_loads": loads,
                "guesses_dropped_link_busy": st["prefetch_skipped_busy"] - before["prefetch_skipped_busy"],
                "guesses_dropped_protected": st["prefetch_skipped_protected"] - before["prefetch_skipped_protected"],
                "guess_accuracy": round((st["guess_right"] - before["guess_right"]) / max(1, st["guess_scored"] - before["guess_scored"]), 3),
                "repeat_rate": round((st["reuse_right"] - before["reuse_right"]) / max(1, st["reuse_scored"] - before["reuse_scored"]), 3),
                "misses": st["misses"] - before["misses"],
                "GB_copied_host_to_device": round((st["bytes_copied"] - before["bytes_copied"]) / 1e9, 2)}
            model.speculate = False
        del model
        gc.collect()
        torch.cuda.empty_cache()

    # the other mixed-quant variant of the reference: 3-bit g64 experts under the same 4-bit attention
    from mixtral_offloading_amd.hqq_core import BaseQuantizeConfig
    qc3 = bm.QuantConfig(ffn_config=BaseQuantizeConfig(nbits=3, group_size=64, quant_zero=True, quant_scale=True),
                         attn_config=bm.default_quant_config().attn_config)
    off = bm.OffloadConfig(main_size=32 * 8, offload_size=0, buffer_size=4, offload_per_layer=0)
    model = bm.build_model(dev, qc3, off, model_config=cfg, seed=0, max_positions=1024)
    dec = DecodeGraph(model, 64 + 128 + 4)
    dec.prefill(prompt)
    dec.capture()
    dec.prefill(prompt)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(128):
        dec.step()
    torch.cuda.synchronize()
    out["experts_3bit_g64_all_resident_graph_tok_s"] = round(128 / (time.perf_counter() - t0), 1)
    del dec, model
    gc.collect()
    torch.cuda.empty_cache()
    return out


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=400)
    ap.add_argument("--warmup", type=int, default=40)
    ap.add_argument("--batch", type=int, default=1, help="tokens per step (1 is the headline; 4 and 16 are parity-test sizes)")
    ap.add_argument("--experts", type=int, default=8, help="distinct experts the steps rotate over")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-decode", action="store_true", help="skip the whole-model decode section")
    ap.add_argument("--prefill-only", type=int, default=0, metavar="TOKENS",
                    help="time only the prompt pass of the whole model over TOKENS tokens and print that (for profiling)")
    ap.add_argument("--survey", action="store_true",
                    help="also time every kernel of the path (packers, de-quantiser, 2/3/4-bit matmuls at the Mixtral-8x7B "
                         "shapes and batches) and add the table as 'kernels'")
    ap.add_argument("--kernel-hash", action="store_true", help="print the hash of the dominant kernel's sources (the "
                    "counter profile records it beside its traffic figure) and exit")
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="also run plain 256 MiB device copies, so that a counter run can scale FETCH_SIZE / WRITE_SIZE "
                         "by what the same counters read for a copy of known size")
    args = ap.parse_args()
    if args.kernel_hash:
        print(kernel_source_hash())
        return
    if args.gpus != 1:
        print("bench.py measures one GPU: this build runs on a single MI355X (--gpus 1)", file=sys.stderr)
        sys.exit(2)

    import torch

    from mixtral_offloading_amd import _lib, hip_kernels

    assert torch.cuda.is_available(), "bench.py needs a GPU"
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    if args.prefill_only:
        print(json.dumps(prefill_section(dev, args.prefill_only)))
        return
    m = args.batch
    experts = [make_expert(i, dev) for i in range(args.experts)]
    descs = [(e[0]._desc(), e[1]._desc(), e[2]._desc()) for e in experts]
    gx = torch.Generator(device=dev).manual_seed(1234)
    x = torch.randn((m, HIDDEN), device=dev, generator=gx).half()
    y = torch.empty((m, HIDDEN), device=dev, dtype=torch.float16)
    h = torch.empty((m, FFN), device=dev, dtype=torch.float16)
    lib = _lib.lib
    need = lib.hqq_expert_ffn_workspace_bytes(descs[0][0].ref, descs[0][1].ref, descs[0][2].ref, m)
    ws = torch.zeros(max(int(need), 256), dtype=torch.uint8, device=dev)  # counters in its head start at zero
    stream = torch.cuda.Stream(device=dev)
    sp = stream.cuda_stream

    def ffn_step(i):
        w1, w2, w3 = descs[i % len(descs)]
        rc = lib.hqq_expert_ffn(w1.ref, w2.ref, w3.ref, x.data_ptr(), m, y.data_ptr(), None, 0, ws.data_ptr(),
                                ws.numel(), sp)
        if rc != 0:
            raise _lib.HqqError(rc, "hqq_expert_ffn")

    def gate_up_step(i):
        w1, _, w3 = descs[i % len(descs)]
        rc = lib.hqq_gate_up(w1.ref, w3.ref, x.data_ptr(), m, h.data_ptr(), ws.data_ptr(), ws.numel(), sp)
        if rc != 0:
            raise _lib.HqqError(rc, "hqq_gate_up")

    def timed(fn, warmup, steps):
        with torch.cuda.stream(stream):
            for i in range(warmup):
                fn(i)
            torch.cuda.synchronize()
            e0 = torch.cuda.Event(enable_timing=True)
            e1 = torch.cuda.Event(enable_timing=True)
            e0.record(stream)
            for i in range(steps):
                fn(warmup + i)
            e1.record(stream)
            torch.cuda.synchronize()
        return e0.elapsed_time(e1) / steps  # ms per step

    ms_step = timed(ffn_step, args.warmup, args.steps)
    ms_gate = timed(gate_up_step, args.warmup, args.steps)

    # Two reference points for the dominant kernel, timed the same way in the same process: the same launch on ONE
    # expert (its 44 MB stay in the 256 MB last-level cache, so HBM is out of the picture), and a plain 128-bit
    # streaming read of the launch's algorithmic bytes, rotating over more than 256 MB like the kernel itself.
    def gate_up_resident(i):
        w1, _, w3 = descs[0]
        rc = lib.hqq_gate_up(w1.ref, w3.ref, x.data_ptr(), m, h.data_ptr(), ws.data_ptr(), ws.numel(), sp)
        if rc != 0:
            raise _lib.HqqError(rc, "hqq_gate_up")

    ms_gate_resident = timed(gate_up_resident, args.warmup, args.steps)
    probe = load_probe()
    nbytes = gate_up_bytes(m)
    span = (nbytes + 4095) // 4096 * 4096
    slots = (320 << 20) // span + 1
    pool = torch.empty(slots * span, dtype=torch.uint8, device=dev).fill_(3)
    sink = torch.zeros(4, dtype=torch.int32, device=dev)

    def stream_read_step(i):
        rc = probe.hqq_probe_stream_read(pool.data_ptr() + (i % slots) * span, nbytes, sink.data_ptr(), sp)
        if rc != 0:
            raise RuntimeError(f"hqq_probe_stream_read: {rc}")

    ms_read = timed(stream_read_step, args.warmup, args.steps)
    del pool
    if args.calibrate_copy:
        src = torch.empty(256 << 20, dtype=torch.uint8, device=dev).fill_(1)
        dst = torch.empty_like(src)
        for _ in range(4):
            dst.copy_(src)
        torch.cuda.synchronize()
        print(f"calibration: 4 device copies of {src.numel()} bytes (reads {src.numel()}, writes {src.numel()} each)",
              file=sys.stderr)

    traffic, traffic_note = profiled_traffic()
    value = ffn_step_bytes(m) / (ms_step * 1e-3) / 1e9
    achieved = gate_up_bytes(m) / (ms_gate * 1e-3) / 1e9
    out = {
        "metric": "dequant-GEMV HBM GB/s (% of peak); Mixtral-8x7B mixed-quant decode tok/s",
        "value": round(value, 1), "unit": "GB/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(ms_step, 5), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "f16", "data": "synthetic",
        "config": {"workload": f"configs[1]: 2-bit g16 expert FFN GEMV at Mixtral shapes (w1,w3 14336x4096, w2 4096x14336), "
                               f"batch {m}, 8-bit meta-quantised scale/zero (meta group 128), rotating over "
                               f"{args.experts} experts ({args.experts * 66.4:.0f} MB of weights)",
                   "bytes_per_step": ffn_step_bytes(m), "pct_of_hbm_peak": round(100 * value / HBM_PEAK_GBS, 2)},
        "roofline": {"bound": "hbm", "achieved": round(achieved, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": round(achieved / HBM_PEAK_GBS, 4),
                     # a recorded figure, read from the tracked counter profile (taken at batch 1), not measured here
                     "traffic": traffic if m == 1 else None,
                     "traffic_source": "profiles/gemv_strip_kernel_ffn_2bit_g16_m1.txt: " + traffic_note,
                     "kernel": "gemv_strip_kernel<2,1,4,2,8,1,2,1,false,0> as launched by hqq_gate_up (w1 and w3 in one grid, one launch)",
                     "bytes_per_launch": gate_up_bytes(m), "us_per_launch": round(ms_gate * 1e3, 3),
                     "us_per_launch_cache_resident": round(ms_gate_resident * 1e3, 3),
                     "stream_read_us": round(ms_read * 1e3, 3),
                     "frac_of_stream_read": round(ms_read / ms_gate, 4)},
    }
    if not args.no_cpu_baseline:
        out["cpu_baseline"] = cpu_baseline(experts[0], x, attention=make_attention(dev))
    if args.survey:
        out["kernels"] = survey_section(dev)
    if not args.no_decode:
        del experts, descs
        torch.cuda.empty_cache()
        out["decode"] = decode_section(dev)
    print(json.dumps(out))


if __name__ == "__main__":
    main()
