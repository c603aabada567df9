#!/usr/bin/env python3
"""Benchmark of the gfx950 INT8 W8A8 fused-MoE layer on one MI355X.

A step is one ``fused_experts`` call (quant → align → gate_up GEMM + SiLU·mul → quant → down GEMM →
combine) on one batch of M tokens of the Qwen3-30B-A3B-shaped layer (E=128, top-8, H=2048, I=768,
moe_align block 64), inputs resident in HBM.  The headline value is tokens/s at ``--m`` (default
8192, the prefill point); ``sweep_detail`` repeats the measurement at M = 16, 128, 512, 1024, 8192 and
reports layer-level INT8 TOP/s and HBM GB/s from the algorithmic work of the sampled routing; the
line ends with compact views of the same (``stages``, ``decode_mix``, ``sweep``).  Successive
steps rotate over several independent weight copies so that no step finds its weights in the
256 MB last-level cache.

Prints one JSON line.  ``roofline`` describes the dominant kernel (the gate_up GEMM), timed with
events on the launch stream; ``cpu_baseline`` is the torch-native W8A8 MoE of the CPU oracle timed
on the host cores (a reported baseline, not a target).
"""

from __future__ import annotations

import argparse
import importlib
import json
import os
import sys
import time
from pathlib import Path

ROOT = Path(__file__).resolve().parent
if str(ROOT) not in sys.path:
    sys.path.insert(0, str(ROOT))

PEAK_INT8_OPS = 5.0e15  # MI355X dense INT8 MFMA, op/s
PEAK_HBM_BPS = 8.0e12  # MI355X HBM3E, byte/s
SWEEP_M = (16, 128, 512, 1024, 8192)


def _profile_traffic(kernel: str, M: int):
    """HBM bytes per launch from the rocprofv3 --pmc summary committed under profiles/ (FETCH_SIZE and
    WRITE_SIZE, each scaled by what the counter reads for a plain copy of known size), when one has
    been recorded for this kernel and batch size; otherwise None.  A hardware counter cannot be read from
    inside this process, so the figure is a recorded one and says where it was recorded."""
    name = "profiles/hbm_traffic_gate_up.txt"
    path = ROOT / name
    if not path.exists():
        return None, None
    for line in path.read_text().splitlines():
        f = line.split()
        if len(f) == 7 and f[0] == "traffic" and f[1] == kernel and f[2] == f"M={M}":
            return (float(f[3]) * float(f[5]) + float(f[4]) * float(f[6])) * 1024.0, name
    return None, None


def build_workload(pkg, torch, shape_name: str, M: int, copies: int, seed: int):
    inputs = pkg.inputs
    shape = inputs.SHAPES[shape_name]
    base = inputs.make_inputs(shape, M, seed=seed)
    dev = base.to("cuda:0")
    weights = [(dev.w1, dev.w2, dev.w1_scale, dev.w2_scale)]
    for c in range(1, copies):
        # independent copies: same distribution, different bits (a roll along the expert axis)
        weights.append(tuple(t.roll(c, 0).contiguous() for t in weights[0]))
    return shape, base, dev, weights


def time_layer(pkg, torch, dev, weights, steps: int, warmup: int, variant: str) -> float:
    def step(i):
        w1, w2, s1, s2 = weights[i % len(weights)]
        return pkg.fused_experts(dev.hidden_states, w1, w2, dev.topk_weights, dev.topk_ids,
                                 use_int8_w8a8=True, per_channel_quant=True, w1_scale=s1, w2_scale=s2,
                                 gemm_variant=variant)

    for i in range(warmup):
        step(i)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for i in range(steps):
        step(i)
    torch.cuda.synchronize()
    return (time.perf_counter() - t0) / steps


def layer_percentiles(pkg, torch, dev, weights, steps: int, variant: str) -> dict:
    """Spread of the single-call duration: an event pair around every call (the mean of these reads a
    little above the back-to-back figure, which overlaps host work with the device)."""
    pairs = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(steps)]
    torch.cuda.synchronize()
    for i, (a, b) in enumerate(pairs):
        w1, w2, s1, s2 = weights[i % len(weights)]
        a.record()
        pkg.fused_experts(dev.hidden_states, w1, w2, dev.topk_weights, dev.topk_ids, use_int8_w8a8=True,
                          per_channel_quant=True, w1_scale=s1, w2_scale=s2, gemm_variant=variant)
        b.record()
    torch.cuda.synchronize()
    ts = sorted(a.elapsed_time(b) * 1e3 for a, b in pairs)
    pick = lambda q: ts[min(len(ts) - 1, int(q * len(ts)))]
    return {"p10": pick(0.10), "p50": pick(0.50), "p90": pick(0.90)}


def time_gate_up_kernel(pkg, torch, shape, dev, weights, steps: int, warmup: int, variant: str) -> float:
    """Average duration (s) of the gate_up GEMM launch, from event pairs on the launch stream."""
    M, k = dev.topk_ids.shape
    x_q, a1 = pkg.per_token_quant_int8(dev.hidden_states)
    s, e, npp = pkg.moe_align_block_size(dev.topk_ids, 64, shape.E_total)
    starts = [torch.cuda.Event(enable_timing=True) for _ in range(steps)]
    stops = [torch.cuda.Event(enable_timing=True) for _ in range(steps)]
    for i in range(warmup):
        w1, _, s1, _ = weights[i % len(weights)]
        pkg.gemm_gate_up_silu(x_q, a1, w1, s1, s, e, npp, k, 64, M * k, variant)
    torch.cuda.synchronize()
    for i in range(steps):
        w1, _, s1, _ = weights[i % len(weights)]
        starts[i].record()
        pkg.gemm_gate_up_silu(x_q, a1, w1, s1, s, e, npp, k, 64, M * k, variant)
        stops[i].record()
    torch.cuda.synchronize()
    return sum(a.elapsed_time(b) for a, b in zip(starts, stops)) / steps * 1e-3


def time_stages(pkg, torch, shape, dev, weights, steps: int, warmup: int, variant: str) -> list:
    """Every launch of the layer on its own: direct C-ABI calls into preallocated buffers, an event pair per
    call on the launch stream (median), with the algorithmic bytes / int8 ops of that launch and the fraction of
    the roofline that bounds it.  (A launch that does almost nothing still reads about 4 us.  Timed alone back to
    back the gate_up GEMM reads about 10 % above its duration inside the layer, where the memory-bound
    launches around it let the clock recover; the dispatch durations of a kernel trace of the whole layer are
    the in-situ figures.)"""
    abi = pkg._abi
    lib = abi.load()
    M, k = dev.topk_ids.shape
    P, H, I, E = M * k, shape.H, shape.I, shape.E_total
    n_act = int(torch.unique(dev.topk_ids).numel())
    x_q, a1 = pkg.per_token_quant_int8(dev.hidden_states)
    s, e, npp = pkg.moe_align_block_size(dev.topk_ids, 64, E)
    w1, w2, s1, s2 = weights[0]
    act = pkg.gemm_gate_up_silu(x_q, a1, w1, s1, s, e, npp, k, 64, P, variant)
    h_q, a2 = pkg.per_token_quant_int8(act)
    down = pkg.gemm_down(h_q, a2, w2, s2, dev.topk_weights, s, e, npp, 64, variant)
    out = torch.empty_like(dev.hidden_states)
    ws_bytes = lib.moe_i8_align_workspace_bytes(P, E, 64)
    ws = torch.empty(max(ws_bytes, 256), dtype=torch.uint8, device="cuda:0")
    ids32 = dev.topk_ids.to(torch.int32).contiguous()
    tw = dev.topk_weights.reshape(-1).contiguous()
    stream = torch.cuda.current_stream().cuda_stream
    v = {"auto": abi.GEMM_AUTO, "stream": abi.GEMM_STREAM, "tile": abi.GEMM_TILE, "narrow": abi.GEMM_NARROW,
         "tile_wide": abi.GEMM_TILE_WIDE, "tile_deep": abi.GEMM_TILE_DEEP,
         "tile_ring": abi.GEMM_TILE_RING}[variant]
    n = len(weights)
    p_ = lambda t: t.data_ptr()
    stages = [
        ("quant input",
         lambda i: lib.moe_i8_quant_rows(p_(dev.hidden_states), abi.DTYPE_BF16, M, H, H, None, 1, M, p_(x_q), p_(a1), stream),
         3 * M * H + 4 * M, 0),
        ("moe_align",
         lambda i: lib.moe_i8_align_block_size(p_(ids32), P, E, 64, p_(s), s.numel(), p_(e), e.numel(), p_(npp), p_(ws),
                                               ws.numel(), stream),
         8 * P, 0),
        ("gemm gate_up + SiLU*mul",
         lambda i: lib.moe_i8_gemm_gate_up_silu(p_(x_q), p_(a1), p_(weights[i % n][0]), p_(weights[i % n][2]), p_(s), p_(e),
                                                p_(npp), P, k, E, H, I, 64, s.numel(), p_(act), v, stream),
         n_act * (2 * I * H + 8 * I) + M * H + 4 * M + 2 * P * I + 4 * P, 4 * P * I * H),
        ("quant activations",
         lambda i: lib.moe_i8_quant_rows(p_(act), abi.DTYPE_BF16, P, I, I, None, 1, P, p_(h_q), p_(a2), stream),
         3 * P * I + 4 * P, 0),
        ("gemm down * routed weight",
         lambda i: lib.moe_i8_gemm_down(p_(h_q), p_(a2), p_(weights[i % n][1]), p_(weights[i % n][3]), p_(tw), p_(s), p_(e),
                                        p_(npp), P, E, H, I, 64, s.numel(), p_(down), v, stream),
         n_act * (H * I + 4 * H) + P * I + 8 * P + 2 * P * H, 2 * P * I * H),
        ("moe_sum", lambda i: lib.moe_i8_sum(p_(down), p_(out), M, k, H, stream), 2 * (k + 1) * M * H, 0),
    ]
    result = []
    # After a stretch of light launches the first dozens of calls of a matrix-bound kernel run through a
    # transient of the board's power control (first faster, then up to 25 % slower, then steady): every stage
    # gets at least 40 untimed calls, and the median of the timed ones is reported.
    warmup = max(warmup, 40)
    for name, fn, nbytes, ops in stages:
        for i in range(warmup):
            abi.check(fn(i))
        pairs = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(steps)]
        torch.cuda.synchronize()
        for i, (a, b) in enumerate(pairs):
            a.record()
            fn(i)
            b.record()
        torch.cuda.synchronize()
        times = sorted(a.elapsed_time(b) for a, b in pairs)
        t = times[len(times) // 2] * 1e-3
        hbm, mfma = nbytes / t / PEAK_HBM_BPS, ops / t / PEAK_INT8_OPS
        result.append({"stage": name, "us": t * 1e6, "bytes": nbytes, "int8_ops": ops, "hbm_frac": hbm,
                       "mfma_frac": mfma, "bound": "mfma" if mfma > hbm else "hbm"})
    return result


def gate_up_work(shape, M: int, topk_ids):
    """Algorithmic work of one gate_up GEMM launch: int8 ops, and HBM bytes (weights and channel
    scales of the routed-to experts, int8 activations and their scales in, bf16 activations out)."""
    import torch

    k = topk_ids.shape[1]
    P = M * k
    n_act = int(torch.unique(topk_ids).numel())
    ops = 4 * P * shape.I * shape.H
    nbytes = n_act * (2 * shape.I * shape.H + 8 * shape.I) + M * shape.H + 4 * M + 2 * P * shape.I + 4 * P
    return ops, nbytes, n_act


def time_weight_requant(pkg, torch, shape, steps: int, warmup: int) -> dict:
    """Trainer bf16 expert weights of the whole layer → int8 kernel layout, written in place into the
    engine's tensors (what happens to every MoE layer after each policy step).  HBM-bound: 2 bytes
    read and 1 written per weight, plus one fp32 scale per output channel."""
    E, I, H = shape.E_total, shape.I, shape.H
    g = torch.Generator(device="cuda:0").manual_seed(1)
    gate, up = (torch.randn(E, I, H, generator=g, device="cuda:0").mul_(0.02).to(torch.bfloat16) for _ in range(2))
    down = torch.randn(E, H, I, generator=g, device="cuda:0").mul_(0.02).to(torch.bfloat16)
    params = pkg.quantize_expert_weights(gate, up, down)
    for _ in range(warmup):
        pkg.quantize_expert_weights(gate, up, down, out=params)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps):
        pkg.quantize_expert_weights(gate, up, down, out=params)
    torch.cuda.synchronize()
    t = (time.perf_counter() - t0) / steps
    nbytes = 3 * E * I * H * 3 + 4 * E * (2 * I + H)
    return {"us": t * 1e6, "bytes": nbytes, "hbm_gbps": nbytes / t / 1e9, "hbm_frac": nbytes / t / PEAK_HBM_BPS,
            "layers_per_s": 1.0 / t}


def time_router(pkg, torch, shape, M: int, steps: int, warmup: int) -> dict:
    """The routing step in front of the layer: fp32 logits [M, E] → top-k weights and ids (and the
    compact routed-experts record), one launch through the C-ABI with preallocated outputs, timed
    with an event pair per launch on the launch stream."""
    E, k = shape.E, shape.k
    grouped = shape.routing == "grouped"
    g = torch.Generator(device="cuda:0").manual_seed(2)
    logits = torch.randn(M, E, generator=g, device="cuda:0")
    bias = torch.randn(E, generator=g, device="cuda:0").mul_(0.1) if grouped else None
    w = torch.empty(M, k, dtype=torch.float32, device="cuda:0")
    ids = torch.empty(M, k, dtype=torch.int32, device="cuda:0")
    record = torch.empty(M, 1, k, dtype=torch.uint8 if E <= 256 else torch.uint16, device="cuda:0")
    lib, abi = pkg._abi.load(), pkg._abi
    stream = torch.cuda.current_stream().cuda_stream

    def launch():
        abi.check(lib.moe_i8_route_topk(
            logits.data_ptr(), M, E, k, abi.SCORE_SIGMOID if grouped else abi.SCORE_SOFTMAX,
            None if bias is None else bias.data_ptr(), shape.n_group if grouped else 1,
            shape.topk_group if grouped else 1, int(grouped), 1, 1.0, w.data_ptr(), ids.data_ptr(),
            record.data_ptr(), 1 if E <= 256 else 2, k, 0, stream))

    for _ in range(warmup):
        launch()
    pairs = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(steps)]
    torch.cuda.synchronize()
    for a, b in pairs:
        a.record()
        launch()
        b.record()
    torch.cuda.synchronize()
    t = sum(a.elapsed_time(b) for a, b in pairs) / steps * 1e-3
    nbytes = M * E * 4 + M * k * (4 + 4 + record.element_size())
    return {"M": M, "us": t * 1e6, "bytes": nbytes, "hbm_gbps": nbytes / t / 1e9}


DECODE_BUCKETS = (1, 2, 4, 8, 16, 24, 32, 48, 64, 96, 128, 160, 192, 224, 256)


def time_decode_mix(pkg, torch, shape_name: str, layers: int, steps: int) -> dict:
    """Continuous-batching decode: `layers` independently seeded layers of the shape called back to back,
    `steps` steps whose batch size is drawn uniformly from 1..256, routing re-drawn for every step and
    layer, every layer fed a fresh N(0,1) input (chaining random layers would overflow bf16 within a few
    layers).  Two ways: eager calls with the true batch size, and HIP-graph replays of the whole stack
    captured once per batch-size bucket with the batch padded up to the bucket (padding rows are routed
    like row 0 and thrown away) — the way a serving engine replays captured graphs.  Tokens per second
    count real tokens only."""
    shape = pkg.inputs.SHAPES[shape_name]
    E, k, H, I = shape.E_total, shape.k + (1 if shape.shared_expert else 0), shape.H, shape.I
    dev = "cuda:0"
    g = torch.Generator(device=dev).manual_seed(5)
    stack = []
    for _ in range(layers):
        stack.append((torch.randint(-127, 128, (E, 2 * I, H), generator=g, dtype=torch.int8, device=dev),
                      torch.randint(-127, 128, (E, H, I), generator=g, dtype=torch.int8, device=dev),
                      torch.empty(E, 2 * I, device=dev).uniform_(0.002, 0.01, generator=g),
                      torch.empty(E, H, device=dev).uniform_(0.002, 0.01, generator=g)))
    cpu = torch.Generator().manual_seed(6)
    max_m = DECODE_BUCKETS[-1]
    sizes = torch.randint(1, max_m + 1, (steps,), generator=cpu).tolist()
    n_tables = 64  # routing tables and inputs drawn beforehand, walked cyclically by (step, layer)
    tables = [tuple(t.to(dev) for t in pkg.inputs.route(shape, max_m, cpu)) for _ in range(n_tables)]
    xs = [torch.randn(max_m, H, generator=cpu).to(torch.bfloat16).to(dev) for _ in range(8)]
    ws = torch.empty(pkg.workspace_bytes(max_m, k, E, H, I, 64), dtype=torch.uint8, device=dev)
    kw = dict(use_int8_w8a8=True, per_channel_quant=True, workspace=ws)

    def eager_step(t, M):
        for l, (w1, w2, s1, s2) in enumerate(stack):
            tw, ids = tables[(t * layers + l) % n_tables]
            pkg.fused_experts(xs[(t + l) % len(xs)][:M], w1, w2, tw[:M], ids[:M], w1_scale=s1, w2_scale=s2, **kw)

    for t in range(3):
        eager_step(t, sizes[t])
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for t, M in enumerate(sizes):
        eager_step(t, M)
    torch.cuda.synchronize()
    eager = time.perf_counter() - t0

    # graphs: static inputs per bucket; the routing of every layer is refreshed by device copies before a replay
    static_x = torch.zeros(max_m, H, dtype=torch.bfloat16, device=dev)
    static_tw = torch.zeros(layers, max_m, k, dtype=torch.float32, device=dev)
    static_ids = torch.zeros(layers, max_m, k, dtype=torch.int32, device=dev)
    all_tw = torch.stack([t[0] for t in tables])   # [n_tables, max_m, k]
    all_ids = torch.stack([t[1] for t in tables])
    graphs = {}
    side = torch.cuda.Stream()
    for b in DECODE_BUCKETS:
        def run_stack():
            for l, (w1, w2, s1, s2) in enumerate(stack):
                pkg.fused_experts(static_x[:b], w1, w2, static_tw[l, :b], static_ids[l, :b], w1_scale=s1, w2_scale=s2, **kw)
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            run_stack()
        torch.cuda.current_stream().wait_stream(side)
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            run_stack()
        graphs[b] = graph
    order = torch.arange(layers, device=dev)

    def graph_step(t, M):
        b = next(x for x in DECODE_BUCKETS if x >= M)
        idx = (t * layers + order) % n_tables
        static_tw.copy_(all_tw[idx])
        static_ids.copy_(all_ids[idx])
        if M < b:  # padding rows follow row 0's routing
            static_tw[:, M:b] = static_tw[:, :1]
            static_ids[:, M:b] = static_ids[:, :1]
        static_x[:M].copy_(xs[t % len(xs)][:M])
        graphs[b].replay()

    for t in range(3):
        graph_step(t, sizes[t])
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for t, M in enumerate(sizes):
        graph_step(t, M)
    torch.cuda.synchronize()
    replay = time.perf_counter() - t0
    tokens = sum(sizes)
    small = sum(1 for M in sizes if M * k <= 3 * E)
    del stack, graphs
    torch.cuda.empty_cache()
    return {"shape": shape_name, "layers": layers, "steps": steps, "tokens": tokens,
            "batch_sizes": f"uniform 1..{max_m}, mean {tokens / steps:.1f}",
            "eager": {"wall_s": eager, "tokens_per_s": tokens / eager, "us_per_layer_call": eager / (steps * layers) * 1e6},
            "hip_graph": {"wall_s": replay, "tokens_per_s": tokens / replay,
                          "us_per_layer_call": replay / (steps * layers) * 1e6, "buckets": list(DECODE_BUCKETS),
                          "note": "one captured graph of the whole stack per bucket; batch padded up to the bucket; "
                                  "includes the device copies that refresh inputs and routing"},
            "launches_per_layer": {"4 (down GEMM quantises its own input)": small, "5": steps - small}}


def time_mfma_ceiling(pkg, torch) -> dict:
    """What the device sustains on a register-only int8 MFMA loop (no memory traffic at all) with constant
    and with pseudo-random operand bits: the board's power limit lowers the clock as the operand bits
    toggle, so the second figure, not the published peak, is the ceiling of any int8 GEMM on real data
    here.  One launch of a few milliseconds on one workgroup per compute unit, best of four.  Next to it,
    as a datum that owes nothing to this repository: the vendor library's dense int8 GEMM (torch._int_mm)
    on the problem the gate_up GEMM of the headline point would be without experts, on the same kind of
    random data."""
    import ctypes

    res = {"unit": "TOP/s", "note": "int8 operations per second, v_mfma_i32_32x32x32_i8 from registers on every "
                                    "compute unit"}
    path = pkg._abi.PROBE_LIB_PATH
    if path.exists():
        lib = ctypes.CDLL(str(path))
        lib.moe_i8_probe_mfma_ops.restype = ctypes.c_double
        lib.moe_i8_probe_mfma_ops.argtypes = [ctypes.c_int, ctypes.c_int]
        lib.moe_i8_probe_mfma.restype = ctypes.c_int
        lib.moe_i8_probe_mfma.argtypes = [ctypes.c_int, ctypes.c_int, ctypes.c_int, ctypes.c_void_p, ctypes.c_longlong,
                                          ctypes.c_void_p]
        wgs = torch.cuda.get_device_properties(0).multi_processor_count
        iters = 20000
        sink = torch.empty(wgs * 512, dtype=torch.int32, device="cuda:0")
        stream = torch.cuda.current_stream().cuda_stream
        ops = lib.moe_i8_probe_mfma_ops(wgs, iters)
        for name, rnd in (("constant_operands", 0), ("random_operands", 1)):
            best = float("inf")
            for _ in range(4):
                a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
                a.record()
                rc = lib.moe_i8_probe_mfma(rnd, wgs, iters, sink.data_ptr(), sink.numel() * 4, stream)
                b.record()
                torch.cuda.synchronize()
                if rc != 0:
                    raise RuntimeError(f"MFMA probe launch failed with HIP error {rc}")
                best = min(best, a.elapsed_time(b) * 1e-3)
            res[name] = ops / best / 1e12
            res[name + "_frac_of_peak"] = ops / best / PEAK_INT8_OPS
    else:
        res["constant_operands"] = res["random_operands"] = None
    m, k, n = 65536, 2048, 1536
    try:
        g = torch.Generator(device="cuda:0").manual_seed(7)
        a_ = torch.randint(-127, 128, (m, k), generator=g, dtype=torch.int8, device="cuda:0")
        b_ = torch.randint(-127, 128, (n, k), generator=g, dtype=torch.int8, device="cuda:0")
        for _ in range(3):
            torch._int_mm(a_, b_.t())
        pairs = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(10)]
        torch.cuda.synchronize()
        for e0, e1 in pairs:
            e0.record()
            torch._int_mm(a_, b_.t())
            e1.record()
        torch.cuda.synchronize()
        t = sum(e0.elapsed_time(e1) for e0, e1 in pairs) / len(pairs) * 1e-3
        res["library_int_mm"] = {"m": m, "k": k, "n": n, "us": t * 1e6, "int8_tops": 2.0 * m * k * n / t / 1e12,
                                 "frac_of_peak": 2.0 * m * k * n / t / PEAK_INT8_OPS,
                                 "note": "torch._int_mm (vendor library), dense, no scale epilogue, no SiLU"}
    except Exception as exc:  # the datum is optional: a build of torch without the routine must not fail the bench
        res["library_int_mm"] = None
        res["library_int_mm_error"] = repr(exc)[:200]
    return res


def time_hbm_ceiling(torch) -> dict:
    """What a plain device-to-device copy of 1 GiB sustains (bytes read plus bytes written per second):
    the practical counterpart of the published HBM peak for the streaming kernels of the layer."""
    n = 1 << 30
    src = torch.empty(n, dtype=torch.uint8, device="cuda:0").random_(0, 255)
    dst = torch.empty_like(src)
    best = float("inf")
    for _ in range(5):
        a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        a.record()
        dst.copy_(src)
        b.record()
        torch.cuda.synchronize()
        best = min(best, a.elapsed_time(b) * 1e-3)
    return {"copy_GBps": 2 * n / best / 1e9, "frac_of_peak": 2 * n / best / PEAK_HBM_BPS, "unit": "GB/s"}


def time_dense_mlp(pkg, torch, M: int, H: int, I: int, steps: int, warmup: int) -> dict:
    """The shared-expert / dense W8A8 gated MLP on the same GEMM kernels with one group."""
    g = torch.Generator(device="cuda:0").manual_seed(3)
    x = torch.randn(M, H, generator=g, device="cuda:0").to(torch.bfloat16)
    w13 = torch.randint(-127, 128, (2 * I, H), generator=g, dtype=torch.int8, device="cuda:0")
    w2 = torch.randint(-127, 128, (H, I), generator=g, dtype=torch.int8, device="cuda:0")
    s13 = torch.rand(2 * I, generator=g, device="cuda:0") * 0.002 + 0.001
    s2 = torch.rand(H, generator=g, device="cuda:0") * 0.002 + 0.001
    for _ in range(warmup):
        pkg.w8a8_mlp(x, w13, s13, w2, s2)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps):
        pkg.w8a8_mlp(x, w13, s13, w2, s2)
    torch.cuda.synchronize()
    t = (time.perf_counter() - t0) / steps
    ops = 6 * M * I * H
    return {"M": M, "H": H, "I": I, "us": t * 1e6, "int8_tops": ops / t / 1e12, "mfma_frac": ops / t / PEAK_INT8_OPS}


OTHER_SHAPES = (
    ("glm-4.5-air", (32, 512, 4096)),  # Zipf-skewed routing, one always-on shared expert as expert id E
    ("deepseek-v3", (8, 64, 2048, 16384)),  # grouped top-k, all 256 experts on the one GPU
)


def time_other_shape(pkg, torch, oracle, shape_name: str, M: int, steps: int, warmup: int, cpu: bool) -> dict:
    """One layer-level line for a shape that is a parity case, not the headline: layer time, the
    algorithmic HBM / MFMA fractions of the sampled routing, the padded-row ratio of moe_align, and
    (for the small batches) the CPU checker's time on the experts this batch touches.  The weights of
    these shapes (2-11 GB) are far larger than the 256 MB last-level cache, so one copy is enough."""
    shape = pkg.inputs.SHAPES[shape_name]
    inp = pkg.inputs.make_inputs(shape, M, seed=M + 3, device="cuda:0", weights_on_device=True)

    def step():
        return pkg.fused_experts(*inp.fused_experts_args(), **inp.fused_experts_kwargs())

    for _ in range(warmup):
        step()
    pairs = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(steps)]
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for a, b in pairs:
        a.record()
        step()
        b.record()
    torch.cuda.synchronize()
    t = (time.perf_counter() - t0) / steps
    ts = sorted(a.elapsed_time(b) * 1e3 for a, b in pairs)
    _, _, npp = pkg.moe_align_block_size(inp.topk_ids, 64, shape.E_total)
    P = M * inp.topk_ids.shape[1]
    ids_cpu = inp.topk_ids.cpu()
    ops, nbytes = pkg.inputs.algorithmic_ops(shape, M), pkg.inputs.algorithmic_bytes(shape, M, ids_cpu)
    r3 = lambda x: float(f"{x:.4g}")
    line = {"shape": shape_name, "M": M, "us": r3(t * 1e6), "p50_us": r3(ts[len(ts) // 2]),
            "n_active": int(torch.unique(ids_cpu).numel()), "padded_over_pairs": r3(int(npp.cpu()) / P),
            "layer_hbm_frac": r3(nbytes / t / PEAK_HBM_BPS), "layer_mfma_frac": r3(ops / t / PEAK_INT8_OPS),
            "bound": "hbm" if nbytes / PEAK_HBM_BPS >= ops / PEAK_INT8_OPS else "mfma"}
    if cpu:
        # only the experts this batch routes to travel to the host (ids remapped), so the checker does the same
        # arithmetic on a few GB instead of the whole layer
        used = torch.unique(ids_cpu.to(torch.int64))
        remap = torch.full((shape.E_total,), -1, dtype=torch.int64)
        remap[used] = torch.arange(used.numel())
        dev_used = used.to("cuda:0")
        args = (inp.hidden_states.cpu(), inp.w1[dev_used].cpu(), inp.w2[dev_used].cpu(), inp.topk_weights.cpu(),
                remap[ids_cpu.to(torch.int64)].to(torch.int32), inp.w1_scale[dev_used].cpu(), inp.w2_scale[dev_used].cpu())
        t0 = time.perf_counter()
        oracle.native_w8a8_moe(*args)
        tc = time.perf_counter() - t0
        # the CPU checker on the whole batch, one pass, no warm-up
        line["cpu_tokens_per_s"] = r3(M / tc)
        line["cpu_cores"] = torch.get_num_threads()
    del inp
    torch.cuda.empty_cache()
    return line


def cpu_baseline(oracle, torch, base, sample_m: int) -> dict:
    m = min(sample_m, base.hidden_states.shape[0])
    args = (base.hidden_states[:m], base.w1, base.w2, base.topk_weights[:m], base.topk_ids[:m],
            base.w1_scale, base.w2_scale)
    oracle.native_w8a8_moe(*args)  # warm-up
    best = float("inf")
    passes = 5
    for _ in range(passes):
        t0 = time.perf_counter()
        oracle.native_w8a8_moe(*args)
        best = min(best, time.perf_counter() - t0)
    return {
        "value": m / best,
        "unit": "tokens/s",
        "cores": torch.get_num_threads(),
        "kind": "port",
        "sample": f"first {m} tokens of the same seeded workload, torch-native W8A8 MoE of the oracle, "
                  f"best of {passes} after 1 warm-up ({best:.2f} s per pass; os.cpu_count()={os.cpu_count()})",
    }


def main() -> int:
    ap = argparse.ArgumentParser(description=__doc__, formatter_class=argparse.RawDescriptionHelpFormatter)
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=10)
    ap.add_argument("--m", type=int, default=8192, help="tokens per step of the headline measurement")
    ap.add_argument("--shape", default="qwen3-30b-a3b")
    ap.add_argument("--variant", default="auto", choices=["auto", "stream", "tile", "narrow", "tile_wide", "tile_deep", "tile_ring"])
    ap.add_argument("--weight-copies", type=int, default=4)
    ap.add_argument("--no-sweep", action="store_true")
    ap.add_argument("--no-cpu", action="store_true")
    ap.add_argument("--no-decode-mix", action="store_true")
    ap.add_argument("--no-other-shapes", action="store_true")
    ap.add_argument("--decode-layers", type=int, default=48)
    ap.add_argument("--decode-steps", type=int, default=500)
    ap.add_argument("--cpu-sample", type=int, default=8192, help="tokens of the workload the CPU baseline runs")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py measures one GPU: this build has no multi-GPU path (run with --gpus 1)", file=sys.stderr)
        return 2

    import torch

    pkg = importlib.import_module("prime_rl_amd")
    pkg._abi.load()  # fails loudly if the HIP library is not built
    if not torch.cuda.is_available():
        print("bench.py needs a GPU", file=sys.stderr)
        return 2

    sweep = []
    headline = None
    ms = [args.m] if args.no_sweep else sorted(set(SWEEP_M) | {args.m})
    base_headline = None
    for M in ms:
        shape, base, dev, weights = build_workload(pkg, torch, args.shape, M, args.weight_copies, seed=M)
        t_layer = time_layer(pkg, torch, dev, weights, args.steps, args.warmup, args.variant)
        t_k = time_gate_up_kernel(pkg, torch, shape, dev, weights, args.steps, args.warmup, args.variant)
        ops_layer = pkg.inputs.algorithmic_ops(shape, M)
        bytes_layer = pkg.inputs.algorithmic_bytes(shape, M, base.topk_ids)
        k_ops, k_bytes, n_act = gate_up_work(shape, M, base.topk_ids)
        hbm_bound = (bytes_layer / PEAK_HBM_BPS) >= (ops_layer / PEAK_INT8_OPS)
        if hbm_bound:
            roof = {"bound": "hbm", "achieved": k_bytes / t_k / 1e9, "peak": PEAK_HBM_BPS / 1e9, "unit": "GB/s"}
        else:
            roof = {"bound": "mfma", "achieved": k_ops / t_k / 1e12, "peak": PEAK_INT8_OPS / 1e12, "unit": "TOP/s",
                    "note": "int8 operations per second against the dense INT8 MFMA peak"}
        roof["frac"] = roof["achieved"] / roof["peak"]
        roof["kernel"] = "gemm gate_up + SiLU*mul"
        roof["kernel_us"] = t_k * 1e6
        # `traffic` = HBM bytes per launch as the hardware counters saw them, a recorded figure (a counter
        # cannot be read from inside this process): `traffic_source` names the summary it was read from
        roof["traffic"], roof["traffic_source"] = _profile_traffic("gate_up", M)
        roof["algorithmic_bytes"] = k_bytes
        point = {
            "M": M,
            "tokens_per_s": M / t_layer,
            "ms_per_step": t_layer * 1e3,
            "call_us": layer_percentiles(pkg, torch, dev, weights, args.steps, args.variant),
            "n_active_experts": n_act,
            "layer_int8_tops": ops_layer / t_layer / 1e12,
            "layer_mfma_frac": ops_layer / t_layer / PEAK_INT8_OPS,
            "layer_hbm_gbps": bytes_layer / t_layer / 1e9,
            "layer_hbm_frac": bytes_layer / t_layer / PEAK_HBM_BPS,
            "roofline": roof,
        }
        if M == args.m:
            point["stages"] = time_stages(pkg, torch, shape, dev, weights, max(args.steps // 2, 1),
                                          max(args.warmup // 2, 1), args.variant)
        sweep.append(point)
        if M == args.m:
            headline, base_headline = point, base
        del dev, weights
        torch.cuda.empty_cache()

    out = {
        "metric": "moe_layer_tokens_per_s",
        "value": headline["tokens_per_s"],
        "unit": "tokens/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": headline["ms_per_step"],
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "int8",
        "data": "synthetic",
        "config": {
            "workload": f"{args.shape} INT8 W8A8 MoE layer, M={args.m} tokens per step, top-8 of 128 experts, "
                        f"H=2048 I=768, moe_align block 64, {args.weight_copies} rotating weight copies",
            "shape": args.shape,
            "tokens_per_step": args.m,
            "gemm_variant": args.variant,
        },
        "roofline": {k: headline["roofline"][k]
                     for k in ("bound", "achieved", "peak", "unit", "frac", "traffic", "traffic_source", "algorithmic_bytes")},
        "roofline_kernel": headline["roofline"]["kernel"],
        "roofline_kernel_us": headline["roofline"]["kernel_us"],
        "layer_int8_tops": headline["layer_int8_tops"],
        "layer_mfma_frac": headline["layer_mfma_frac"],
        "layer_hbm_gbps": headline["layer_hbm_gbps"],
        "layer_hbm_frac": headline["layer_hbm_frac"],
        "sweep_detail": sweep,
    }
    if not args.no_sweep:
        out["router"] = [time_router(pkg, torch, pkg.inputs.SHAPES[args.shape], M, args.steps, args.warmup)
                         for M in ms]
        shape_h = pkg.inputs.SHAPES[args.shape]
        out["dense_mlp"] = [time_dense_mlp(pkg, torch, M, shape_h.H, shape_h.I, args.steps, args.warmup)
                            for M in (args.m, 8 * args.m)]
        out["weight_requant"] = time_weight_requant(pkg, torch, pkg.inputs.SHAPES[args.shape],
                                                    max(args.steps // 2, 1), max(args.warmup // 2, 1))
        out["mfma_ceiling"] = time_mfma_ceiling(pkg, torch)
        out["hbm_ceiling"] = time_hbm_ceiling(torch)
        if not args.no_decode_mix:
            out["decode_mix"] = time_decode_mix(pkg, torch, args.shape, args.decode_layers, args.decode_steps)
    oracle = None if args.no_cpu else importlib.import_module("oracle.moe_i8_oracle")
    if not args.no_sweep and not args.no_other_shapes:
        out["other_shapes"] = [
            time_other_shape(pkg, torch, oracle, name, M, max(args.steps // 2, 5), max(args.warmup // 2, 2),
                             cpu=oracle is not None and i < 2)
            for name, sizes in OTHER_SHAPES for i, M in enumerate(sizes)
        ]
    if not args.no_cpu:
        out["cpu_baseline"] = cpu_baseline(oracle, torch, base_headline, args.cpu_sample)
    # The last keys of the line are a compact view of both targets (whoever keeps only the end of a long
    # line still sees every batch size): per launch [name, us, fraction of its roofline, bound]; per batch
    # size the layer time, the p90 of single calls, the layer's fractions of 8 TB/s and of 5 POP/s, and
    # the gate_up kernel's duration and fraction of the roofline that bounds it.
    r3 = lambda x: float(f"{x:.4g}")
    if "decode_mix" in out:
        dm = out.pop("decode_mix")
        out["decode_mix_detail"] = dm
        out["decode_mix"] = {"us_per_layer_call": r3(dm["eager"]["us_per_layer_call"]),
                             "tokens_per_s": r3(dm["eager"]["tokens_per_s"]),
                             "hip_graph_us_per_layer_call": r3(dm["hip_graph"]["us_per_layer_call"]),
                             "layers": dm["layers"], "steps": dm["steps"]}
    if "stages" in headline:
        out["stages"] = [[st["stage"], r3(st["us"]), r3(max(st["hbm_frac"], st["mfma_frac"])), st["bound"]]
                         for st in headline["stages"]]
    out["sweep"] = [{"M": pt["M"], "us": r3(pt["ms_per_step"] * 1e3), "p90_us": r3(pt["call_us"]["p90"]),
                     "layer_hbm_frac": r3(pt["layer_hbm_frac"]), "layer_mfma_frac": r3(pt["layer_mfma_frac"]),
                     "kernel_us": r3(pt["roofline"]["kernel_us"]), "kernel_frac": r3(pt["roofline"]["frac"]),
                     "bound": pt["roofline"]["bound"]} for pt in sweep]
    print(json.dumps(out))
    return 0


if __name__ == "__main__":
    sys.exit(main())
