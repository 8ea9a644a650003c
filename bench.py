#!/usr/bin/env python3
"""Benchmark of the MI355X FP8 linear hot path.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload NAME] [--no-cpu]
    python bench.py --table          # every shape of the benchmark configurations -> bench_table.json in the results folder

A "step" is one pass of the hot path over one batch of synthetic input already resident
in HBM: dynamic activation quantisation (bf16 -> e4m3fn + f32 scales) followed by the
scaled FP8 matmul (bf16 out), or the grouped matmul for the MoE workload.  Inputs rotate
through enough copies to exceed twice the 256 MB Infinity Cache, so no step finds its
operands cached.  Prints ONE JSON line with the whole-step throughput, the roofline of
the dominant kernel (timed with events on the launch stream inside the timed region) and
the CPU oracle timed on this host's cores on a bounded slice of the same workload.  The
default run times the block-scaled GEMM the MFMA target is quoted on and adds a "decode"
record (same fields) for the HBM half of the metric; --workload NAME prints that workload alone.
"""
from __future__ import annotations

import argparse
import json
import math
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

METRIC = "FP8 GEMM TFLOPS & % of MI355X FP8 peak; decode-M HBM GB/s & % of peak"
PEAK_FP8_TFLOPS = 5000.0   # MI355X dense FP8 MFMA
PEAK_HBM_GBS = 8000.0      # MI355X HBM3E
CACHE_BUST_BYTES = 2 * 256 * 2 ** 20

# name -> (kind, M, K, N, model label)
WORKLOADS = {
    # configs[1]: Llama-3.1-8B-shaped blockwise FP8 linears (default: the largest, gate_up at M=2048)
    "llama8b_gate_up_m2048": ("block", 2048, 4096, 28672),
    "llama8b_qkv_m2048": ("block", 2048, 4096, 6144),
    "llama8b_down_m2048": ("block", 2048, 14336, 4096),
    "llama8b_o_proj_m2048": ("block", 2048, 4096, 4096),
    "llama8b_gate_up_m128": ("block", 128, 4096, 28672),
    "llama8b_gate_up_m16": ("block", 16, 4096, 28672),
    "llama8b_gate_up_m1": ("block", 1, 4096, 28672),
    # configs[0]
    "single_linear_m64": ("block", 64, 4096, 4096),
    # configs[2]: DeepSeek-V3 attention projections
    "dsv3_q_a_m4096": ("block", 4096, 7168, 1536),
    "dsv3_q_b_m4096": ("block", 4096, 1536, 24576),
    "dsv3_kv_a_m4096": ("block", 4096, 7168, 576),
    "dsv3_kv_b_m4096": ("block", 4096, 512, 32768),
    "dsv3_o_proj_m4096": ("block", 4096, 16384, 7168),
    "dsv3_o_proj_m1024": ("block", 1024, 16384, 7168),
    "dsv3_o_proj_m256": ("block", 256, 16384, 7168),
    # configs[3]: Llama-3.1-70B decode, per-token x per-channel scales
    "decode70b_qkv_m1": ("row", 1, 8192, 10240),
    "decode70b_qkv_m8": ("row", 8, 8192, 10240),
    "decode70b_gate_up_m1": ("row", 1, 8192, 57344),
    "decode70b_gate_up_m8": ("row", 8, 8192, 57344),
    "decode70b_down_m1": ("row", 1, 28672, 8192),
    "decode70b_down_m8": ("row", 8, 28672, 8192),
    # configs[4]: DeepSeek-V3 MoE grouped GEMM, 256 experts, 32768 routed rows
    "moe_gate_up": ("grouped", 32768, 7168, 4096),
    "moe_down": ("grouped", 32768, 2048, 7168),
    # the step before a per-token FP8 linear: RMSNorm fused with the dynamic quantisation (N unused)
    "rmsnorm_quant_m4096_k7168": ("rmsq", 4096, 7168, 0),
    "rmsnorm_quant_m32768_k7168": ("rmsq", 32768, 7168, 0),
}
# The two halves of the metric, each on the shape its target is quoted on: the block-scaled GEMM at M >= 2048 on a
# DeepSeek-V3 projection (configs[2]; the headline line) and an M <= 8 decode matmul of configs[3] (the "decode"
# record of the same line).
DEFAULT = "dsv3_o_proj_m4096"
DEFAULT_DECODE = "decode70b_gate_up_m8"


def measured_traffic(name):
    """HBM bytes per launch of the workload's matmul kernel, measured with rocprofv3 --pmc
    FETCH_SIZE / WRITE_SIZE (profiles/hbm_traffic_pmc.txt); None when it was not measured."""
    try:
        for line in open(os.path.join(ROOT, "profiles", "hbm_traffic_pmc.txt")):
            parts = line.split()
            if len(parts) == 3 and parts[0] == "traffic" and parts[1] == name:
                return int(parts[2])
    except OSError:
        pass
    return None


def measured_ceiling(plan, kind):
    """The issue ceiling of the dense kernel that `plan` launches (the library's own description of the launches), from
    the committed run of `bench.py --mfma-ceiling` (profiles/mfma_issue_ceiling.txt): the rate of the kernel's main loop
    on operands that never leave the chip -- the MFMA loop alone (row scaling) or with its promotions (block scaling),
    fragments from LDS; and the whole loop with its copies, waits and barriers, operands in L2.  None where the
    workload's kernel has no such probe (decode, grouped, the per-tile kernels) or the file is missing."""
    first = plan.split(" + ")[0]
    if "four waves" in first:
        label = "four waves, %s x 256 tiles" % first.split("x")[0]
    elif first.startswith("256x256") and "persistent" in first:
        label = "eight waves, 256 x 256 tiles"
    else:
        return None
    found = {}
    try:
        for line in open(os.path.join(ROOT, "profiles", "mfma_issue_ceiling.txt")):
            parts = [x.strip() for x in line.split("|")]
            if len(parts) >= 8 and parts[0] == "ceiling" and parts[1].startswith(label) and parts[2] == kind:
                found["mfma_loop" if parts[3].startswith("MFMA loop") else "whole_loop"] = float(parts[5])
    except OSError:
        return None
    if len(found) != 2:
        return None
    return {"kernel": label, "mfma_loop_lds_resident": found["mfma_loop"], "whole_loop_l2_resident": found["whole_loop"],
            "unit": "TFLOP/s",
            "source": "profiles/mfma_issue_ceiling.txt: bench.py --mfma-ceiling (maxfp8_mfma_issue_probe: the kernel's own "
                      "main loop, one block per CU, operands that never leave the chip); committed figures, not values of this run"}


def algorithmic(kind, M, K, N):
    """(flops, HBM bytes) of one step's matmul, and bytes of the quantisation."""
    flops = 2.0 * M * N * K
    if kind == "row":
        mm_bytes = N * K + 4 * N + M * K + 4 * M + 2 * M * N
        q_bytes = 3 * M * K + 4 * M
    else:
        mm_bytes = N * K + 4 * math.ceil(N / 128) * (K // 128) + M * K + 4 * M * (K // 128) + 2 * M * N
        q_bytes = 3 * M * K + 4 * M * (K // 128)
    return flops, mm_bytes, q_bytes


class Workload:
    def __init__(self, name, dev):
        import torch
        import modular_amd as mx
        from modular_amd import synth

        self.name = name
        self.kind, self.M, self.K, self.N = WORKLOADS[name]
        self.dev = dev
        self.mx = mx
        kind, M, K, N = self.kind, self.M, self.K, self.N
        self.cfg = mx.rowwise_fp8_config() if kind in ("row", "rmsq") else mx.blockwise_fp8_config()
        if kind == "rmsq":
            self.copies = max(2, min(8, math.ceil(CACHE_BUST_BYTES / (3 * M * K)) + 1))
            self.x = [synth.activations(M, K, seed=c, outlier_frac=0.01, device=dev) for c in range(self.copies)]
            g = torch.Generator(device="cpu").manual_seed(7)
            self.gamma = (1.0 + 0.1 * torch.randn(K, generator=g)).to(torch.bfloat16).to(dev)
            self.w, self.ws = [None] * self.copies, [None] * self.copies
            torch.cuda.synchronize()
            return
        E = 256 if kind == "grouped" else 1
        w_bytes = E * N * K
        per_copy = w_bytes + 2 * M * K + 2 * M * N
        self.copies = max(2, min(8, math.ceil(CACHE_BUST_BYTES / per_copy) + 1))
        if kind == "grouped":
            self.copies = 2 if w_bytes > 2 ** 32 else 3
        self.x, self.w, self.ws = [], [], []
        for c in range(self.copies):
            self.x.append(synth.activations(M, K, seed=c, outlier_frac=0.0 if kind == "row" else 0.01, device=dev))
            if kind == "row":
                wq, ws = synth.quantize_weight_rowwise(synth.weights_f32(N, K, seed=100 + c, device=dev))
            elif kind == "block":
                wq, ws = synth.quantize_weight_block(synth.weights_f32(N, K, seed=100 + c, device=dev))
            else:
                wq = torch.empty((E, N, K), dtype=torch.float8_e4m3fn, device=dev)
                ws = torch.empty((E, math.ceil(N / 128), K // 128), dtype=torch.float32, device=dev)
                for e0 in range(0, E, 16):
                    q16, s16 = synth.quantize_weight_block(
                        synth.weights_f32(16 * N, K, seed=1000 * c + e0, device=dev).reshape(16, N, K))
                    wq[e0:e0 + 16], ws[e0:e0 + 16] = q16, s16
            self.w.append(wq)
            self.ws.append(ws)
        if kind == "grouped":
            self.off, self.ids, self.counts, self.stats = synth.moe_routing(4096, 256, 8, seed=0, device=dev)
            assert int(self.counts.sum()) == M
        torch.cuda.synchronize()

    def quantise(self, c):
        import torch
        if self.kind == "rmsq":
            return (None, None)
        return self.mx.quantize_dynamic_scaled_float8(self.x[c], self.cfg.input_scale, self.cfg.weight_scale,
                                                      scales_type=torch.float32)

    def matmul(self, c, q, sa):
        """the workload's dominant kernel (the fused norm + quantise itself for the rmsq kind)"""
        mx, cfg = self.mx, self.cfg
        if self.kind == "rmsq":
            return mx.rms_norm_fused_quantize_dynamic_scaled_fp8(self.x[c], self.gamma, 1e-6)
        if self.kind == "grouped":
            return mx.grouped_dynamic_scaled_fp8_matmul(q, self.w[c], sa, self.ws[c], self.off, self.ids, self.stats,
                                                        cfg.input_scale, cfg.weight_scale)
        return mx.dynamic_scaled_matmul(q, self.w[c], sa, self.ws[c], cfg.input_scale, cfg.weight_scale)

    def step(self, i):
        """one pass of the hot path: quantise + matmul on input copy i"""
        c = i % self.copies
        q, sa = self.quantise(c)
        return self.matmul(c, q, sa)


RESULTS_DIR = "gpurun_out"
SETTLE_S = 0.5  # the workload runs this long, untimed, before the warm-up steps (see run_gpu)


def run_gpu(name, steps, warmup, settle_s=None):
    """Before anything is timed the workload runs for `settle_s` seconds: an idle MI355X starts at
    low clocks and takes some tenths of a second of sustained load to reach the clocks it then
    holds (the same 30 steps measure 10-15 % slower straight after start-up than after half a
    second of load); a serving process lives in the settled state.  Then `warmup` untimed steps.

    Times `steps` passes of the hot path with the host clock (whole-step throughput), then
    the matmul launches of the same passes with HIP events on the launch stream: once with a
    pair of events per launch (median, minimum) and once with one pair around all launches
    (average).  Both passes queue their launches behind untimed launches of the same matmul."""
    import torch

    dev = torch.device("cuda:0")
    wl = Workload(name, dev)
    settle_s = SETTLE_S if settle_s is None else settle_s
    t_end, i = time.perf_counter() + settle_s, 0
    while time.perf_counter() < t_end:
        for _ in range(16):
            wl.step(i)
            i += 1
        torch.cuda.synchronize()
    for i in range(warmup):
        wl.step(i)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for i in range(steps):
        wl.step(warmup + i)
    torch.cuda.synchronize()
    t1 = time.perf_counter()
    ms_step = (t1 - t0) * 1e3 / steps

    quantised = [wl.quantise(c) for c in range(wl.copies)]
    events = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(steps)]
    # Runway: untimed launches of the same matmul in front of the timed ones.  While the GPU works through
    # them the host queues the timed launches, so the intervals hold kernels and not launch latency, and the
    # GPU stays under the load (and at the clocks) of the timed region above.
    runway = min(2000, 20 + int(steps * 0.012 / max(ms_step, 1e-3)))

    def launch(i):
        c = (warmup + i) % wl.copies
        wl.matmul(c, *quantised[c])

    torch.cuda.synchronize()
    for i in range(runway):
        launch(i)
    for i in range(steps):
        events[i][0].record()
        launch(i)
        events[i][1].record()
    torch.cuda.synchronize()
    mm_ms = sorted(e[0].elapsed_time(e[1]) for e in events)
    # The average comes from one pair of events around all `steps` launches: an event pair around a single
    # launch also holds the few microseconds the command processor needs between the event and the
    # dispatch, which back-to-back launches overlap.
    first, last = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    for i in range(runway):
        launch(i)
    first.record()
    for i in range(steps):
        launch(i)
    last.record()
    torch.cuda.synchronize()
    mm_avg = first.elapsed_time(last) / steps
    return wl, ms_step, mm_avg, mm_ms[len(mm_ms) // 2], mm_ms[0]


def config_cells():
    """Every cell of BASELINE.json's configs[1..3]: name -> (kind, M, K, N)."""
    cells = {}
    for proj, (K, N) in (("qkv", (4096, 6144)), ("o_proj", (4096, 4096)), ("gate_up", (4096, 28672)), ("down", (14336, 4096))):
        for M in (1, 16, 128, 2048):
            cells[f"llama8b_{proj}_m{M}"] = ("block", M, K, N)
    # (q_a_kv_a: the one matmul over the stacked q_a and kv_a weights that the reference's FP8 MLA issues, N = 1536 + 576)
    for proj, (K, N) in (("q_a", (7168, 1536)), ("q_b", (1536, 24576)), ("kv_a", (7168, 576)), ("kv_b", (512, 32768)),
                         ("o_proj", (16384, 7168)), ("q_a_kv_a", (7168, 2112))):
        for M in (256, 1024, 4096):
            cells[f"dsv3_{proj}_m{M}"] = ("block", M, K, N)
    for proj, (K, N) in (("qkv", (8192, 10240)), ("gate_up", (8192, 57344)), ("down", (28672, 8192))):
        for M in (1, 2, 4, 8):
            cells[f"decode70b_{proj}_m{M}"] = ("row", M, K, N)
    return cells


def graph_time_ms(wl, launches):
    """Milliseconds per matmul when `launches` of them (rotating over the operand copies) replay from one HIP graph:
    the launch-to-launch interval on the GPU with no host in between, which is what a kernel of a few microseconds
    needs to be timed at all (a call through the Python wrappers takes longer than such a kernel runs)."""
    import torch

    quantised = [wl.quantise(c) for c in range(wl.copies)]
    side = torch.cuda.Stream()
    graph = torch.cuda.CUDAGraph()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        for i in range(3):
            wl.matmul(i % wl.copies, *quantised[i % wl.copies])
        side.synchronize()
        with torch.cuda.graph(graph, stream=side):
            for i in range(launches):
                wl.matmul(i % wl.copies, *quantised[i % wl.copies])
    torch.cuda.current_stream().wait_stream(side)
    t_end = time.perf_counter() + SETTLE_S
    while time.perf_counter() < t_end:
        graph.replay()
        torch.cuda.synchronize()
    first, last = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    times = []
    for _ in range(5):
        first.record()
        graph.replay()
        last.record()
        torch.cuda.synchronize()
        times.append(first.elapsed_time(last) / launches)
    return sorted(times)[len(times) // 2]


def moe_layer_ms(steps, fuse):
    """Milliseconds per call (host clock around `steps` calls, clocks settled) of the expert matmuls of a block-scaled FP8
    MoE layer on BASELINE's configs[4] routing: 4096 tokens, top-8 of 256 experts (popularity ~ rank^-1.1), hidden 7168,
    intermediate 2048 -- grouping, gathered quantise, grouped gate_up, silu(gate) * up, quantise, grouped down."""
    import torch
    import modular_amd as mx
    from modular_amd import synth

    dev = torch.device("cuda:0")
    cfg = mx.blockwise_fp8_config()
    seq, k, E, hidden, inter = 4096, 8, 256, 7168, 2048
    x = synth.activations(seq, hidden, seed=1, device=dev)
    g = torch.Generator().manual_seed(0)
    perm = torch.randperm(E, generator=g)
    rank = torch.empty(E)
    rank[perm] = torch.arange(1, E + 1, dtype=torch.float32)
    logits = torch.randn((seq, E), generator=g) - 1.1 * torch.log(rank)
    router_idx = torch.topk(torch.softmax(logits, dim=-1), k, dim=-1).indices.to(torch.int32).to(dev)
    wgu = synth.random_fp8((E, 2 * inter, hidden), 2, device=dev)
    sgu = synth.random_scales((E, 2 * inter // 128, hidden // 128), 3, device=dev, lo=0.001, hi=0.01)
    wd = synth.random_fp8((E, hidden, inter), 4, device=dev)
    sd = synth.random_scales((E, hidden // 128, inter // 128), 5, device=dev, lo=0.001, hi=0.01)

    def run():
        return mx.expert_matmuls_fp8(x, router_idx, wgu, sgu, wd, sd, cfg, host_sync=False, fuse_activation_quant=fuse)

    t_end = time.perf_counter() + max(SETTLE_S, 0.5)
    while time.perf_counter() < t_end:
        run()
        torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps):
        run()
    torch.cuda.synchronize()
    return (time.perf_counter() - t0) * 1e3 / steps


def moe_routings(steps):
    """The grouped block-scaled matmul (DeepSeek-V3's two MoE shapes, 256 experts, top-8) over several routings -- the
    skew of the experts' popularity and the number of tokens -- in both of its forms: the four-wave launch beside the
    persistent one (the default) and one persistent launch (MAXFP8_GROUPED_W4=0), interleaved in one process.  Yields one
    record per (shape, routing): microseconds per matmul from a pair of HIP events around `steps` launches, after 0.3 s
    of the same launches."""
    import torch
    import modular_amd as mx
    from modular_amd import _lib, synth

    dev = torch.device("cuda:0")
    cfg = mx.blockwise_fp8_config()
    E = 256

    def form(two_launches):
        if two_launches:
            os.environ.pop("MAXFP8_GROUPED_W4", None)
        else:
            os.environ["MAXFP8_GROUPED_W4"] = "0"
        _lib.tuning_reload()

    def timed(fn):
        t_end = time.perf_counter() + 0.3
        while time.perf_counter() < t_end:
            fn()
            torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(steps):
            fn()
        e1.record()
        torch.cuda.synchronize()
        return e0.elapsed_time(e1) / steps * 1e3

    before = os.environ.get("MAXFP8_GROUPED_W4")
    try:
        for proj, N, K in (("gate_up", 4096, 7168), ("down", 7168, 2048)):
            w = synth.random_fp8((E, N, K), 1, device=dev)
            ws = synth.random_scales((E, N // 128, K // 128), 2, device=dev, lo=0.001, hi=0.01)
            for tokens, zipf in ((4096, 1.1), (4096, 0.0), (4096, 0.5), (4096, 2.0), (1024, 1.1), (512, 1.1), (16384, 1.1), (8192, 0.0)):
                off, ids, counts, stats = synth.moe_routing(tokens, E, 8, seed=0, zipf_a=zipf, device=dev)
                T = int(counts.sum())
                a = synth.random_fp8((T, K), 3, device=dev)
                sa = synth.random_scales((K // 128, T), 4, device=dev, lo=0.01, hi=0.1)

                def fn():
                    return mx.grouped_dynamic_scaled_fp8_matmul(a, w, sa, ws, off, ids, stats, cfg.input_scale, cfg.weight_scale)

                us = {}
                for rep in range(2):  # (interleaved: one launch, two launches, and again; the second pair is reported)
                    for two in (False, True):
                        form(two)
                        us[two] = timed(fn)
                c = counts.tolist()
                yield {"projection": proj, "N": N, "K": K, "tokens": tokens, "zipf": zipf, "rows": T, "active_experts": sum(x > 0 for x in c),
                       "largest_expert": max(c), "experts_with_192_rows_or_more": sum(x >= 192 for x in c),
                       "one_launch_us": round(us[False], 1), "two_launches_us": round(us[True], 1),
                       "two_over_one": round(us[True] / us[False], 3)}
                del a, sa
                torch.cuda.empty_cache()
            del w, ws
            torch.cuda.empty_cache()
    finally:
        if before is None:
            os.environ.pop("MAXFP8_GROUPED_W4", None)
        else:
            os.environ["MAXFP8_GROUPED_W4"] = before
        _lib.tuning_reload()


def read_ceiling(wl, steps):
    """Average time of the decode matmul's read-only probe (the same grid, LDS ring and DMA instructions streaming
    the same weight copies, nothing else) over `steps` back-to-back launches, in milliseconds."""
    import torch
    from modular_amd import _lib

    L, stream = _lib.lib(), torch.cuda.current_stream().cuda_stream

    def launch(i):
        w = wl.w[i % wl.copies]
        _lib.check(L.maxfp8_decode_weight_read_probe(w.data_ptr(), wl.M, wl.N, wl.K, w.stride(0), stream))

    first, last = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    t_end, i = time.perf_counter() + 0.3, 0
    while time.perf_counter() < t_end:
        for _ in range(64):
            launch(i)
            i += 1
        torch.cuda.synchronize()
    for i in range(200):
        launch(i)
    first.record()
    for i in range(steps):
        launch(i)
    last.record()
    torch.cuda.synchronize()
    return first.elapsed_time(last) / steps


MFMA_CEILING_KERNELS = {0: ("eight waves, 256 x 256 tiles (gemm_persist_kernel)", 256),
                        4: ("four waves, 128 x 256 tiles (gemm_w4_kernel)", 128),
                        5: ("four waves, 160 x 256 tiles (gemm_w4_kernel)", 160),
                        6: ("four waves, 192 x 256 tiles (gemm_w4_kernel)", 192)}


def mfma_ceiling(slabs=4096, reps=20, settle_s=0.5):
    """The main loops of the dense kernels on operands that never leave the chip (maxfp8_mfma_issue_probe): one block per
    CU runs `slabs` K slabs of one tile -- level 2: the MFMA loop alone, fragments read from LDS (row scaling: MFMA only;
    block scaling: with the per-slab promotions); level 1: with the LDS-DMA copies, waits and barriers, operands in L2.
    Yields one record per (kernel, scaling, level): microseconds per slab and the rate over all CUs."""
    import torch
    from modular_amd import _lib, synth

    dev = torch.device("cuda:0")
    L, stream = _lib.lib(), torch.cuda.current_stream().cuda_stream
    # operands like the workloads': quantised normal data (no NaN bytes), scales of the usual size
    a = synth.random_fp8((256, 1024), 1, std=150.0).to(dev)
    b = synth.random_fp8((256, 1024), 2, std=150.0).to(dev)
    a_s = synth.random_scales((8, 256), 3).to(dev)
    b_s = synth.random_scales((2, 8), 4).to(dev)
    c = torch.empty((256, 256), dtype=torch.bfloat16, device=dev)
    cus = torch.cuda.get_device_properties(0).multi_processor_count
    clocks = torch.zeros((cus, 2), dtype=torch.int64, device=dev)
    first, last = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    for kernel, (label, rows) in MFMA_CEILING_KERNELS.items():
        for block in (0, 1):
            for level in (2, 1):
                def launch(n):
                    _lib.check(L.maxfp8_mfma_issue_probe(kernel, block, level, n, a.data_ptr(), b.data_ptr(), a_s.data_ptr(),
                                                         b_s.data_ptr(), c.data_ptr(), clocks.data_ptr(), stream))
                t_end = time.perf_counter() + settle_s   # the clocks of an idle GPU take tenths of a second to settle
                while time.perf_counter() < t_end:
                    launch(slabs)
                    torch.cuda.synchronize()
                first.record()
                for _ in range(reps):
                    launch(slabs)
                last.record()
                torch.cuda.synchronize()
                us_slab = first.elapsed_time(last) * 1e3 / reps / slabs
                flops_slab = 2.0 * rows * 256 * 128 * cus
                # the last launch's counters: core-clock cycles over 100 MHz ticks = the clock held in the slab loop;
                # an MFMA of this shape occupies its SIMD's matrix pipe for 32 cycles
                cyc, ticks = clocks[:, 0].double().mean().item(), clocks[:, 1].double().mean().item()
                ghz = cyc / ticks * 0.1
                busy = (rows // 4) * 32.0 * slabs / cyc   # rows / 4 MFMAs per SIMD and slab
                yield {"kernel": label, "scaling": "block" if block else "row",
                       "level": "MFMA loop on LDS-resident operands" + (" + promotions" if block else "") if level == 2 else
                                "whole loop (copies, waits, barriers), operands in L2",
                       "us_per_slab": round(us_slab, 4), "TFLOP/s": round(flops_slab / us_slab / 1e6, 1),
                       "frac_of_peak": round(flops_slab / us_slab / 1e6 / PEAK_FP8_TFLOPS, 3),
                       "core_clock_GHz": round(ghz, 3), "matrix_pipe_busy": round(busy, 3), "slabs": slabs, "launches": reps,
                       "blocks": cus}


VENDOR_CELLS = [(4096, 7168, 16384), (8192, 8192, 8192), (2048, 28672, 4096), (2048, 6144, 4096), (4096, 24576, 1536),
                (256, 2304, 16384), (16, 2304, 16384), (64, 28672, 4096), (128, 8192, 28672), (8, 57344, 8192)]


def vendor_compare(steps=30):
    """Per-token x per-channel scaled FP8 matmuls (the one scaling form the vendor library has) through this library and
    through hipBLASLt (reached by torch._scaled_mm) on the same operands, weights rotating through enough copies to come
    from HBM.  Yields one record per (M, N, K): microseconds each, and the largest difference of the two bf16 results in
    bf16 steps of the larger value."""
    import torch
    from modular_amd import kernels as mx, synth
    from modular_amd.quant_config import InputScaleSpec, ScaleGranularity, ScaleOrigin, WeightScaleSpec

    dev = torch.device("cuda:0")
    in_spec = InputScaleSpec(granularity=ScaleGranularity.COLWISE, origin=ScaleOrigin.DYNAMIC, dtype=torch.float32)
    w_spec = WeightScaleSpec(granularity=ScaleGranularity.ROWWISE, dtype=torch.float32)

    def timed(fn):
        t_end = time.perf_counter() + 0.3
        i = 0
        while time.perf_counter() < t_end:
            fn(i)
            i += 1
            torch.cuda.synchronize()
        first, last = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        for i in range(5):
            fn(i)
        first.record()
        for i in range(steps):
            fn(i)
        last.record()
        torch.cuda.synchronize()
        return first.elapsed_time(last) * 1e3 / steps

    for (M, N, K) in VENDOR_CELLS:
        copies = max(2, int(CACHE_BUST_BYTES // (N * K)) + 1)
        a = synth.random_fp8((M, K), 1, device=dev)
        ws = [synth.random_fp8((N, K), 2 + i, device=dev) for i in range(copies)]
        sa = synth.random_scales((1, M), 3, device=dev, lo=0.01, hi=0.1)
        sb = synth.random_scales((N, 1), 4, device=dev, lo=0.001, hi=0.01)
        sa_col = sa.t().contiguous()  # [M, 1], the vendor call's layout
        sb_row = sb.t().contiguous()  # [1, N]
        ours = lambda i: mx.dynamic_scaled_matmul(a, ws[i % copies], sa, sb, in_spec, w_spec, out_type=torch.bfloat16)
        theirs = lambda i: torch._scaled_mm(a, ws[i % copies].t(), scale_a=sa_col, scale_b=sb_row, out_dtype=torch.bfloat16)
        rec = {"M": M, "N": N, "K": K, "scaling": "per-token x per-channel", "weight_copies": copies}
        try:
            c_v = theirs(0)
        except Exception as e:  # a shape the vendor path does not take
            rec["vendor_error"] = str(e)[:200]
            c_v = None
        c_o = ours(0)
        torch.cuda.synchronize()
        rec["ours_us"] = round(timed(ours), 2)
        if c_v is not None:
            rec["vendor_us"] = round(timed(theirs), 2)
            rec["vendor_over_ours"] = round(rec["vendor_us"] / rec["ours_us"], 3)
            big = torch.maximum(c_o.float().abs(), c_v.float().abs()).clamp_min(1e-30)
            step = torch.exp2(torch.floor(torch.log2(big)) - 7)
            rec["max_diff_bf16_steps"] = round(float(((c_o.float() - c_v.float()).abs() / step).max()), 2)
        rec["TFLOP/s_ours"] = round(2.0 * M * N * K / rec["ours_us"] / 1e6, 1)
        yield rec
        del ws
        torch.cuda.empty_cache()


def cpu_baseline(wl, budget_s=15.0):
    """The oracle (a port of the reference's host loops) on this host's cores, on a bounded
    slice of the same workload; throughput in the metric's unit."""
    import numpy as np
    import oracle

    threads = oracle.default_threads()
    kind, M, K, N = wl.kind, wl.M, wl.K, wl.N
    x = wl.x[0].cpu()
    if kind == "rmsq":
        import torch
        rows = min(M, 4096)
        xb = x[:rows].contiguous().view(torch.int16).numpy().view(np.uint16)
        gb = wl.gamma.cpu().view(torch.int16).numpy().view(np.uint16)
        t0 = time.perf_counter()
        reps = 0
        while time.perf_counter() - t0 < budget_s / 3 or reps == 0:
            oracle.rms_norm_fused_quantize(xb, gb, 1e-6, threads=threads)
            reps += 1
        t = (time.perf_counter() - t0) / reps
        return {"value": 3.0 * rows * K / t / 1e9, "unit": "GB/s", "cores": threads, "kind": "port",
                "sample": f"oracle rms_norm_fused_quantize on rows 0..{rows - 1} of M={M}, K={K}: {t:.3f} s per pass, {reps} passes"}
    w = wl.w[0] if kind != "grouped" else wl.w[0][0]
    ws = wl.ws[0] if kind != "grouped" else wl.ws[0][0]
    wb = w.cpu().view(__import__("torch").uint8).numpy()
    wsn = ws.cpu().numpy()
    G = K if kind == "row" else 128

    def run(rows):
        xb = x[:rows].contiguous().view(__import__("torch").int16).numpy().view(np.uint16)
        t0 = time.perf_counter()
        q, sa = oracle.quantize_dynamic_scaled_fp8(xb, G, threads=threads)
        if kind == "row":
            oracle.matmul_rowwise(q, wb, sa, wsn, c_dtype=oracle.BF16, threads=threads)
        else:
            oracle.matmul_blockwise(q, wb, sa, wsn, c_dtype=oracle.BF16, mode=1, threads=threads)
        return time.perf_counter() - t0

    rows = min(M, max(1, threads))
    t = run(rows)
    per_row = t / rows
    rows2 = int(min(M, max(rows, budget_s / max(per_row, 1e-9))))
    if rows2 > rows:
        t, rows = run(rows2), rows2
    flops = 2.0 * rows * N * K
    if kind == "row":
        value, unit = (N * K + rows * K + 2 * rows * N) / t / 1e9, "GB/s"
    else:
        value, unit = flops / t / 1e12, "TFLOP/s"
    order = "one f32 dot product per row pair, scales applied once" if kind == "row" else \
        "oracle mode 1: one f32 partial sum per 128-wide K group, then acc += partial * (a_s * b_s) -- the order a tiled kernel uses, not the reference's element order (mode 0)"
    sample = (f"oracle quantise + matmul ({order}) on rows 0..{rows - 1} of M={M}"
              + (" against expert 0's weights" if kind == "grouped" else "")
              + f", N={N}, K={K}: {t:.2f} s")
    return {"value": value, "unit": unit, "cores": threads, "kind": "port", "sample": sample}


def kernels_launched(kind, M, K, N):
    """(name of the dominant kernel, description of every launch of the matmul), from the plan the library itself
    reports for the shape (maxfp8_matmul_describe)."""
    if kind == "rmsq":
        return "rmsnorm_quant_row_bf16_kernel", "one launch"
    if kind == "grouped":
        if os.environ.get("MAXFP8_GROUPED_PERSIST", "1") == "0":
            return "gemm_grouped_kernel", ("gemm_grouped_large_kernel (full 256-row tiles of experts with >= 1024 rows) + "
                                           "gemm_grouped_kernel (the rest), side by side on two streams")
        if os.environ.get("MAXFP8_GROUPED_W4", "1") != "0":
            return "gemm_w4_grouped_kernel", ("gemm_w4_grouped_kernel (four waves, 192 x 256 tiles: every slot's full 192 rows, a rest of more "
                                              "than 32 rows behind them, and slots of 129-191 rows) on the caller's stream + "
                                              "gemm_grouped_persist_kernel (the other rows: 128 x 256 tiles, weight-streaming rings for at most "
                                              "32 rows) on a second stream, side by side; the blocks of the first launch past its share "
                                              "of the chip, which they work out from the group sizes, exit at once")
        return "gemm_grouped_persist_kernel", ("one persistent launch, a block per CU: 256 x 256 tiles of every full 256 rows, "
                                               "256 x 128 / 128 x 256 tiles of the rests, weight-streaming rings for rests of at "
                                               "most 32 rows; the CUs are shared out between the matrix-bound and the streaming tiles")
    from modular_amd import _lib
    plan = _lib.matmul_describe(M, N, K, kind == "block", True)
    first = plan.split(" + ")[0]
    if plan.startswith("skinny"):
        return "gemm_skinny_kernel", plan
    if "four waves" in first:
        return "gemm_w4_kernel", plan
    if "persistent" in first:
        return "gemm_persist_kernel", plan
    if "stream-K" in first:
        return "gemm_streamk_kernel", plan
    return "gemm_tiled_kernel", plan


def result_line(name, steps, warmup, with_cpu=True):
    wl, ms_step, mm_avg, mm_med, mm_min = run_gpu(name, steps, warmup)
    kind, M, K, N = wl.kind, wl.M, wl.K, wl.N
    flops, mm_bytes, q_bytes = algorithmic(kind, M, K, N)
    if kind == "rmsq":
        flops, mm_bytes, q_bytes = 0.0, 3 * M * K + 2 * K + 4 * M, 0
    if kind == "grouped":
        # weights of every expert that received tokens are streamed once (experts without tokens are never read)
        active = int((wl.counts > 0).sum())
        mm_bytes += (active - 1) * N * K + 4 * (active - 1) * math.ceil(N / 128) * (K // 128)
    # the roof that binds at the published peaks: a matmul is HBM-bound when moving its bytes at 8 TB/s takes longer
    # than its flops at 5 PFLOP/s (under ~625 flops per byte: every decode shape, and prefill shapes up to M ~ 256)
    hbm_bound = kind in ("row", "rmsq") or mm_bytes / (PEAK_HBM_GBS * 1e9) > flops / (PEAK_FP8_TFLOPS * 1e12)
    if hbm_bound:
        value, unit = (mm_bytes + q_bytes) / (ms_step * 1e-3) / 1e9, "GB/s"
        roof = {"bound": "hbm", "achieved": mm_bytes / (mm_avg * 1e-3) / 1e9, "peak": PEAK_HBM_GBS, "unit": "GB/s"}
    else:
        value, unit = flops / (ms_step * 1e-3) / 1e12, "TFLOP/s"
        roof = {"bound": "mfma", "achieved": flops / (mm_avg * 1e-3) / 1e12, "peak": PEAK_FP8_TFLOPS, "unit": "TFLOP/s"}
    roof["frac"] = roof["achieved"] / roof["peak"]
    if kind == "grouped":
        # the grouped matmul is priced against both roofs: 2 * T * N * K flops of real rows, and the weights of the
        # experts in use streamed once
        roof["frac_mfma"] = flops / (mm_avg * 1e-3) / 1e12 / PEAK_FP8_TFLOPS
        roof["frac_hbm"] = mm_bytes / (mm_avg * 1e-3) / 1e9 / PEAK_HBM_GBS
    roof["traffic"] = measured_traffic(name)
    roof["traffic_source"] = ("profiles/hbm_traffic_pmc.txt: rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE runs of this command, "
                              "scaled by the copy kernel; a committed figure, not a value of this run")
    roof["algorithmic_bytes"] = mm_bytes
    # the matmul can be more than one launch (two regions in different tile shapes; the grouped matmul's
    # large-tile launch and the rest): kernel_ms_* is the time of all of them
    roof["kernel"], roof["launches"] = kernels_launched(kind, M, K, N)
    roof["kernel_ms_avg"], roof["kernel_ms_median"], roof["kernel_ms_min"] = mm_avg, mm_med, mm_min
    if roof["bound"] == "mfma" and kind in ("block", "row"):
        ceiling = measured_ceiling(roof["launches"], kind)
        if ceiling is not None:
            ceiling["frac_of_whole_loop"] = roof["achieved"] / ceiling["whole_loop_l2_resident"]
            roof["ceiling"] = ceiling
    out = {
        "metric": METRIC, "value": value, "unit": unit, "n_gpus": 1, "steps": steps, "warmup": warmup,
        "ms_per_step": ms_step, "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "fp8_e4m3fn (f32 accumulate, bf16 out)", "data": "synthetic",
        "config": {"workload": name, "M": M, "K": K, "N": N,
                   "scaling": "per-token" if kind == "rmsq" else
                              "per-token x per-channel" if kind == "row" else "1x128 activations, 128x128 weights",
                   "step": "RMSNorm fused with dynamic quantise" if kind == "rmsq" else
                           "dynamic quantise + " + ("grouped " if kind == "grouped" else "") + "scaled matmul",
                   "input_copies": wl.copies, "settle_s": SETTLE_S,
                   "timing": "value: host clock around the steps (quantise + matmul); roofline: events around the matmul "
                             "launches alone in passes of their own -- the passes differ by a few per cent, so "
                             "ms_per_step is not kernel_ms_avg plus the quantiser"},
        "roofline": roof,
    }
    if with_cpu:
        out["cpu_baseline"] = cpu_baseline(wl)
    return out


def main():
    global SETTLE_S
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=100)
    ap.add_argument("--warmup", type=int, default=10)
    ap.add_argument("--workload", default=None, choices=sorted(WORKLOADS),
                    help=f"one workload alone (default: {DEFAULT}, with a 'decode' record for {DEFAULT_DECODE})")
    ap.add_argument("--settle", type=float, default=SETTLE_S,
                    help="seconds the workload runs, untimed, before the warm-up steps (clock ramp of an idle GPU)")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU oracle timing")
    ap.add_argument("--table", action="store_true", help="run every workload, write bench_table.json into the results folder")
    ap.add_argument("--calibrate", action="store_true",
                    help="also launch the plain copy kernel on 256 MiB three times (the known-size unit that "
                         "hardware byte counters of a rocprofv3 --pmc run are scaled by)")
    ap.add_argument("--cells", action="store_true",
                    help="every cell of configs[1..3] (each projection at each M): the matmul's time per launch when 100 "
                         "launches replay from one HIP graph, against the roof that binds it; one JSON line each")
    ap.add_argument("--moe-layer", action="store_true",
                    help="the expert matmuls of the FP8 MoE layer on configs[4]'s routing (grouping, gathered quantise, grouped "
                         "gate_up, silu * up, quantise, grouped down): milliseconds per call, one JSON line for each way of the "
                         "activation quantisation (two kernels, one kernel)")
    ap.add_argument("--moe-routings", action="store_true",
                    help="the grouped block-scaled matmul of DeepSeek-V3's two MoE shapes over several routings (skew, number of "
                         "tokens), as the four-wave launch beside the persistent one and as one persistent launch: one JSON line "
                         "per shape and routing")
    ap.add_argument("--mfma-ceiling", action="store_true",
                    help="the dense kernels' main loops on operands that stay on the chip (LDS-resident: MFMA loop alone and "
                         "with promotions; L2-resident: with copies and barriers), one JSON line each: the issue ceiling the "
                         "dense matmuls are measured against")
    ap.add_argument("--vendor", action="store_true",
                    help="per-token x per-channel scaled matmuls through this library and through hipBLASLt (torch._scaled_mm) "
                         "on the same operands, one JSON line per shape")
    ap.add_argument("--read-ceiling", action="store_true",
                    help="for every decode workload (M <= 16): the matmul kernel's time beside the time of its read-only "
                         "probe (same grid and weight traffic, no arithmetic), one JSON line each")
    args = ap.parse_args()
    SETTLE_S = max(0.0, args.settle)
    if args.gpus != 1:
        print("bench.py: this build measures one GPU only (the path has no collective); run with --gpus 1",
              file=sys.stderr)
        sys.exit(2)
    import torch

    if not torch.cuda.is_available():
        print("bench.py: no GPU visible; the HIP kernels are the only compute path", file=sys.stderr)
        sys.exit(1)
    if args.table:
        os.makedirs(os.path.join(ROOT, RESULTS_DIR), exist_ok=True)
        rows = []
        for name in WORKLOADS:
            print(f"[bench] {name}", file=sys.stderr, flush=True)
            r = result_line(name, args.steps, args.warmup, with_cpu=False)
            rows.append(r)
            print(json.dumps({"workload": name, "value": r["value"], "unit": r["unit"], "ms_per_step": r["ms_per_step"],
                              "kernel_ms": r["roofline"]["kernel_ms_avg"], "frac": r["roofline"]["frac"]}),
                  file=sys.stderr, flush=True)
            with open(os.path.join(ROOT, RESULTS_DIR, "bench_table.json"), "w") as f:
                json.dump(rows, f, indent=1)
            torch.cuda.empty_cache()
        return
    if args.cells:
        from modular_amd import _lib
        for name, cell in config_cells().items():
            WORKLOADS[name] = cell
            wl = Workload(name, torch.device("cuda:0"))
            ms = graph_time_ms(wl, 100)
            kind, M, K, N = cell
            flops, mm_bytes, _ = algorithmic(kind, M, K, N)
            hbm_bound = mm_bytes / (PEAK_HBM_GBS * 1e9) > flops / (PEAK_FP8_TFLOPS * 1e12)
            achieved = mm_bytes / (ms * 1e-3) / 1e9 if hbm_bound else flops / (ms * 1e-3) / 1e12
            print(json.dumps({"cell": name, "scaling": kind, "M": M, "K": K, "N": N, "us_per_launch": round(ms * 1e3, 2),
                              "bound": "hbm" if hbm_bound else "mfma", "achieved": round(achieved, 1),
                              "unit": "GB/s" if hbm_bound else "TFLOP/s",
                              "frac": round(achieved / (PEAK_HBM_GBS if hbm_bound else PEAK_FP8_TFLOPS), 3),
                              "launches": _lib.matmul_describe(M, N, K, kind == "block", True)}), flush=True)
            del wl
            torch.cuda.empty_cache()
        return
    if args.moe_layer:
        for fuse in (False, True):
            ms = moe_layer_ms(args.steps, fuse)
            print(json.dumps({"workload": "expert_matmuls_fp8: 4096 tokens x top-8 of 256 experts, hidden 7168, intermediate 2048",
                              "fuse_activation_quant": fuse, "ms_per_call": round(ms, 4), "steps": args.steps,
                              "timing": "host clock around the calls, no host synchronisation inside a call"}), flush=True)
            torch.cuda.empty_cache()
        return
    if args.moe_routings:
        for rec in moe_routings(min(args.steps, 30)):
            print(json.dumps(rec), flush=True)
        return
    if args.mfma_ceiling:
        for rec in mfma_ceiling():
            print(json.dumps(rec), flush=True)
        return
    if args.vendor:
        for rec in vendor_compare():
            print(json.dumps(rec), flush=True)
        return
    if args.read_ceiling:
        for name in ([args.workload] if args.workload else [n for n, w in WORKLOADS.items() if w[0] == "row" and w[1] <= 16]):
            wl, _, mm_avg, _, _ = run_gpu(name, max(args.steps, 200), args.warmup)
            probe = read_ceiling(wl, max(args.steps, 200))
            _, mm_bytes, _ = algorithmic(wl.kind, wl.M, wl.K, wl.N)
            print(json.dumps({"workload": name, "M": wl.M, "K": wl.K, "N": wl.N, "weight_bytes": wl.N * wl.K,
                              "matmul_us": round(mm_avg * 1e3, 2), "read_only_us": round(probe * 1e3, 2),
                              "matmul_over_read_only": round(mm_avg / probe, 3),
                              "matmul_GBps": round(mm_bytes / mm_avg / 1e6), "read_only_GBps": round(wl.N * wl.K / probe / 1e6)}),
                  flush=True)
            del wl
            torch.cuda.empty_cache()
        return
    if args.calibrate:
        from modular_amd import kernels
        src = torch.ones((256 << 20,), dtype=torch.uint8, device="cuda:0")
        dst = torch.empty_like(src)
        for _ in range(3):
            kernels.copy_bytes(dst, src)
        torch.cuda.synchronize()
    if args.workload is not None:
        print(json.dumps(result_line(args.workload, args.steps, args.warmup, with_cpu=not args.no_cpu)))
        return
    line = result_line(DEFAULT, args.steps, args.warmup, with_cpu=not args.no_cpu)
    torch.cuda.empty_cache()
    # the HBM half of the metric: same fields, its own timed region (more steps: a launch takes ~75 microseconds)
    dec = result_line(DEFAULT_DECODE, max(args.steps, 200), args.warmup, with_cpu=False)
    line["decode"] = {k: dec[k] for k in ("value", "unit", "steps", "warmup", "ms_per_step", "config", "roofline")}
    print(json.dumps(line))


if __name__ == "__main__":
    main()
