#!/usr/bin/env python3
"""Benchmark of the fused-MoE expert path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload NAME]

A step is one call of the whole layer path (router softmax/top-k, alignment,
gate-up GEMM + SiLU*up, down GEMM * routed weight, top-k combine) on the
Qwen3-30B-A3B-shaped layer (H 2048, 128 experts, I 768, top-8) with synthetic
seeded inputs already resident in HBM.  The headline workload is the
layered-prefill iteration: 8192 prefill + 256 decode tokens in one call.  The
decode-only 256-token call (memory-bound) is measured in the same run and
reported under "decode".  One JSON line goes to stdout.
"""
from __future__ import annotations

import argparse
import importlib
import json
import os
import statistics
import sys
import time

import torch

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

METRIC = "MoE layer TFLOP/s @8192+256 tok & decode HBM GB/s, Qwen3-30B-A3B layer"
PEAK_BF16_TFLOPS = 2500.0   # MI355X dense bf16 MFMA
PEAK_HBM_GBS = 8000.0       # MI355X HBM3E

TRAFFIC_JSON = os.path.join(ROOT, "profiles", "hbm_traffic_grouped_gemm_kernels.json")
KERNEL_SOURCE = os.path.join(ROOT, "layered-prefill_amd", "csrc", "grouped_gemm.hip")


def measured_traffic(workload: str, kernel: str, grid: int):
    """HBM bytes per launch of the dominant kernel from the committed counter run
    (profiles/hbm_traffic_grouped_gemm_kernels.json: FETCH_SIZE and WRITE_SIZE of
    rocprofv3 --pmc runs, scaled by a plain copy).  The record names the kernel, its
    grid and the sha256 of the kernel source it was measured on: when any of the
    three no longer matches the build being timed the figure would be stale, and
    None is reported instead."""
    import hashlib
    try:
        rec = json.load(open(TRAFFIC_JSON))
        src = hashlib.sha256(open(KERNEL_SOURCE, "rb").read()).hexdigest()
    except (OSError, ValueError):
        return None
    if rec.get("source_sha256") != src:
        return None
    for e in rec.get("launches", []):
        if e.get("workload") == workload and e.get("kernel") == kernel and e.get("grid") == grid:
            return int(e["fetch_bytes"]) + int(e["write_bytes"])
    return None


def one_launch_grid(layer) -> int:
    """Workgroups of the one-launch kernel for this layer: 8 XCDs x the longest m-block
    range the plan may give an XCD x (gate-up + down n-tiles)."""
    s = layer.shape
    cap = layer.T * s.top_k + s.experts * (layer.bm - 1)
    mbs = -(-cap // 256)
    cap_mb = min(2 * -(-mbs // 8), mbs)
    return 8 * cap_mb * (-(-s.intermediate // 128) + -(-s.hidden // 256))


def _events(n):
    return [torch.cuda.Event(enable_timing=True) for _ in range(n)]


class Layer:
    """Inputs of one workload on the GPU plus the pre-allocated scratch a
    serving loop would reuse."""

    def __init__(self, moe, name: str, dev, layout: str = "plain", weights=None):
        """``layout`` "tiled": the expert weights the steps run on are the copies that
        ``FusedMoE.process_weights_after_loading`` makes once after loading
        (``ops.tile_expert_weights``); ``w13`` / ``w2`` stay the row-major tensors.
        ``weights``: (w13, w2, w13_run, w2_run) of another Layer of the same model, shared."""
        wl = moe.workloads
        self.moe = moe
        self.name = name
        self.shape, x, logits, w13, w2 = wl.make_config(name)
        self.T = x.shape[0]
        self.x, self.logits = x.to(dev), logits.to(dev)
        self.layout = layout
        if weights is not None:
            self.w13, self.w2, self.w13_run, self.w2_run = weights
        else:
            self.w13, self.w2 = w13.to(dev), w2.to(dev)
            self.w13_run, self.w2_run = self.w13, self.w2
            if layout == "tiled":
                self.w13_run = moe.ops.tile_expert_weights(self.w13, True)
                self.w2_run = moe.ops.tile_expert_weights(self.w2, False)
        self.dev = dev
        s = self.shape
        self.bm = moe.try_get_optimal_moe_config(self.w13.shape, self.w2.shape, s.top_k, None,
                                                 self.T)["BLOCK_SIZE_M"]
        ws = moe.fused_moe.fused_experts_workspace_bytes(self.T, s.hidden, s.intermediate,
                                                         s.experts, s.top_k, self.bm, x.dtype)
        self.workspace = torch.empty(ws, dtype=torch.uint8, device=dev)
        self.out = torch.empty_like(self.x)

    def experts(self, x, tw, ids):
        """``fused_experts`` on this layer's weights in the layout it runs with."""
        return self.moe.fused_experts(x, self.w13_run, self.w2_run, None, None, tw, ids, weight_layout=self.layout)

    def with_layout(self, layout: str) -> "Layer":
        """The same inputs, weights and scratch run with the other weight layout."""
        other = Layer.__new__(Layer)
        other.__dict__.update(self.__dict__)
        other.layout = layout
        if layout == "plain":
            other.w13_run, other.w2_run = self.w13, self.w2
        elif self.layout != "tiled":
            other.w13_run = self.moe.ops.tile_expert_weights(self.w13, True)
            other.w2_run = self.moe.ops.tile_expert_weights(self.w2, False)
        return other

    def step(self):
        """The layer call as ``FusedMoE.forward`` makes it (``UnquantizedFusedMoEMethod.apply``):
        ``fused_topk`` then ``fused_experts`` through ``fused_topk_experts``."""
        return self.moe.fused_topk_experts(self.x, self.logits, self.w13_run, self.w2_run, self.shape.top_k, True,
                                           weight_layout=self.layout)

    def step_instrumented(self, ev):
        """Same work with an event after every stage (5 stages -> 6 events), the two
        GEMM passes as separate launches; then both passes the way ``step`` enqueues
        them (for the 16-bit large tile: one launch behind the 5 us range-plan kernel),
        between events 6 and 7."""
        moe, s = self.moe, self.shape
        fm = moe.fused_moe
        ev[0].record()
        tw, ids, _ = moe.fused_topk(self.x, self.logits, s.top_k, True)
        ev[1].record()
        sorted_ids, expert_ids, npp = fm.moe_align_block_size(ids, self.bm, s.experts)
        ev[2].record()
        for i, mask in enumerate((1, 2, 4)):
            fm.launch_fused_experts(self.x, self.out, self.w13_run, self.w2_run, None, None, None, None, tw,
                                    sorted_ids, expert_ids, npp, self.bm, workspace=self.workspace,
                                    passes=mask, weight_layout=self.layout)
            ev[3 + i].record()
        ev[6].record()
        fm.launch_fused_experts(self.x, self.out, self.w13_run, self.w2_run, None, None, None, None, tw,
                                sorted_ids, expert_ids, npp, self.bm, workspace=self.workspace, passes=3,
                                weight_layout=self.layout)
        ev[7].record()
        return ids

    def n_active(self, ids) -> int:
        return int(torch.unique(ids).numel())


def time_steps(layer: Layer, steps: int, warmup: int):
    for _ in range(warmup):
        layer.step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps):
        layer.step()
    torch.cuda.synchronize()
    return (time.perf_counter() - t0) * 1e3 / steps


def time_steps_rotating(layer: Layer, steps: int, warmup: int, nsets: int = 4):
    """Back-to-back steps, no host synchronisation, each on the next of ``nsets`` distinct
    copies of the expert weights (the experts rotated by one per copy, so every copy is a
    different 1.2 GB in memory: 4.8 GB in all against 256 MB of memory-side cache).  A step
    then finds none of its weights in any cache, as in a model whose layers each bring their
    own experts, while the GPU stays in the sustained state of the timed loop."""
    sets = [(layer.w13_run.roll(k, 0).contiguous(), layer.w2_run.roll(k, 0).contiguous()) for k in range(nsets)]
    moe, s = layer.moe, layer.shape

    def step(i):
        w13, w2 = sets[i % nsets]
        return moe.fused_topk_experts(layer.x, layer.logits, w13, w2, s.top_k, True, weight_layout=layer.layout)

    for i in range(warmup):
        step(i)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for i in range(steps):
        step(i)
    torch.cuda.synchronize()
    ms = (time.perf_counter() - t0) * 1e3 / steps
    del sets
    return ms


def time_steps_flushed(layer: Layer, steps: int):
    """Per-step event timing with L2 and the 256 MB memory-side cache overwritten
    between steps (a 1 GiB fill), so that no expert weight of the previous step
    is served from a cache.  Returns (median, p10, p90) in ms."""
    flush = torch.empty(1 << 30, dtype=torch.uint8, device=layer.dev)
    times = []
    for i in range(steps + 3):
        flush.fill_(i & 0xff)
        ev = _events(2)
        ev[0].record()
        layer.step()
        ev[1].record()
        torch.cuda.synchronize()
        if i >= 3:
            times.append(ev[0].elapsed_time(ev[1]))
    del flush
    times.sort()
    pick = lambda q: times[min(len(times) - 1, int(q * len(times)))]
    return pick(0.5), pick(0.1), pick(0.9)


def time_graph_replays(layer: Layer, steps: int, warmup: int, inner: int = 1):
    """`inner` steps recorded once into a HIP graph and replayed: what a serving loop
    that captures its decode iteration pays (the reference runs this layer inside
    captured graph segments that hold many layers, nanovllm/models/qwen3_moe.py:673-759).
    Returns (ms per step, max |graph - eager| of the last step's output)."""
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        for _ in range(3):
            layer.step()
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    eager = layer.step().float()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        for _ in range(inner):
            out = layer.step()
    replays = max(1, steps // inner)
    for _ in range(max(1, warmup // inner)):
        graph.replay()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(replays):
        graph.replay()
    torch.cuda.synchronize()
    ms = (time.perf_counter() - t0) * 1e3 / (replays * inner)
    return ms, float((out.float() - eager).abs().max())


def time_router_gate(moe, layer: Layer, steps: int):
    """The two steps ahead of the measured path: the residual add + RMSNorm that
    produces the block's input (csrc/layernorm_kernels.cu:77-108 of the reference;
    four tensors of T*H elements move once each) and the router gate, as gate linear
    + fused_topk the way the reference runs them (nanovllm/models/qwen3_moe.py:93-104,113)
    against the one-kernel fused_gate_topk.  Microseconds per call, events around
    `steps` calls."""
    s = layer.shape
    g = torch.Generator().manual_seed(99)
    wg = (torch.randn(s.experts, s.hidden, generator=g) * 0.02).to(layer.x.dtype).to(layer.dev)

    def two_step():
        return moe.fused_topk(layer.x, torch.nn.functional.linear(layer.x, wg), s.top_k, True)

    def fused():
        return moe.fused_gate_topk(layer.x, wg, s.top_k, True)

    res = torch.randn_like(layer.x)
    normed = torch.empty_like(layer.x)
    wn = torch.ones(s.hidden, dtype=layer.x.dtype, device=layer.dev)

    def norm():
        moe.ops.add_rms_norm(normed, res, layer.x, wn, 1e-6)

    out = {}
    for name, fn in (("linear_then_topk_us", two_step), ("fused_gate_topk_us", fused), ("add_rms_norm_us", norm)):
        for _ in range(5):
            fn()
        ev = _events(2)
        ev[0].record()
        for _ in range(steps):
            fn()
        ev[1].record()
        torch.cuda.synchronize()
        out[name] = round(ev[0].elapsed_time(ev[1]) * 1e3 / steps, 2)
    out["add_rms_norm_gbs"] = round(4 * layer.x.numel() * layer.x.element_size() / out["add_rms_norm_us"] * 1e-3, 1)
    return out


def trace_mix(moe, layer: Layer, steps: int):
    """Layer calls as a layered-prefill engine would issue them on the ShareGPT length
    sample: the schedule (nanovllm/engine/scheduler.py:181-328 restated on the host) over
    400 requests with Poisson arrivals, a 48-layer model, 16 configured stages, 256
    sequences and 8192 prompt tokens per group at most.  Call sizes are bucketed (64-token
    steps up to 512 tokens, 1024-token steps above), the buckets that carry the most tokens
    are timed with this layer's weights, and the token throughput of the mix is reported."""
    sch = moe.schedule
    wl = moe.workloads
    s = layer.shape
    num_layers = 48
    reqs = sch.poisson_requests(sch.load_length_trace(), 400, per_iteration=0.4, seed=0)
    shapes = sch.simulate(reqs, num_layers=num_layers, configured_stages=16, max_num_seqs=256,
                          max_num_batched_tokens=8192)
    sizes = sch.moe_call_sizes(shapes, num_layers)
    buckets = {}
    for t, calls in sizes.items():
        b = -(-t // 64) * 64 if t <= 512 else max(1024, int(round(t / 1024.0)) * 1024)
        c, tok = buckets.get(b, (0, 0))
        buckets[b] = (c + calls, tok + calls * t)
    total_tok = sum(tok for _, tok in buckets.values())
    total_calls = sum(c for c, _ in buckets.values())
    picked = sorted(buckets, key=lambda b: -buckets[b][1])[:6]
    rows, t_ms, t_tok = [], 0.0, 0
    for b in sorted(picked):
        x, logits = wl.make_inputs(s, b, 700 + b, layer.x.dtype)
        x, logits = x.to(layer.dev), logits.to(layer.dev)

        def step():
            return moe.fused_topk_experts(x, logits, layer.w13_run, layer.w2_run, s.top_k, True,
                                          weight_layout=layer.layout)

        # sustained rate per bucket: about 40 ms of warm-up, then `steps` timed calls
        for _ in range(max(3, min(200, int(40.0 / (0.1 + b * 1e-4))))):
            step()
        ev = _events(2)
        ev[0].record()
        for _ in range(steps):
            step()
        ev[1].record()
        torch.cuda.synchronize()
        ms = ev[0].elapsed_time(ev[1]) / steps
        calls, tok = buckets[b]
        rows.append({"tokens": b, "calls_share": round(calls / total_calls, 4),
                     "tokens_share": round(tok / total_tok, 4), "ms": round(ms, 4)})
        t_ms += calls * ms
        t_tok += tok
    return {"trace": "sharegpt_8k_lengths_first2048.csv", "requests": len(reqs), "iterations": len(shapes),
            "layers": num_layers, "stages": 16, "buckets": rows,
            "covered_tokens_share": round(t_tok / total_tok, 4),
            "layer_tokens_per_s": round(t_tok / (t_ms * 1e-3), 0)}


def time_stages(layer: Layer, steps: int, warmup: int = 10):
    """Per-stage times from events recorded inside a run of back-to-back steps: no
    synchronisation between steps, so the GPU is in the same sustained state as in
    the timed loop (after an idle gap the first ~20 steps of this layer run up to
    15 % slower while the power management settles)."""
    names = ["topk_softmax", "moe_align_block_size", "gate_up_gemm_act", "down_gemm_weighted",
             "topk_combine"]
    per = {n: [] for n in names + ["both_gemm_passes"]}
    ids = None
    for _ in range(warmup):
        layer.step_instrumented(_events(8))
    evs = []
    for _ in range(steps):
        ev = _events(8)
        ids = layer.step_instrumented(ev)
        evs.append(ev)
    torch.cuda.synchronize()
    for ev in evs:
        for i, n in enumerate(names):
            per[n].append(ev[i].elapsed_time(ev[i + 1]))
        per["both_gemm_passes"].append(ev[6].elapsed_time(ev[7]))
    return {n: statistics.fmean(v) for n, v in per.items()}, ids


def balanced_routing(moe, layer: "Layer", steps: int, warmup: int):
    """The same layer with every expert receiving the same number of rows: the first
    7936 tokens, token t's choice k going to expert (37 * (K t + k)) mod E with weight
    1/K, which at E = 128, K = 8 gives every expert 496 rows: one full 256-slot block and
    one of 240 rows, and no workgroup left streaming the weights of an expert with a
    handful of rows.  (7936 rather than 8192 tokens so that the launch has a grid of its
    own in a kernel trace.)  Routing and alignment are timed with it, as in the headline
    step.  The number says how much of the headline's distance to the peak is the
    benchmark routing's skew and how much is the kernels'."""
    s = layer.shape
    K, E = s.top_k, s.experts
    T = min(layer.T, 7936)
    x, logits = layer.x[:T].contiguous(), layer.logits[:T].contiguous()
    t = torch.arange(T, device=layer.dev).view(T, 1)
    k = torch.arange(K, device=layer.dev).view(1, K)
    ids = ((t * K + k) * 37 % E).to(torch.int32).contiguous()
    tw = torch.full((T, K), 1.0 / K, dtype=torch.float32, device=layer.dev)
    counts = torch.bincount(ids.flatten().long(), minlength=E)

    def step():
        moe.fused_topk(x, logits, K, True)          # timed like the headline, result unused
        return layer.experts(x, tw, ids)

    for _ in range(warmup):
        step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps):
        step()
    torch.cuda.synchronize()
    ms = (time.perf_counter() - t0) * 1e3 / steps
    fl = moe.workloads.layer_flops(T, s)
    return {"tokens": T, "rows_per_expert": [int(counts.min()), int(counts.max())], "ms_per_step": round(ms, 4),
            "tflops": round(fl / (ms * 1e-3) / 1e12, 2),
            "frac_of_bf16_peak": round(fl / (ms * 1e-3) / 1e12 / PEAK_BF16_TFLOPS, 4)}


def chunk_amplification(moe, layer: "Layer", reps: int, mode: str = "both"):
    """Config 4: the 8192-token prompt as 16 chunks of 512 tokens, each co-batched
    with the 256 decode tokens (16 calls of T=768), against the single 8192+256
    pass on the same layer.  Chunked prefill streams every active expert's
    weights once per chunk; the layered pass streams them once."""
    wl, s = moe.workloads, layer.shape
    dec = torch.arange(8192, 8448, device=layer.dev)
    chunks = []
    for c in range(16):
        sel = torch.cat([torch.arange(c * 512, (c + 1) * 512, device=layer.dev), dec])
        chunks.append((layer.x[sel].contiguous(), layer.logits[sel].contiguous()))

    def run_chunked():
        act = 0
        for xc, lc in chunks:
            tw, ids, _ = moe.fused_topk(xc, lc, s.top_k, True)
            layer.experts(xc, tw, ids)
        return act

    def timed(fn):
        fn()
        torch.cuda.synchronize()
        ev = _events(2)
        ev[0].record()
        for _ in range(reps):
            fn()
        ev[1].record()
        torch.cuda.synchronize()
        return ev[0].elapsed_time(ev[1]) / reps

    out = {}
    per_expert = 3 * s.hidden * s.intermediate * 2
    if mode in ("both", "chunked"):
        out["chunked_16x(512+256)_ms"] = round(timed(run_chunked), 4)
        act = 0
        for xc, lc in chunks:
            _, ids, _ = moe.fused_topk(xc, lc, s.top_k, True)
            act += int(torch.unique(ids).numel())
        out["chunked_expert_weight_bytes"] = act * per_expert
    if mode in ("both", "single"):
        out["single_pass_ms"] = round(timed(layer.step), 4)
        _, ids, _ = moe.fused_topk(layer.x, layer.logits, s.top_k, True)
        out["single_expert_weight_bytes"] = int(torch.unique(ids).numel()) * per_expert
    if mode == "both":
        out["time_ratio"] = round(out["chunked_16x(512+256)_ms"] / out["single_pass_ms"], 3)
        out["weight_bytes_ratio"] = round(out["chunked_expert_weight_bytes"] / out["single_expert_weight_bytes"], 3)
    return out


def cpu_baseline(moe, name: str, runs: int):
    """The oracle (PyTorch fp32 restatement of the reference's MoE math; bf16
    weights upcast per expert) on this host's cores: bounded sample."""
    oracle = importlib.import_module("oracle.moe_oracle")
    wl = moe.workloads
    shape, x, logits, w13, w2 = wl.make_config(name)
    cores = os.cpu_count() or 1
    env = os.environ.get("OMP_NUM_THREADS")
    if env and env.isdigit():
        cores = min(cores, int(env))
    torch.set_num_threads(cores)

    def once():
        tw, ids, _ = oracle.fused_topk(x, logits, shape.top_k, True)
        oracle.moe_align_block_size(ids, 64, shape.experts)
        return oracle.fused_experts_ref(x, w13, w2, tw, ids)

    once()  # warm-up
    t0 = time.perf_counter()
    for _ in range(runs):
        once()
    dt = (time.perf_counter() - t0) / runs
    return dt, torch.get_num_threads()


def legs(a, moe, dev, wl, main_layer, shape, flops, out) -> None:
    """Everything but the headline: the decode-only call (config 2), router gate,
    call-size mix, chunk amplification (config 4), e4m3 (config 5)."""
    compute_bound = a.workload == "layered_8192p_256d"
    # the light legs first and the compute-bound ones last: the headline steps that follow this
    # function then start from the clocks and power state of sustained large calls, not from the
    # low-power state the decode-sized legs leave behind
    if compute_bound:
        dec = Layer(moe, "decode_256", dev, a.weight_layout)
        dms = time_steps(dec, max(a.steps, 50), max(a.warmup, 10))
        dstages, dids = time_stages(dec, 20)
        dact = dec.n_active(dids)
        dbytes = wl.layer_bytes(dec.T, dec.shape, dact)
        dgbs = dbytes / (dms * 1e-3) / 1e9
        out["decode"] = {"workload": "decode_256", "tokens": dec.T, "ms_per_step": round(dms, 4),
                         "hbm_gbs": round(dgbs, 1), "frac_of_hbm_peak": round(dgbs / PEAK_HBM_GBS, 4),
                         "active_experts": dact, "block_size_m": dec.bm,
                         "stage_ms": {k: round(v, 4) for k, v in dstages.items()}}
        rms = time_steps_rotating(dec, max(a.steps, 60), max(a.warmup, 12))
        out["decode"]["rotating_weights"] = {"weight_sets": 4, "ms_per_step": round(rms, 4),
                                             "hbm_gbs": round(dbytes / (rms * 1e-3) / 1e9, 1),
                                             "frac_of_hbm_peak": round(dbytes / (rms * 1e-3) / 1e9 / PEAK_HBM_GBS, 4)}
        if a.weight_layout != "plain":
            pms = time_steps(dec.with_layout("plain"), max(a.steps, 50), max(a.warmup, 10))
            out["decode"]["plain_layout"] = {"ms_per_step": round(pms, 4),
                                             "hbm_gbs": round(dbytes / (pms * 1e-3) / 1e9, 1),
                                             "frac_of_hbm_peak": round(dbytes / (pms * 1e-3) / 1e9 / PEAK_HBM_GBS, 4)}
        out["decode"]["router_gate"] = time_router_gate(moe, dec, 100)
        fmed, fp10, fp90 = time_steps_flushed(dec, 30)
        out["decode"]["cache_flushed"] = {"ms_median": round(fmed, 4), "ms_p10": round(fp10, 4),
                                          "ms_p90": round(fp90, 4),
                                          "hbm_gbs": round(dbytes / (fmed * 1e-3) / 1e9, 1)}
        if not a.no_graph:
            # one step per graph (every replay pays the launch of a graph), and eight steps per
            # graph (a captured model segment holds many layers: that cost is shared)
            gms1, gerr1 = time_graph_replays(dec, max(a.steps, 50), max(a.warmup, 10))
            gms, gerr = time_graph_replays(dec, max(a.steps, 80), max(a.warmup, 16), inner=8)
            ggbs = dbytes / (gms * 1e-3) / 1e9
            out["decode"]["hip_graph"] = {"steps_per_graph": 8, "ms_per_step": round(gms, 4),
                                          "hbm_gbs": round(ggbs, 1),
                                          "frac_of_hbm_peak": round(ggbs / PEAK_HBM_GBS, 4),
                                          "one_step_per_graph_ms": round(gms1, 4),
                                          "max_abs_diff_vs_eager": max(gerr, gerr1)}
        del dec
    out["router_gate"] = time_router_gate(moe, main_layer, 50)
    if compute_bound and not a.no_trace_mix:
        out["trace_mix"] = trace_mix(moe, main_layer, max(10, a.steps // 4))
    if compute_bound and a.chunk_mode != "off":
        out["chunk_amplification"] = chunk_amplification(moe, main_layer, max(2, a.steps // 10), a.chunk_mode)
    if compute_bound and not a.no_balanced:
        out["balanced_routing"] = balanced_routing(moe, main_layer, max(20, a.steps // 4), max(20, a.warmup // 2))
    if compute_bound and not a.no_fp8:
        # config 5: e4m3 weights (per-output-channel scales), per-token e4m3 activations
        w13q, w13s, w2q, w2s = moe.quantize_expert_weights(main_layer.w13, main_layer.w2)

        def fp8_step():
            tw, ids8, _ = moe.fused_topk(main_layer.x, main_layer.logits, shape.top_k, True)
            return moe.fused_experts(main_layer.x, w13q, w2q, None, None, tw, ids8,
                                     per_channel_quant=True, w1_scale=w13s, w2_scale=w2s)

        for _ in range(a.warmup):
            fp8_step()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(a.steps):
            fp8_step()
        torch.cuda.synchronize()
        fms = (time.perf_counter() - t0) * 1e3 / a.steps
        out["fp8_e4m3"] = {"workload": a.workload, "ms_per_step": round(fms, 4),
                           "tflops": round(flops / (fms * 1e-3) / 1e12, 2),
                           "frac_of_fp8_peak": round(flops / (fms * 1e-3) / 1e12 / 5000.0, 4),
                           "block_size_m": moe.try_get_optimal_moe_config(
                               main_layer.w13.shape, main_layer.w2.shape, shape.top_k, "fp8_w8a8",
                               main_layer.T)["BLOCK_SIZE_M"]}
        del w13q, w2q



def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    # defaults long enough to measure the sustained rate: after an idle gap the first
    # ~20 steps (20 ms) of this layer run up to 15 % slower while the clocks settle
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=50)
    ap.add_argument("--workload", default="layered_8192p_256d",
                    choices=["layered_8192p_256d", "decode_256"])
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--cpu-runs", type=int, default=16,
                    help="timed passes of the CPU baseline (about 0.65 s each on 16 cores)")
    ap.add_argument("--chunk-mode", default="both", choices=["both", "chunked", "single", "off"],
                    help="config 4 (chunk amplification) leg: both sides, one side only (for "
                         "rocprofv3 counter runs), or off")
    ap.add_argument("--no-fp8", action="store_true", help="skip the e4m3 leg (config 5)")
    ap.add_argument("--no-graph", action="store_true", help="skip the HIP-graph replay of the decode leg")
    ap.add_argument("--no-balanced", action="store_true", help="skip the balanced-routing leg")
    ap.add_argument("--no-trace-mix", action="store_true",
                    help="skip the layered-prefill call-size mix of the ShareGPT length sample")
    ap.add_argument("--copy-calibration", action="store_true",
                    help="also run three plain 1 GiB device copies, the known-size kernel that "
                         "FETCH_SIZE / WRITE_SIZE readings are scaled by")
    ap.add_argument("--only-chunk-leg", action="store_true",
                    help="run nothing but the chunk-amplification leg")
    ap.add_argument("--weight-layout", default="tiled", choices=["tiled", "plain"],
                    help="expert weights as FusedMoE(weight_layout=...).process_weights_after_loading leaves "
                         "them: re-ordered once into the DMA kernels' unit order (tiled), or row-major as "
                         "loaded (plain; with tiled, the plain figures are reported next to it)")
    ap.add_argument("--block-size-m", type=int, default=0,
                    help="override the alignment block size (0 = the library's choice)")
    a = ap.parse_args()
    if a.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        print("bench.py: this build is the single-GPU (TP=1) expert path; it has no collectives "
              "and measures one GPU only. Run with --gpus 1.", file=sys.stderr)
        return 2
    if not torch.cuda.is_available():
        print("bench.py: no GPU visible; the HIP path has no CPU fallback.", file=sys.stderr)
        return 3
    moe = importlib.import_module("layered-prefill_amd")
    moe._lib.lib()
    dev = torch.device("cuda:0")
    wl = moe.workloads

    if a.block_size_m:
        moe.fused_moe.try_get_optimal_moe_config = lambda *x, **k: {"BLOCK_SIZE_M": a.block_size_m}
        moe.try_get_optimal_moe_config = moe.fused_moe.try_get_optimal_moe_config
    if a.copy_calibration:
        src = torch.empty(1 << 30, dtype=torch.uint8, device=dev).fill_(1)
        dst = torch.empty_like(src)
        for _ in range(3):
            dst.copy_(src)
        torch.cuda.synchronize()
        del src, dst
    main_layer = Layer(moe, a.workload, dev, a.weight_layout)
    if a.only_chunk_leg:
        print(json.dumps({"chunk_amplification": chunk_amplification(moe, main_layer, max(2, a.steps // 10),
                                                                      a.chunk_mode)}))
        return 0
    # The same W warm-up + K timed steps twice: here, right after the inputs were built on the
    # host (the GPU has been idle for seconds and its clocks take about 20 ms of work to settle),
    # and at the end of the GPU legs of this run (clocks settled: the rate a serving loop that
    # runs layer after layer sees).  The second is the headline; both are reported.
    ms_after_idle = time_steps(main_layer, a.steps, a.warmup)
    shape = main_layer.shape
    flops = wl.layer_flops(main_layer.T, shape)
    out = {}
    legs(a, moe, dev, wl, main_layer, shape, flops, out)
    ms = time_steps(main_layer, a.steps, a.warmup)
    ms_plain = time_steps(main_layer.with_layout("plain"), a.steps, a.warmup) if a.weight_layout != "plain" else None
    ms_rot = time_steps_rotating(main_layer, a.steps, a.warmup)
    stages, ids = time_stages(main_layer, max(5, a.steps // 2))
    n_active = main_layer.n_active(ids)
    abytes = wl.layer_bytes(main_layer.T, shape, n_active)
    tflops = flops / (ms * 1e-3) / 1e12
    gbs = abytes / (ms * 1e-3) / 1e9

    compute_bound = a.workload == "layered_8192p_256d"
    # dominant kernel: with blocks of 256 both grouped GEMMs (gate-up + SiLU*up, down x
    # routed weight) are one launch, timed between two events together with the range
    # plan kernel in front of it (5 us); with blocks of 32 the gate-up streaming kernel
    one_launch = main_layer.bm % 256 == 0
    if compute_bound:
        # 6*T*K*H*I algorithmic flops in the one launch, 4*T*K*H*I in a gate-up launch
        k_flops = (6 if one_launch else 4) * main_layer.T * shape.top_k * shape.hidden * shape.intermediate
        k_ms = stages["both_gemm_passes" if one_launch else "gate_up_gemm_act"]
        ach = k_flops / (k_ms * 1e-3) / 1e12
        roofline = {"bound": "mfma",
                    "kernel": "big_fused_kernel<MmaBF16> (gate-up GEMM + SiLU*up and down GEMM x routed weight, one launch)"
                              if one_launch else "gate-up grouped GEMM",
                    "achieved": round(ach, 2), "peak": PEAK_BF16_TFLOPS, "unit": "TFLOP/s",
                    "frac": round(ach / PEAK_BF16_TFLOPS, 4), "kernel_ms": round(k_ms, 4),
                    "traffic": measured_traffic(a.workload, "big_fused_kernel<MmaBF16>", one_launch_grid(main_layer))
                               if one_launch else None}
        value, unit, metric = tflops, "TFLOP/s", METRIC
    else:
        # weights of the active experts once (3*H*I each), x read, c3 written
        k_bytes = (n_active * (3 if one_launch else 2) * shape.hidden * shape.intermediate * 2
                   + main_layer.T * shape.hidden * 2
                   + (main_layer.T * shape.top_k * shape.hidden * 2 if one_launch else 0))
        k_ms = stages["both_gemm_passes" if one_launch else "gate_up_gemm_act"]
        ach = k_bytes / (k_ms * 1e-3) / 1e9
        roofline = {"bound": "hbm",
                    "kernel": "big_fused_kernel<MmaBF16> (both grouped GEMMs, one launch)" if one_launch
                              else "stream_gemm_kernel<MmaBF16, gated> (gate-up GEMM, SiLU*up epilogue)",
                    "achieved": round(ach, 1), "peak": PEAK_HBM_GBS, "unit": "GB/s",
                    "frac": round(ach / PEAK_HBM_GBS, 4), "kernel_ms": round(k_ms, 4),
                    "traffic": measured_traffic(a.workload, "big_fused_kernel<MmaBF16>", one_launch_grid(main_layer))
                               if one_launch else None}
        value, unit, metric = gbs, "GB/s", METRIC + " [decode-only workload: HBM GB/s]"

    head = {
        "metric": metric, "value": round(value, 2), "unit": unit, "n_gpus": 1, "steps": a.steps,
        "warmup": a.warmup, "ms_per_step": round(ms, 4), "higher_is_better": True,
        "scaling": "weak", "vs_baseline": None, "dtype": "bf16", "data": "synthetic",
        "config": {"workload": a.workload, "tokens": main_layer.T, "hidden": shape.hidden,
                   "experts": shape.experts, "intermediate": shape.intermediate,
                   "top_k": shape.top_k, "block_size_m": main_layer.bm, "active_experts": n_active,
                   "weight_layout": a.weight_layout + (
                       " (FusedMoE(weight_layout='tiled').process_weights_after_loading: the loaded "
                       "weights re-ordered once; plain_layout = row-major as loaded)"
                       if a.weight_layout == "tiled" else " (row-major, as loaded)")},
        "layer_tflops": round(tflops, 2), "layer_frac_of_bf16_peak": round(tflops / PEAK_BF16_TFLOPS, 4),
        "layer_algorithmic_gbs": round(gbs, 1),
        "stage_ms": {k: round(v, 4) for k, v in stages.items()},
        "roofline": roofline,
        "gpu_state": "value / ms_per_step: W warm-up + K timed steps at the end of this run's GPU legs (clocks "
                     "settled); after_idle: the same W + K right after start-up, inside the clock ramp that "
                     "follows an idle GPU; stage_ms and roofline come from the run of stage events right after "
                     "the headline steps",
        "after_idle": {"ms_per_step": round(ms_after_idle, 4),
                       "tflops": round(flops / (ms_after_idle * 1e-3) / 1e12, 2)},
        "rotating_weights": {"weight_sets": 4, "ms_per_step": round(ms_rot, 4),
                             "tflops": round(flops / (ms_rot * 1e-3) / 1e12, 2)},
    }
    if ms_plain is not None:
        head["plain_layout"] = {"ms_per_step": round(ms_plain, 4),
                                "tflops": round(flops / (ms_plain * 1e-3) / 1e12, 2)}
    head.update(out)
    out = head

    if not a.no_cpu_baseline:
        del main_layer
        torch.cuda.empty_cache()
        dt, cores = cpu_baseline(moe, a.workload, a.cpu_runs)
        if compute_bound:
            cv, cu = flops / dt / 1e12, "TFLOP/s"
        else:
            cv, cu = abytes / dt / 1e9, "GB/s"
        out["cpu_baseline"] = {"value": round(cv, 4), "unit": cu, "cores": cores, "kind": "port",
                               "sample": f"{a.cpu_runs} full passes of {a.workload} (1 warm-up), "
                                         f"oracle fp32 torch matmul, bf16 weights upcast per expert, "
                                         f"{dt:.2f} s per pass"}
    print(json.dumps(out))
    return 0


if __name__ == "__main__":
    sys.exit(main())
