#!/usr/bin/env python3
"""Benchmark of the low-bit KV-cache decode step on one MI355X.

A step is one decode-attention call (split-KV kernel + combine) over one batch of synthetic
input.  Workload = Llama-3-8B-shape GQA decode: batch 1, 32 q heads / 8 kv heads, head_dim 128,
32768 packed tokens at 4 bits (group 128) plus a 128-token fp16 residual window (--workload selects the
other shapes, among them a ragged batch of 16).  Prints ONE JSON line; see --help for the side
measurements it carries.
"""
from __future__ import annotations

import argparse
import json
import math
import os
import sys
import time

import torch

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0

# HBM bytes per launch of the split-KV kernel, from rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE
# (profiles/fwd_splitkv_hbm_traffic_all_workloads.md): mean counter values per dispatch at the default split
# count; a 256 MiB device copy in the same runs reads 131085 and 262144, i.e. the fetch counter is in units of
# 2 KiB and the write counter in KiB.
MEASURED_TRAFFIC_BYTES = {
    "llama3-8b-gqa-32k-4bit-g128": int(17978.92 * 2048 + 619.61 * 1024),
    "llama2-7b-mha-4k-4bit-g128": int(9901.16 * 2048 + 162.56 * 1024),
    "llama3-8b-gqa-128k-2bit-g64": int(41589.20 * 2048 + 618.75 * 1024),
    "llama3-8b-gqa-ragged-1k-8k-b16-4bit-g128": int(56196.71 * 2048 + 1377.33 * 1024),
    "llama3-70b-gqa-64k-2bit-g128-b8": int(150066.51 * 2048 + 1376.00 * 1024),
}

WORKLOADS = {
    # name: (b, h, h_k, S, R, bits, gs, dtype)
    "llama3-8b-gqa-32k-4bit-g128": (1, 32, 8, 32768, 128, 4, 128, torch.float16),
    "llama2-7b-mha-4k-4bit-g128": (1, 32, 32, 4096, 128, 4, 128, torch.float16),
    "llama3-8b-gqa-128k-2bit-g64": (1, 32, 8, 131072, 128, 2, 64, torch.float16),
    "llama3-70b-gqa-64k-2bit-g128-b8": (8, 64, 8, 65536, 128, 2, 128, torch.bfloat16),
    # further shapes, used to tune the launch heuristics (not BASELINE configurations)
    "llama3-8b-gqa-128k-4bit-g128": (1, 32, 8, 131072, 128, 4, 128, torch.float16),
    "llama3-8b-gqa-8k-4bit-g128-b16": (16, 32, 8, 8192, 128, 4, 128, torch.float16),
    "llama3-70b-gqa-64k-4bit-g128-b8": (8, 64, 8, 65536, 128, 4, 128, torch.bfloat16),
    "llama3-8b-gqa-96k-4bit-g128": (1, 32, 8, 98304, 128, 4, 128, torch.float16),
    "llama3-8b-gqa-64k-4bit-g128": (1, 32, 8, 65536, 128, 4, 128, torch.float16),
    "llama3-8b-gqa-48k-4bit-g128": (1, 32, 8, 49152, 128, 4, 128, torch.float16),
    "llama3-8b-gqa-16k-4bit-g128-b4": (4, 32, 8, 16384, 128, 4, 128, torch.float16),
    "llama3-8b-gqa-8k-4bit-g128-b4": (4, 32, 8, 8192, 128, 4, 128, torch.float16),
    # ragged batch: 16 sequences of seeded lengths in [1024, 8192]; S is the cache capacity, R the window
    # capacity.  Whole 128-token blocks of a sequence are packed; the remainder (< 128) plus the 128 newest
    # tokens stay in the fp16 window (128-255 tokens), as in a decode loop just before the next block is packed.
    "llama3-8b-gqa-ragged-1k-8k-b16-4bit-g128": (16, 32, 8, 8192, 256, 4, 128, torch.float16),
}
RAGGED = {"llama3-8b-gqa-ragged-1k-8k-b16-4bit-g128": (1024, 8192)}
DEFAULT_WORKLOAD = "llama3-8b-gqa-32k-4bit-g128"
# the other four BASELINE shapes, timed compactly by the default run ("other_configs")
OTHER_CONFIGS = ("llama2-7b-mha-4k-4bit-g128", "llama3-8b-gqa-128k-2bit-g64",
                 "llama3-8b-gqa-ragged-1k-8k-b16-4bit-g128", "llama3-70b-gqa-64k-2bit-g128-b8")


def ragged_lengths(name, b):
    """(packed tokens, window tokens) per sequence of a ragged workload, from a fixed seed."""
    lo, hi = RAGGED[name]
    g = torch.Generator().manual_seed(0)
    total = torch.randint(lo, hi + 1, (b,), generator=g)
    packed = (total - 128).clamp(min=0) // 128 * 128         # the newest 128 tokens are still in the window
    return packed.to(torch.int32), (total - packed).to(torch.int32)


def make_inputs(b, h, h_k, n_tokens, seed, dtype):
    """Seeded N(0,1) on the CPU (so a CPU checker sees the same bits); 3 of 128 K channels per
    kv-head are multiplied by 10 (2 % outlier channels)."""
    g = torch.Generator().manual_seed(seed)
    q = torch.randn((b, 1, h, 128), generator=g)
    k = torch.randn((b, n_tokens, h_k, 128), generator=g)
    v = torch.randn((b, n_tokens, h_k, 128), generator=g)
    for hk in range(h_k):
        ch = torch.randperm(128, generator=g)[:3]
        k[:, :, hk, ch] *= 10.0
    return q.to(dtype), k.to(dtype), v.to(dtype)


def algorithmic_bytes(b, h, h_k, S, R, bits, gs):
    packed = b * h_k * S * 128 * 2 * (bits / 8 + 4 / gs)
    resid = b * h_k * R * 128 * 2 * 2
    qo = 2 * b * h * 128 * 2
    return int(packed + resid + qo), int(packed)


def alloc_cache(b, S, h_k, bits, gs, dev):
    pn = 16 // bits
    return (torch.zeros((b, S // pn, h_k, 128), dtype=torch.uint16, device=dev),
            torch.zeros((b, S // gs, h_k, 128), dtype=torch.float32, device=dev),
            torch.zeros((b, S, h_k, 128 // pn), dtype=torch.uint16, device=dev),
            torch.zeros((b, 128 // gs, h_k, S), dtype=torch.float32, device=dev))


def workload_bytes(name):
    """(algorithmic bytes per step, of which packed stream, packed lengths, window lengths) of a workload; the
    lengths are None unless the workload is ragged."""
    b, h, h_k, S, R, bits, gs, _ = WORKLOADS[name]
    if name in RAGGED:
        packed_len, win_len = ragged_lengths(name, b)
        per_tok = h_k * 128 * 2
        packed_bytes = int(packed_len.sum().item() * per_tok * (bits / 8 + 4 / gs))
        total_bytes = packed_bytes + int(win_len.sum().item()) * per_tok * 2 + 2 * b * h * 128 * 2
        return total_bytes, packed_bytes, packed_len, win_len
    total_bytes, packed_bytes = algorithmic_bytes(b, h, h_k, S, R, bits, gs)
    return total_bytes, packed_bytes, None, None


def make_inputs_gpu(b, h, h_k, n_tokens, seed, dtype, dev):
    """The same distribution generated on the GPU (for the workloads no CPU checker looks at)."""
    g = torch.Generator(device=dev).manual_seed(seed)
    q = torch.randn((b, 1, h, 128), generator=g, device=dev).to(dtype)
    k = torch.randn((b, n_tokens, h_k, 128), generator=g, device=dev, dtype=torch.float16).to(dtype)
    v = torch.randn((b, n_tokens, h_k, 128), generator=g, device=dev, dtype=torch.float16).to(dtype)
    for hk in range(h_k):
        ch = torch.randperm(128, generator=g, device=dev)[:3]
        k[:, :, hk, ch] *= 10.0
    return q, k, v


def build_workload(name, num_splits=0, no_rotate=False, want_sources=False, cpu_inputs=True, max_bufs=16):
    """Packed caches, windows and decode plans of a workload: enough distinct caches that consecutive steps
    cannot be served from the 256 MB Infinity Cache.  With `cpu_inputs` every cache gets its own CPU-seeded
    tensors (a CPU checker sees the same bits); otherwise two GPU-generated sources are packed in turn."""
    from bitladder_amd import kvcache_pack_int, plan_fwd_kvcache_int
    dev = torch.device("cuda:0")
    b, h, h_k, S, R, bits, gs, dtype = WORKLOADS[name]
    scale = 1.0 / math.sqrt(128)
    ragged = name in RAGGED
    total_bytes, packed_bytes, packed_len, win_len = workload_bytes(name)
    if ragged:
        packed_dev, win_dev = packed_len.to(dev), win_len.to(dev)
    nbuf = 1 if no_rotate else max(2, math.ceil(320e6 / total_bytes))
    nbuf = min(nbuf, max_bufs)
    plans, keep, srcs = [], [], []
    first = None
    gpu_src = []
    for i in range(nbuf):
        if cpu_inputs:
            q, k, v = make_inputs(b, h, h_k, S + R, seed=i, dtype=dtype)
            if i == 0:
                first = (q, k, v)
            qd, kd, vd = q.to(dev), k.to(dev), v.to(dev)
        else:
            if i < 2:
                gpu_src.append(make_inputs_gpu(b, h, h_k, S + R, i, dtype, dev))
            qd, kd, vd = gpu_src[i % 2]
        cache = alloc_cache(b, S, h_k, bits, gs, dev)
        kvcache_pack_int(kd[:, :S], cache[0], cache[1], vd[:, :S], cache[2], cache[3], None, None, S,
                         "k-channel", gs, bits)
        if ragged:
            # window of sequence j: its tokens behind the packed prefix
            kres = torch.zeros((b, R, h_k, 128), dtype=dtype, device=dev)
            vres = torch.zeros_like(kres)
            for j in range(b):
                p0, r0 = int(packed_len[j]), int(win_len[j])
                kres[j, :r0], vres[j, :r0] = kd[j, p0:p0 + r0], vd[j, p0:p0 + r0]
            plan = plan_fwd_kvcache_int(qd, *cache, None, scale, "k-channel", gs, bits,
                                        seqlens_k=packed_dev, max_seqlen_k=int(packed_len.max()),
                                        k_residual=kres, v_residual=vres, residual_len=win_dev,
                                        max_residual_len=int(win_len.max()), num_splits=num_splits)
        else:
            kres, vres = kd[:, S:].contiguous(), vd[:, S:].contiguous()
            plan = plan_fwd_kvcache_int(qd, *cache, None, scale, "k-channel", gs, bits,
                                        k_residual=kres, v_residual=vres, num_splits=num_splits)
        plans.append(plan)
        keep.append((cache, kres, vres))
        if want_sources and (i < 2 or sum(a.numel() + b_.numel() for a, b_ in srcs) * 2 < 640e6):
            # fp16 sources for the quantize-pack leg: at least two, and enough of them (more than twice the
            # 256 MB Infinity Cache in total) that no pack call finds its input cached
            srcs.append((kd, vd))
        del kd, vd
    del gpu_src
    torch.cuda.synchronize(dev)
    return {"nbuf": nbuf, "plans": plans, "keep": keep, "srcs": srcs, "first_inputs": first or (None, None, None),
            "total_bytes": total_bytes, "packed_bytes": packed_bytes}


MIN_GRAPH_NODES = 200      # steps captured into one graph (a multiple of --steps): keeps the gaps between graph launches rare
MIN_TIMED_STEPS = 400      # steps inside the timed region
WARM_STEPS = 1600          # untimed replayed steps in front of it: the first ~10 ms after idle run 3-10 % slower


def time_steps(run_step, steps, warmup, use_graph, quantile_reps=0, steady=True, replay_prologue=None):
    """Times `run_step`.  Eager warm-up of `warmup` steps, then one HIP graph of `nodes` steps (`steps` times
    a whole number, at least MIN_GRAPH_NODES when `steady`) is captured, replayed untimed (once to upload it,
    then for WARM_STEPS steps when `steady`) and replayed `replays` times between two events and two host
    synchronisations.  Without a graph the eager loop runs the same number of steps.  Returns a dict with the
    wall and event time per step and what was run.  `replay_prologue`, if given, is captured as the first
    node(s) of the graph (and called before every `nodes` eager steps): state that the steps advance is reset there."""
    dev = torch.device("cuda:0")
    for i in range(warmup):
        run_step(i)
    torch.cuda.synchronize(dev)
    nodes = steps * (max(1, math.ceil(MIN_GRAPH_NODES / steps)) if steady else 1)
    replays = max(1, math.ceil(MIN_TIMED_STEPS / nodes)) if steady else 1
    warm = math.ceil(WARM_STEPS / nodes) if steady else 0
    graph = None
    if use_graph:
        try:
            side = torch.cuda.Stream(dev)
            side.wait_stream(torch.cuda.current_stream(dev))
            with torch.cuda.stream(side):
                run_step(0)
            torch.cuda.current_stream(dev).wait_stream(side)
            graph = torch.cuda.CUDAGraph()
            with torch.cuda.graph(graph):
                if replay_prologue is not None:
                    replay_prologue()
                for i in range(nodes):
                    run_step(i)
            for _ in range(1 + warm):
                graph.replay()          # untimed: the first replay uploads the graph
            torch.cuda.synchronize(dev)
        except Exception as e:      # noqa: BLE001
            print(f"[bench] graph capture unavailable ({e}); timing eager launches", file=sys.stderr)
            graph = None
    if graph is None:
        for i in range(warm * nodes):
            if replay_prologue is not None and i % nodes == 0:
                replay_prologue()
            run_step(i)
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    torch.cuda.synchronize(dev)
    t0 = time.perf_counter()
    e0.record()
    if graph is not None:
        for _ in range(replays):
            graph.replay()
    else:
        for i in range(nodes * replays):
            if replay_prologue is not None and i % nodes == 0:
                replay_prologue()
            run_step(i)
    e1.record()
    torch.cuda.synchronize(dev)
    t1 = time.perf_counter()
    timed = nodes * replays
    res = {"wall_us": (t1 - t0) / timed * 1e6, "event_us": e0.elapsed_time(e1) * 1e3 / timed,
           "graphed": graph is not None, "timed_steps": timed, "graph_nodes": nodes if graph is not None else 0,
           "replays": replays if graph is not None else 0,
           "untimed_replays": 1 + warm if graph is not None else 0, "quantiles": None}
    if quantile_reps and graph is not None:
        # spread of the per-step time over further replays of the same graph (outside the timed region)
        per_step = []
        for _ in range(quantile_reps):
            a, b_ = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            a.record()
            graph.replay()
            b_.record()
            torch.cuda.synchronize(dev)
            per_step.append(a.elapsed_time(b_) * 1e3 / nodes)
        per_step.sort()
        pick = lambda f: round(per_step[min(len(per_step) - 1, int(f * len(per_step)))], 3)
        res["quantiles"] = {"p20": pick(0.2), "p50": pick(0.5), "p80": pick(0.8), "replays": quantile_reps}
    return res


# Read probe (libbitdecode_probe.so, built next to the library; a measurement aid of this file only): kernels that
# read a buffer and do nothing else.  A configuration is (workgroups, threads, mode, depth, nt, pattern); see
# bitladder_amd/csrc/probe.hip.
PROBE_DEFAULT = [   # the configurations the sweep (--probe-sweep) found fastest at one size or another
    (512, 256, 1, 4, 1, 0),
    (512, 256, 1, 8, 1, 0),
    (256, 256, 1, 8, 1, 0),
    (256, 512, 1, 4, 1, 1),
    (1024, 512, 1, 4, 1, 1),
]
_probe_lib = None


def probe_lib():
    global _probe_lib
    if _probe_lib is None:
        import ctypes
        path = os.path.join(ROOT, "bitladder_amd", "libbitdecode_probe.so")
        if not os.path.exists(path):
            raise ImportError(f"{path} is missing: build it with `python -m bitladder_amd.build`")
        L = ctypes.CDLL(path)
        L.bitprobe_read.restype = ctypes.c_int
        L.bitprobe_read.argtypes = [ctypes.c_void_p, ctypes.c_size_t] + [ctypes.c_int] * 6 + [ctypes.c_void_p]
        _probe_lib = L
    return _probe_lib


def probe_name(cfg):
    g, t, mode, depth, nt, pat = cfg
    return "%dx%d %s depth %d%s %s" % (g, t, "lds-dma" if mode else "regs", depth, " nt" if nt else "",
                                     "wg-contiguous" if pat else "round-robin")


def time_probe(nbytes, cfg, steps, warmup, use_graph, bufs, steady=True):
    """us per launch of one read-probe configuration over `nbytes` (rotated buffers); None if it is not built."""
    L = probe_lib()
    dev = torch.device("cuda:0")
    g, t, mode, depth, nt, pat = cfg

    def probe(i):
        buf = bufs[i % len(bufs)]
        if L.bitprobe_read(buf.data_ptr(), nbytes, g, t, mode, depth, nt, pat, torch.cuda.current_stream(dev).cuda_stream):
            raise RuntimeError("probe configuration not available")
    try:
        probe(0)
    except RuntimeError:
        return None
    return time_steps(probe, steps, warmup, use_graph, steady=steady)["event_us"]


def best_probe(nbytes, steps, warmup, use_graph, nbuf, configs=None):
    """(us, configuration name, all timings) of the fastest read-probe configuration over `nbytes`."""
    dev = torch.device("cuda:0")
    nbytes = (nbytes + 4095) // 4096 * 4096
    bufs = [torch.randint(0, 255, (nbytes,), dtype=torch.uint8, device=dev) for _ in range(nbuf)]
    seen = {}
    for cfg in configs or PROBE_DEFAULT:
        us = time_probe(nbytes, cfg, steps, warmup, use_graph, bufs)
        if us is not None:
            seen[probe_name(cfg)] = round(us, 3)
    name = min(seen, key=seen.get)
    return seen[name], name, seen, nbytes


def probe_sweep(args):
    """Table of the read probe over launch shapes and sizes (markdown on stdout)."""
    dev = torch.device("cuda:0")
    sizes = {"20 MB (4K MHA 4-bit)": workload_bytes("llama2-7b-mha-4k-4bit-g128")[0],
             "36 MB (32K GQA 4-bit)": workload_bytes("llama3-8b-gqa-32k-4bit-g128")[0],
             "84 MB (128K GQA 2-bit)": workload_bytes("llama3-8b-gqa-128k-2bit-g64")[0],
             "306 MB (b8 64K 2-bit)": workload_bytes("llama3-70b-gqa-64k-2bit-g128-b8")[0]}
    configs = []
    for g in (256, 512, 1024):
        for t in (256, 512, 1024):
            for nt in (1, 0):
                for pat in (0, 1):
                    for depth in (4, 8, 16):
                        configs.append((g, t, 0, depth, nt, pat))
                    for depth in (4, 8):
                        if (t // 64) * depth <= 128:
                            configs.append((g, t, 1, depth, nt, pat))
    rows = {probe_name(c): {} for c in configs}
    for label, nbytes in sizes.items():
        nbytes = (nbytes + 4095) // 4096 * 4096
        nbuf = max(2, min(16, math.ceil(320e6 / nbytes)))
        bufs = [torch.randint(0, 255, (nbytes,), dtype=torch.uint8, device=dev) for _ in range(nbuf)]
        for c in configs:
            us = time_probe(nbytes, c, 200, 5, True, bufs)
            rows[probe_name(c)][label] = us
            print("[sweep] %s | %s | %s" % (label, probe_name(c), "n/a" if us is None else "%.2f" % us),
                  file=sys.stderr, flush=True)
        del bufs
    print("| configuration | " + " | ".join(sizes) + " |")
    print("|---|" + "---|" * len(sizes))
    for name, r in rows.items():
        print("| %s | " % name + " | ".join("n/a" if r[k] is None else "%.2f" % r[k] for k in sizes) + " |")
    print()
    for label, nbytes in sizes.items():
        ok = {n: r[label] for n, r in rows.items() if r[label] is not None}
        n = min(ok, key=ok.get)
        print("best at %s: %s, %.2f us = %.0f GB/s" % (label, n, ok[n], nbytes / ok[n] / 1e3))
    return 0


# The reference's own sweep (benchmark/bench_single_decode.ipynb:198-207, 311-316: one sequence, MHA 32 x 128,
# S = 1024 ... 524288; and batches 2 ... 64 at S = 4096; fp16, group size 128), its published milliseconds (hardware
# not stated, NVIDIA) as (FA2 fp16, 4-bit, 2-bit).
REFERENCE_SWEEP_MS = {
    ("len", 1024): (0.0430, 0.0215, 0.0174), ("len", 4096): (0.1126, 0.0440, 0.0317),
    ("len", 32768): (0.7741, 0.2202, 0.1536), ("len", 131072): (3.0454, 0.8837, 0.6093),
    ("len", 524288): (12.1876, 4.2557, 2.4873),
    ("batch", 2): (0.2089, 0.0696, 0.0489), ("batch", 16): (1.8463, 0.4567, 0.2949), ("batch", 64): (7.7322, 2.3332, 1.9128),
}


def reference_sweep(args):
    """The reference's sweep on this GPU (markdown on stdout): 4-bit and 2-bit decode and the library's own fp16-KV
    path on the same shapes, every cell timed like the headline (rotated caches, one HIP graph of the steps)."""
    from bitladder_amd import plan_fwd_kvcache_int
    dev = torch.device("cuda:0")
    scale = 1.0 / math.sqrt(128)
    cases = [("len", 1, s_) for s_ in (1024, 2048, 4096, 8192, 16384, 32768, 65536, 131072, 262144, 524288)]
    cases += [("batch", b_, 4096) for b_ in (2, 4, 8, 16, 32, 64)]

    def timed(run, nbytes):
        long_steps = nbytes > 400e6
        return time_steps(run, 40 if long_steps else args.steps, 3 if long_steps else args.warmup, not args.no_graph,
                          steady=not long_steps)["event_us"]

    print("| sweep | b | S | 4-bit us | GB/s | frac of 8 TB/s | 2-bit us | GB/s | frac | fp16-KV us | GB/s | 4-bit x | 2-bit x "
          "| reference ms (fp16 / 4-bit / 2-bit) | reference x |")
    print("|---|---|---|---|---|---|---|---|---|---|---|---|---|---|---|")
    for kind, b, S in cases:
        cells = {}
        for bits in (4, 2):
            name = "sweep-%s-b%d-s%d-%dbit" % (kind, b, S, bits)
            WORKLOADS[name] = (b, 32, 32, S, 128, bits, 128, torch.float16)
            W = build_workload(name, 0, cpu_inputs=False, max_bufs=8)
            n_, plans_ = W["nbuf"], W["plans"]
            us = timed(lambda i, n_=n_, plans_=plans_: plans_[i % n_].run(), W["total_bytes"])
            cells[bits] = (us, W["total_bytes"] / us / 1e3)
            del W, plans_, WORKLOADS[name]
            torch.cuda.empty_cache()
        # the library's fp16 split-KV path over all S + 128 tokens
        tokens = S + 128
        fp16_bytes = b * tokens * 32 * 128 * 2 * 2 + 2 * b * 32 * 128 * 2
        nb16 = max(2, min(8, math.ceil(320e6 / fp16_bytes)))
        dummy = alloc_cache(b, 128, 32, 4, 128, dev)
        fplans = []
        src = [make_inputs_gpu(b, 32, 32, tokens, 50 + i, torch.float16, dev) for i in range(2)]
        for i in range(nb16):
            qd, kd, vd = src[i % 2]
            if i >= 2:
                kd, vd = kd.clone(), vd.clone()
            fplans.append(plan_fwd_kvcache_int(qd, *dummy, None, scale, "k-channel", 128, 4, seqlen_k=0,
                                               k_residual=kd, v_residual=vd))
        us16 = timed(lambda i: fplans[i % nb16].run(), fp16_bytes)
        del fplans, src
        torch.cuda.empty_cache()
        ref = REFERENCE_SWEEP_MS.get((kind, S if kind == "len" else b))
        ref_txt = "%.4f / %.4f / %.4f" % ref if ref else "-"
        ref_x = "%.1f / %.1f" % (ref[0] / ref[1], ref[0] / ref[2]) if ref else "-"
        u4, g4 = cells[4]
        u2, g2 = cells[2]
        print("| %s | %d | %d | %.2f | %.0f | %.3f | %.2f | %.0f | %.3f | %.2f | %.0f | %.2f | %.2f | %s | %s |" % (
            kind, b, S, u4, g4, g4 / HBM_PEAK_GBS, u2, g2, g2 / HBM_PEAK_GBS, us16, fp16_bytes / us16 / 1e3, us16 / u4,
            us16 / u2, ref_txt, ref_x), flush=True)
    return 0


def cpu_baseline(q, k, v, S, R, bits, gs, scale, budget_s=20.0):
    """Reference semantics on the host cores: the torch oracle (dequantize the packed cache to
    fp32, fp32 softmax attention over [packed || residual]) timed on the same inputs."""
    from oracle import torch_oracle as TO
    torch.set_num_threads(os.cpu_count() or 1)
    qkv = TO.quantize_kv(k[:, :S].float(), v[:, :S].float(), bits, gs, k.dtype)
    fn = lambda: TO.dequant_attend(q.float(), qkv, scale, k[:, S:].float(), v[:, S:].float())
    fn()
    times = []
    t_start = time.perf_counter()
    while len(times) < 3 or (time.perf_counter() - t_start < budget_s and len(times) < 50):
        t0 = time.perf_counter()
        out = fn()
        times.append(time.perf_counter() - t0)
    times.sort()
    return out, times[len(times) // 2], len(times)


def main():
    ap = argparse.ArgumentParser(description=__doc__)
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--workload", default=DEFAULT_WORKLOAD, choices=sorted(WORKLOADS))
    ap.add_argument("--num-splits", type=int, default=0)
    ap.add_argument("--no-graph", action="store_true", help="time eager launches instead of one HIP graph")
    ap.add_argument("--no-rotate", action="store_true", help="reuse one KV cache (stays in the 256 MB Infinity Cache)")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--no-fp16", action="store_true", help="skip the fp16-KV baseline leg")
    ap.add_argument("--no-qpack", action="store_true", help="skip the quantize-pack kernel leg")
    ap.add_argument("--no-step", action="store_true", help="skip the decode-step-with-append leg")
    ap.add_argument("--no-dropin", action="store_true", help="skip the eager drop-in call leg")
    ap.add_argument("--no-probe", action="store_true", help="skip the read-probe leg")
    ap.add_argument("--no-others", action="store_true", help="skip the compact timing of the other BASELINE shapes")
    ap.add_argument("--probe-sweep", action="store_true",
                    help="only sweep the read probe over launch shapes and sizes and print the table")
    ap.add_argument("--sweep", action="store_true",
                    help="only run the reference's sweep (one sequence, MHA 32 x 128, S = 1024 ... 524288, and batches "
                         "2 ... 64 at S = 4096; 4-bit, 2-bit and the library's fp16-KV path) and print the table")
    ap.add_argument("--calib-copy", action="store_true",
                    help="also launch three plain 256 MiB device copies (a kernel of known traffic, used to scale "
                         "the FETCH_SIZE / WRITE_SIZE counters of a rocprofv3 --pmc run)")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py measures one GPU: this decode path has no cross-GPU step (it shards by kv-head / batch "
              "with no exchange); run with --gpus 1", file=sys.stderr)
        return 2
    if not torch.cuda.is_available():
        print("bench.py needs a GPU", file=sys.stderr)
        return 2

    from bitladder_amd import kvcache_pack_int, plan_fwd_kvcache_int, plan_fwd_kvcache_int_append

    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    if args.probe_sweep:
        return probe_sweep(args)
    if args.sweep:
        return reference_sweep(args)
    b, h, h_k, S, R, bits, gs, dtype = WORKLOADS[args.workload]
    scale = 1.0 / math.sqrt(128)
    ragged = args.workload in RAGGED
    total_bytes, packed_bytes, packed_len, win_len = workload_bytes(args.workload)
    if ragged:
        packed_dev, win_dev = packed_len.to(dev), win_len.to(dev)

    W = build_workload(args.workload, args.num_splits, no_rotate=args.no_rotate, want_sources=not args.no_qpack,
                       cpu_inputs=True)
    nbuf, plans, keep, srcs = W["nbuf"], W["plans"], W["keep"], W["srcs"]
    q0, k0, v0 = W["first_inputs"]

    def step(i):
        plans[i % nbuf].run()

    if args.calib_copy:
        src = torch.ones(64 << 20, dtype=torch.float32, device=dev)
        dst = torch.empty_like(src)
        for _ in range(3):
            dst.copy_(src)
        torch.cuda.synchronize(dev)
        del src, dst

    # Whatever --steps is, the timed region holds at least MIN_TIMED_STEPS steps in graphs of at least
    # MIN_GRAPH_NODES steps, so the host synchronisation at its end and the gaps between graph launches
    # stay below 1 % of it; `steps` in the JSON line is the command line's value, `config` says what ran.
    T = time_steps(step, args.steps, args.warmup, not args.no_graph, quantile_reps=15)
    us_step, us_step_ev, graphed = T["wall_us"], T["event_us"], T["graphed"]
    achieved = total_bytes / (us_step_ev * 1e-6) / 1e9

    result = {
        "metric": "us/decode step (+ HBM GB/s, % of peak), Llama-3-8B GQA, 4-bit KV @32K ctx"
                  if args.workload.startswith("llama3-8b-gqa-32k") else f"us/decode step, {args.workload}",
        "value": round(us_step, 3),
        "unit": "us/step",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(us_step * 1e-3, 6),
        "higher_is_better": False,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f16" if dtype == torch.float16 else "bf16",
        "data": "synthetic: seeded N(0,1) q/k/v, 3 of 128 K channels per kv-head x10, packed by the library's own "
                "quantize-pack kernel",
        "config": {"workload": args.workload, "batch": b, "q_heads": h, "kv_heads": h_k, "head_dim": 128,
                   "packed_tokens": packed_len.tolist() if ragged else S,
                   "residual_tokens": win_len.tolist() if ragged else R, "bits": bits, "group_size": gs,
                   "num_splits": plans[0].num_splits, "kv_buffers_rotated": nbuf,
                   "launch": "hip-graph" if graphed else "eager",
                   "timed_steps": T["timed_steps"], "steps_per_graph": T["graph_nodes"],
                   "graph_replays_in_timed_region": T["replays"],
                   "untimed_graph_replays_before": T["untimed_replays"]},
        "roofline": {"bound": "hbm", "achieved": round(achieved, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": round(achieved / HBM_PEAK_GBS, 4),
                     "traffic": MEASURED_TRAFFIC_BYTES.get(args.workload) if args.num_splits == 0 else None,
                     "kernel": "fwd_splitkv_kernel", "algorithmic_bytes": total_bytes,
                     "packed_stream_bytes": packed_bytes, "us_per_step_events": round(us_step_ev, 3)},
    }
    if T["quantiles"]:
        result["us_per_step_quantiles"] = T["quantiles"]
    # (kept for the CPU leg's cross-check: the window-fill steps further down pack into the rotated caches)
    out_gpu_first = plans[0].run().float().cpu()

    if not args.no_probe:
        # what the memory system alone allows: kernels that only read as many bytes as one step streams (buffers
        # rotated like the caches), timed the same way; the fastest of a few launch shapes counts
        us_probe, probe_cfg, probe_all, probe_bytes = best_probe(total_bytes, args.steps, args.warmup, not args.no_graph, nbuf)
        result["roofline"]["read_kernel_us"] = us_probe
        result["roofline"]["read_kernel_GBs"] = round(probe_bytes / (us_probe * 1e-6) / 1e9, 1)
        result["roofline"]["read_kernel"] = probe_cfg
        result["roofline"]["read_kernels_tried_us"] = probe_all
        result["roofline"]["frac_of_read_kernel"] = round(us_probe / us_step_ev, 4)

    # the call a user of the reference makes: plain fwd_kvcache_int(...), eager launches, workspace from the
    # per-stream cache (nothing allocated or filled after the first call), output buffer passed in
    if not ragged and not args.no_dropin:
        from bitladder_amd import fwd_kvcache_int
        outs = [torch.empty_like(plans[i].out) for i in range(nbuf)]

        def dropin(i):
            j = i % nbuf
            c, kr, vr = keep[j]
            fwd_kvcache_int(plans[j]._keep[0], *c, None, scale, "k-channel", gs, bits, k_residual=kr, v_residual=vr,
                            num_splits=args.num_splits, out=outs[j])

        n_drop = max(50, args.steps)
        result["dropin_eager_us_per_call"] = round(time_steps(dropin, n_drop, 5, False, steady=False)["event_us"], 3)
        result["dropin_eager_note"] = ("fwd_kvcache_int(...) called %d times in a Python loop (eager launches), GPU "
                                       "time between first and last call / calls: the larger of the host's work "
                                       "per call and the kernel's time" % n_drop)
        assert torch.equal(outs[0], plans[0].run()), "drop-in call and plan disagree"

    if not args.no_qpack:
        # the other kernel of the path: quantize-pack of the whole packed prefix (prefill-side bulk pack)
        # and of one 128-token block per sequence (the append step of a decode loop); every call rewrites
        # a cache with the bytes it already holds
        def pack_all(i):
            j = i % len(srcs)
            kd, vd = srcs[j]
            c = keep[j][0]
            kvcache_pack_int(kd[:, :S], c[0], c[1], vd[:, :S], c[2], c[3], None, None, S, "k-channel", gs, bits)

        def pack_block(i):
            j = i % len(srcs)
            kd, vd = srcs[j]
            c = keep[j][0]
            if ragged:      # every sequence's next block, at its own position
                kvcache_pack_int(kd[:, S - 128:S], c[0], c[1], vd[:, S - 128:S], c[2], c[3], None, None, 128,
                                 "k-channel", gs, bits, dst_offsets=packed_dev)
            else:
                kvcache_pack_int(kd[:, S - 128:S], c[0], c[1], vd[:, S - 128:S], c[2], c[3], None, None, 128,
                                 "k-channel", gs, bits, dst_offset=S - 128)

        n_pack = max(10, args.steps // 4)
        us_pack = time_steps(pack_all, n_pack, 3, not args.no_graph)["event_us"]
        us_app = time_steps(pack_block, args.steps, args.warmup, not args.no_graph)["event_us"]
        rd = b * h_k * S * 128 * 2 * 2
        wr = int(b * h_k * S * 128 * 2 * (bits / 8 + 4 / gs))      # the whole capacity is packed
        gbs = (rd + wr) / (us_pack * 1e-6) / 1e9
        result["qpack"] = {
            "kernel": "qpack_kernel", "bound": "hbm", "tokens": S, "us_per_call": round(us_pack, 3),
            "bytes_read": rd, "bytes_written": wr, "achieved": round(gbs, 1), "peak": HBM_PEAK_GBS,
            "unit": "GB/s", "frac": round(gbs / HBM_PEAK_GBS, 4),
            "append_128_tokens_us_per_call": round(us_app, 3)}
        srcs.clear()

    if not args.no_step:
        # the same decode as one launch that also appends the step's new token (device-side lengths).  A slot
        # is one of the rotated packed caches with a window and a length counter of its own, S packed tokens + 64
        # in the window at the start of every graph replay (one small copy node in front of the steps resets the
        # counters), so that no window fills inside the measurement: a fill is a different, rarer step
        nodes = args.steps * max(1, math.ceil(MIN_GRAPH_NODES / args.steps))
        n_slots = max(nbuf, math.ceil((nodes + args.warmup + 1) / 59))
        start_len = (packed_dev + 64) if ragged else torch.full((b,), S + 64, device=dev)
        lengths_all = start_len.to(torch.int32).repeat(n_slots, 1).contiguous()
        lengths_init = lengths_all.clone()
        splans = []
        for i in range(n_slots):
            cache, kres, vres = keep[i % nbuf]
            q_t = torch.randn((b, 1, h, 128), device=dev).to(dtype)
            kn = torch.randn((b, 1, h_k, 128), device=dev).to(dtype)
            splans.append(plan_fwd_kvcache_int_append(q_t, kn, kn.clone(), *cache, kres.clone(), vres.clone(),
                                                      lengths_all[i], S + 127, None, scale, "k-channel", gs, bits,
                                                      num_splits=args.num_splits))
        us_append = time_steps(lambda i: splans[i % n_slots].run(), args.steps, args.warmup, not args.no_graph,
                               replay_prologue=lambda: lengths_all.copy_(lengths_init))["event_us"]
        result["decode_step_with_append"] = {
            "entry": "bitdecode_fwd_append", "us_per_step": round(us_append, 3),
            "window_tokens": "65-%d" % (64 + math.ceil((nodes + args.warmup + 1) / n_slots)), "does": "attend + store the new token + advance the device-side length"}
        del splans
        # the step that fills the window (one in 128): every slot starts one token short of a full window, so each
        # step of a replay attends, stores the token, quantize-packs the 128-token window behind the prefix and
        # advances the length; one slot per step of the graph (the slots share the rotated caches: their steps pack
        # the same block one after the other)
        f_slots = nodes
        fill_start = (packed_dev - 1) if ragged else torch.full((b,), S - 1, device=dev)
        fl_all = fill_start.to(torch.int32).repeat(f_slots, 1).contiguous()
        fl_init = fl_all.clone()
        fplans_ = []
        for i in range(f_slots):
            cache, kres, vres = keep[i % nbuf]
            q_t = torch.randn((b, 1, h, 128), device=dev).to(dtype)
            kn = torch.randn((b, 1, h_k, 128), device=dev).to(dtype)
            fplans_.append(plan_fwd_kvcache_int_append(q_t, kn, kn.clone(), *cache, kres[:, :128].clone(),
                                                       vres[:, :128].clone(), fl_all[i], S - 1, None, scale, "k-channel",
                                                       gs, bits, num_splits=args.num_splits))
        us_fill = time_steps(lambda i: fplans_[i % f_slots].run(), args.steps, min(args.warmup, 5), not args.no_graph,
                             replay_prologue=lambda: fl_all.copy_(fl_init))["event_us"]
        result["decode_step_with_append"]["fill_us_per_step"] = round(us_fill, 3)
        result["decode_step_with_append"]["fill_does"] = ("the same launch on the step that fills the 128-token window: "
                                                          "also quantize-packs it behind the prefix (packed prefix "
                                                          "128 tokens shorter, window 127 + the new token)")
        del fplans_

    if not args.no_fp16:
        # fp16-KV decode on the same GPU: the library's own fp16 split-KV path over all S+R tokens,
        # and torch SDPA for comparison
        fplans = []
        nb16 = 1 if args.no_rotate else max(2, min(8, math.ceil(320e6 / (b * h_k * (S + R) * 512))))
        dummy = alloc_cache(b, 128, h_k, bits, gs, dev)
        for i in range(nb16):
            q, k, v = make_inputs(b, h, h_k, S + R, seed=100 + i, dtype=dtype)
            kd, vd = k.to(dev), v.to(dev)
            kw16 = dict(residual_len=packed_dev + win_dev, max_residual_len=S + R) if ragged else {}
            fplans.append((plan_fwd_kvcache_int(q.to(dev), *dummy, None, scale, "k-channel", gs, bits, seqlen_k=0,
                                                k_residual=kd, v_residual=vd, **kw16), q.to(dev), kd, vd))
        torch.cuda.synchronize(dev)
        us16 = time_steps(lambda i: fplans[i % nb16][0].run(), args.steps, args.warmup, not args.no_graph)["event_us"]
        fp16_tokens = int((packed_len + win_len).sum()) if ragged else b * (S + R)
        fp16_bytes = fp16_tokens * h_k * 128 * 2 * 2 + 2 * b * h * 128 * 2

        def sdpa(i):
            _, qd, kd, vd = fplans[i % nb16]
            torch.nn.functional.scaled_dot_product_attention(
                qd.transpose(1, 2), kd.transpose(1, 2), vd.transpose(1, 2), scale=scale, enable_gqa=True)
        try:
            if ragged:
                raise RuntimeError("not run on a ragged batch (SDPA would attend the padding as well)")
            us_sdpa = time_steps(sdpa, max(10, args.steps // 4), 3, False, steady=False)["event_us"]
        except Exception as e:  # noqa: BLE001
            print(f"[bench] torch SDPA baseline failed: {e}", file=sys.stderr)
            us_sdpa = None
        result["fp16_kv_baseline"] = {
            "us_per_step": round(us16, 3), "GB/s": round(fp16_bytes / (us16 * 1e-6) / 1e9, 1),
            "kernel": "same library, fp16 split-KV path", "speedup_of_low_bit": round(us16 / us_step_ev, 3),
            "torch_sdpa_us_per_step": None if us_sdpa is None else round(us_sdpa, 3)}
        del fplans

    if not args.no_others and args.workload == DEFAULT_WORKLOAD and args.num_splits == 0 and not args.no_rotate:
        # the other BASELINE shapes, compactly: inputs generated on the GPU, same timing method, read probe beside
        others = {}
        for name in OTHER_CONFIGS:
            Wo = build_workload(name, 0, cpu_inputs=False, max_bufs=8)
            n_o, plans_o = Wo["nbuf"], Wo["plans"]
            us_o = time_steps(lambda i, n_o=n_o, plans_o=plans_o: plans_o[i % n_o].run(), args.steps, args.warmup,
                              not args.no_graph)["event_us"]
            entry = {"us_per_step": round(us_o, 3), "algorithmic_bytes": Wo["total_bytes"],
                     "GB/s": round(Wo["total_bytes"] / us_o / 1e3, 1),
                     "frac": round(Wo["total_bytes"] / us_o / 1e3 / HBM_PEAK_GBS, 4),
                     "num_splits": plans_o[0].num_splits, "kv_buffers_rotated": n_o}
            if not args.no_probe:
                up, cfg, _, _ = best_probe(Wo["total_bytes"], args.steps, args.warmup, not args.no_graph, n_o)
                entry["read_kernel_us"], entry["read_kernel"] = up, cfg
            others[name] = entry
            del Wo, plans_o
            torch.cuda.empty_cache()
        result["other_configs"] = others

    if not args.no_cpu and ragged:
        print("[bench] the CPU baseline leg runs on the uniform workloads only", file=sys.stderr)
    elif not args.no_cpu:
        out_cpu, t_cpu, reps = cpu_baseline(q0, k0, v0, S, R, bits, gs, scale)
        out_gpu = out_gpu_first
        result["cpu_baseline"] = {
            "value": round(t_cpu * 1e6, 1), "unit": "us/step", "cores": torch.get_num_threads(),
            "kind": "port",
            "sample": f"full {args.workload} decode step (dequantize to fp32 + fp32 attention incl. residual), "
                      f"median of {reps} runs, torch CPU ops on {torch.get_num_threads()} threads "
                      f"(os.cpu_count()={os.cpu_count()})",
            "max_abs_err_gpu_vs_cpu": float((out_gpu - out_cpu).abs().max())}

    print(json.dumps(result))
    return 0


if __name__ == "__main__":
    sys.exit(main())
