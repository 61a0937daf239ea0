#!/usr/bin/env python3
"""Benchmark of the int4 MatMulNBits hot path on one MI355X.

A step is one decode step's worth of MatMulNBits calls for a Qwen2.5-7B-shaped stack (28 layers of
qkv 3584->4608, o 3584->3584, gate/up 3584->37888, down 18944->3584, plus lm_head 3584->152064):
bf16 activations, block_size 128, packed 4-bit zero points, M rows (default 1). Every layer has its
own weight buffers (3.7 GB in all), so each step streams its weights from HBM. The calls of one step
are recorded once into a HIP graph through the provider's C ABI and replayed; the timed region is K
replays between two HIP events on the provider's stream.

Prints one JSON line: value = algorithmic GB/s of the whole step, plus `roofline` for the decode
kernel on the gate/up shape, `cpu_baseline` (the reference's MLAS path on this host's cores), and
`sweep` / `prefill` tables.
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

from onnx_genai_amd import ep as E  # noqa: E402
from onnx_genai_amd import synth  # noqa: E402

HBM_PEAK_GBS = 8000.0          # MI355X HBM3E, published
MFMA_F16_PEAK_TFLOPS = 2500.0  # MI355X dense fp16/bf16 MFMA, published
MFMA_I8_PEAK_TOPS = 5000.0     # MI355X dense int8 MFMA, published
MFMA_I8_PEAK_TOPS = 5000.0

LAYERS = 28
HIDDEN, INTER, VOCAB = 3584, 18944, 152064
LAYER_SHAPES = [("qkv", HIDDEN, 4608), ("o", HIDDEN, HIDDEN), ("gate_up", HIDDEN, 2 * INTER), ("down", INTER, HIDDEN)]
LM_HEAD = ("lm_head", HIDDEN, VOCAB)
BS = 128
A_DT = E.BF16


# HBM bytes one gate/up launch (M=1, repacked weights) moves come from two rocprofv3 counter runs of `bench.py --only-roofline`
# (FETCH_SIZE, then WRITE_SIZE, each scaled by what the same counter reads for the 256 MiB copy that run ends with).
# `bench.py --traffic-from <fetch csv> <write csv>` turns the two counter files into this tracked JSON; the benchmark line
# reports its figure only while the kernel variant it was taken on is still the one that runs.
TRAFFIC_JSON = os.path.join(ROOT, "profiles", "decode_gate_up_m1_traffic.txt")


def traffic_from_counters(fetch_csv, write_csv):
    """Reads two rocprofv3 `--pmc` counter files of `bench.py --only-roofline` and writes TRAFFIC_JSON."""
    import csv
    copy_bytes = 256 << 20

    def per_kernel(path, counter):
        by = {}
        for r in csv.DictReader(open(path)):
            if r["Counter_Name"] == counter:
                by.setdefault(r["Kernel_Name"], []).append(float(r["Counter_Value"]))
        return {k: sum(v) / len(v) for k, v in by.items()}, {k: len(v) for k, v in by.items()}

    fetch, n_fetch = per_kernel(fetch_csv, "FETCH_SIZE")
    write, _ = per_kernel(write_csv, "WRITE_SIZE")
    copy = next(k for k in fetch if "copy_kernel" in k)
    decode = max((k for k in fetch if "decode" in k and "pack_decode" not in k), key=lambda k: n_fetch[k])
    fetch_factor = (copy_bytes / 1024.0) / fetch[copy]
    write_factor = (copy_bytes / 1024.0) / write[copy]
    hbm = (fetch[decode] * fetch_factor + write[decode] * write_factor) * 1024.0
    out = {"kernel": decode, "workload": "gate_up 3584->37888, M=1, bf16, block 128, zero points, repacked weights",
           "fetch_size_kib_per_dispatch": round(fetch[decode], 1), "write_size_kib_per_dispatch": round(write[decode], 1),
           "copy_kernel_fetch_size_kib": round(fetch[copy], 1), "copy_kernel_write_size_kib": round(write[copy], 1),
           "fetch_scale": round(fetch_factor, 4), "write_scale": round(write_factor, 4), "dispatches": n_fetch[decode],
           "hbm_bytes_per_launch": int(round(hbm)),
           "commands": ["rocprofv3 --pmc FETCH_SIZE --output-format csv -d <dir> -o run -- python3 bench.py --only-roofline --steps 2 --warmup 1",
                        "rocprofv3 --pmc WRITE_SIZE --output-format csv -d <dir> -o run -- python3 bench.py --only-roofline --steps 2 --warmup 1",
                        "python3 bench.py --traffic-from <fetch run_counter_collection.csv> <write run_counter_collection.csv>"]}
    with open(TRAFFIC_JSON, "w") as f:
        json.dump(out, f, indent=1)
        f.write("\n")
    return out


def trace_summary(kernel_trace_csv):
    """Per kernel and launch shape of a rocprofv3 `--kernel-trace` file of this benchmark: launches, average and shortest
    duration, and the average distance from one launch's start to the next launch's start inside a graph replay (what a
    call costs the step, launch overhead included). No GPU work."""
    import collections
    import csv
    rows = sorted(csv.DictReader(open(kernel_trace_csv)), key=lambda r: int(r["Start_Timestamp"]))

    def key(r):
        grid = int(r.get("Grid_Size_X") or r.get("Grid_Size") or 0)
        wg = int(r.get("Workgroup_Size_X") or r.get("Workgroup_Size") or 0)
        return r["Kernel_Name"].split("(")[0][:90], grid // max(wg, 1), wg

    stats = collections.defaultdict(lambda: {"dur": [], "s2s": []})
    prev = None
    for r in rows:
        start, end = int(r["Start_Timestamp"]), int(r["End_Timestamp"])
        k = key(r)
        stats[k]["dur"].append(end - start)
        if prev is not None and start - prev[1] < 20000:          # the same replay
            stats[prev[2]]["s2s"].append(start - prev[0])
        prev = (start, end, k)
    out = []
    for (name, wgs, wg), v in sorted(stats.items(), key=lambda kv: -sum(kv[1]["dur"])):
        out.append({"kernel": name, "workgroups": wgs, "threads": wg, "launches": len(v["dur"]), "avg_ns": round(sum(v["dur"]) / len(v["dur"])),
                    "min_ns": min(v["dur"]), "avg_start_to_start_ns": round(sum(v["s2s"]) / len(v["s2s"])) if v["s2s"] else None})
    return out


def trace_spread(kernel_trace_csv, calls_per_layer=4, layers=LAYERS):
    """Where the spread of the decode step's launch durations comes from, out of a rocprofv3 `--kernel-trace` file of this
    benchmark's step (one graph replay = `layers` x `calls_per_layer` launches + lm_head, in that order). Per call of a layer:
    percentiles over all launches, and the spread split three ways - between layers (each layer has its own weight buffers:
    a spread that follows the buffer shows here), between replays (clock, temperature), and what is left inside a layer
    across replays. No GPU work."""
    import csv
    import numpy as np
    rows = sorted(csv.DictReader(open(kernel_trace_csv)), key=lambda r: int(r["Start_Timestamp"]))
    rows = [r for r in rows if "decode_packed_kernel" in r["Kernel_Name"] or "decode_wide_kernel" in r["Kernel_Name"]]
    wgs = lambda r: int(r["Grid_Size_X"]) // max(int(r["Workgroup_Size_X"]), 1)
    per_replay = layers * calls_per_layer + 1
    largest = max(wgs(r) for r in rows)
    ends = [i for i, r in enumerate(rows) if wgs(r) == largest and i >= per_replay - 1]
    replays = [rows[i - per_replay + 1:i + 1] for i in ends][2:]            # (without the eager pass and the first warm-up replay)
    dur = np.array([[int(r["End_Timestamp"]) - int(r["Start_Timestamp"]) for r in rep] for rep in replays], dtype=float) / 1e3
    out = []
    for j in range(calls_per_layer):
        sub = dur[:, [calls_per_layer * l + j for l in range(layers)]]        # [replay][layer]
        by_layer = sub.mean(axis=0)
        slow = np.argsort(by_layer)[::-1][:3]
        out.append({"call_of_layer": j, "workgroups": wgs(replays[0][j]), "launches": int(sub.size), "mean_us": round(float(sub.mean()), 2),
                    "min_us": round(float(sub.min()), 2), "p10_us": round(float(np.percentile(sub, 10)), 2), "p50_us": round(float(np.percentile(sub, 50)), 2),
                    "p90_us": round(float(np.percentile(sub, 90)), 2), "max_us": round(float(sub.max()), 2),
                    "mean_over_min": round(float(sub.mean() / sub.min()), 3),
                    "std_between_layers_us": round(float(by_layer.std()), 3), "std_between_replays_us": round(float(sub.mean(axis=1).std()), 3),
                    "std_inside_a_layer_us": round(float(sub.std(axis=0).mean()), 3),
                    "slowest_layers": [{"layer": int(l), "mean_us": round(float(by_layer[l]), 2)} for l in slow]})
    lm = dur[:, -1]
    out.append({"call_of_layer": "lm_head", "workgroups": largest, "launches": int(lm.size), "mean_us": round(float(lm.mean()), 2), "min_us": round(float(lm.min()), 2),
                "max_us": round(float(lm.max()), 2), "mean_over_min": round(float(lm.mean() / lm.min()), 3)})
    out.append({"replays": len(replays), "sum_of_means_us": round(float(dur.mean(axis=0).sum()), 1), "sum_of_minima_us": round(float(dur.min(axis=0).sum()), 1)})
    return out


def measured_traffic(kernel_template_hint):
    """HBM bytes per launch of the gate/up decode kernel from the tracked counter summary, or None when there is none
    or it was taken on another kernel."""
    try:
        with open(TRAFFIC_JSON) as f:
            t = json.load(f)
    except (OSError, ValueError):
        return None
    return t["hbm_bytes_per_launch"] if kernel_template_hint in t.get("kernel", "") else None


def _device_random_weights(ep, n, k, bs, seed, scale_lo, scale_hi, dtype, zero_points=True, reuse=None):
    """Packed nibbles, scales and zero points for one node, resident on the GPU. Random bytes ARE uniform
    nibbles; to keep set-up short the byte pattern of large tensors is generated once per shape and
    shifted per layer (the values do not affect timing, only the buffers must be distinct)."""
    kb = -(-k // bs)
    rng = np.random.default_rng(seed)
    if reuse is None:
        b = rng.integers(0, 256, size=(n, kb, bs // 2), dtype=np.uint8)
    else:
        b = np.roll(reuse, seed % 251 + 1, axis=0)
    scales = synth.to_dtype(rng.uniform(scale_lo, scale_hi, size=(n, kb)).astype(np.float32), dtype)
    zp = rng.integers(0, 256, size=(n, (kb + 1) // 2), dtype=np.uint8) if zero_points else None
    return b, scales, zp


class Node:
    def __init__(self, ep, name, k, n, bs, seed, a_dt, m, *, zero_points=True, scale_range=(0.002, 0.01), accuracy_level=0, reuse=None):
        self.name, self.k, self.n, self.bs, self.m, self.a_dt = name, k, n, bs, m, a_dt
        b, s, zp = _device_random_weights(ep, n, k, bs, seed, scale_range[0], scale_range[1], a_dt, zero_points, reuse)
        self.host_b = b
        self.ops = E.DeviceOperands(ep, b, s, a_dt, zp, n, k, bs, accuracy_level=accuracy_level, rows=m, a_dtype=a_dt)
        self.y = ep.allocate(m * n * 2)
        self.bytes = synth.algorithmic_bytes(m, n, k, bs, a_dtype=a_dt, scale_dtype=a_dt, zero_points=zero_points)
        self.flops = synth.matmul_flops(m, n, k)
        self.workspace = None
        if accuracy_level == 4:
            need, _ = self.ops.kernel.workspace_requirement([((m, k), a_dt)])
            self.workspace = ep.allocate(need)

    def run(self, a_buf):
        out = [E.TensorView(self.y.ptr, self.a_dt, (self.m, self.n), device_index=self.ops.ep.device_index)]
        self.ops.kernel.execute(self.ops.views(a_buf, self.a_dt, self.m), out, workspace=self.workspace)

    def free(self, ep):
        ep.deallocate(self.y)
        if self.workspace:
            ep.deallocate(self.workspace)
        self.ops.free()


def time_graph(ep, graph, reps, warmup):
    for _ in range(warmup):
        graph.replay()
    ep.sync()
    start, stop = ep.event(), ep.event()
    start.record()
    for _ in range(reps):
        graph.replay()
    stop.record()
    ms = start.elapsed_ms(stop)
    return ms / reps


def capture(ep, fn):
    ep.sync()
    ep.capture_begin()
    try:
        fn()
    finally:
        graph = ep.capture_end()
    return graph


def build_decode_stack(ep, m, layers):
    a_bufs = {k: ep.upload(synth.make_activation(m, k, 5, A_DT)) for k in (HIDDEN, INTER)}
    nodes, reuse = [], {}
    for layer in range(layers):
        for name, k, n in LAYER_SHAPES:
            node = Node(ep, f"{name}.{layer}", k, n, BS, 1000 * layer + len(nodes), A_DT, m, reuse=reuse.get(name))
            reuse.setdefault(name, node.host_b)
            node.host_b = None
            nodes.append(node)
    nodes.append(Node(ep, LM_HEAD[0], LM_HEAD[1], LM_HEAD[2], BS, 99, A_DT, m))
    nodes[-1].host_b = None
    return nodes, a_bufs


def small_model_step(ep):
    """configs[1]: the decode step of a Qwen2.5-0.5B-architecture stack (24 layers of q, k, v, o, gate, up, down plus
    lm_head; fp16, M=1, block 32, zero points), replayed as one HIP graph. Reported beside the headline workload."""
    hidden, inter, vocab, layers, kv = 896, 4864, 151936, 24, 128
    shapes = [("q", hidden, hidden), ("k", hidden, kv), ("v", hidden, kv), ("o", hidden, hidden),
              ("gate", hidden, inter), ("up", hidden, inter), ("down", inter, hidden)]
    a_bufs = {k: ep.upload(synth.make_activation(1, k, 6, E.F16)) for k in (hidden, inter)}
    nodes, reuse = [], {}
    for layer in range(layers):
        for name, k, n in shapes:
            node = Node(ep, f"{name}.{layer}", k, n, 32, 7000 + 10 * layer + len(nodes), E.F16, 1, reuse=reuse.get((k, n)))
            reuse.setdefault((k, n), node.host_b)
            node.host_b = None
            nodes.append(node)
    nodes.append(Node(ep, "lm_head", hidden, vocab, 32, 98, E.F16, 1))
    nodes[-1].host_b = None

    def one_step():
        for node in nodes:
            node.run(a_bufs[node.k])

    one_step()
    ep.sync()
    graph = capture(ep, one_step)
    ms = time_graph(ep, graph, 20, 3)
    graph.release()
    step_bytes = sum(n.bytes for n in nodes)
    out = {"workload": "Qwen2.5-0.5B decode-step MatMulNBits sweep (configs[1]): 24 layers x (q, k, v, o, gate, up, down) + lm_head, M=1, fp16, "
                       "block_size 32, zero points; %d calls per step" % len(nodes),
           "ms_per_step": round(ms, 4), "bytes_per_step": step_bytes, "gbs": round(step_bytes / (ms * 1e-3) / 1e9, 1),
           "hbm_frac": round(step_bytes / (ms * 1e-3) / 1e9 / HBM_PEAK_GBS, 4), "us_per_call": round(ms * 1e3 / len(nodes), 2),
           "kernel_variants": sorted({n.ops.kernel.last_variant() for n in nodes})}
    for node in nodes:
        node.free(ep)
    for buf in a_bufs.values():
        ep.deallocate(buf)
    return out


def swiglu_table(ep, copies=8):
    """The fused gate/up node at the 7B shape (3584 -> 2 x 18944, bf16, block 128, zero points): one launch that reads both
    projections and writes silu(gate) * up, over `copies` distinct weight pairs per graph; beside it the unfused pair as one
    MatMulNBits over the concatenated 37888 columns (which a model still follows with an elementwise kernel)."""
    k, n, bs, dt = HIDDEN, INTER, BS, A_DT
    table = []
    for m in (1, 4):
        a = ep.upload(synth.make_activation(m, k, 9, dt))
        fused, reuse = [], None
        for i in range(copies):
            gate = _device_random_weights(ep, n, k, bs, 300 + 2 * i, 0.002, 0.01, dt, True, reuse)
            reuse = gate[0] if reuse is None else reuse
            up = _device_random_weights(ep, n, k, bs, 301 + 2 * i, 0.002, 0.01, dt, True, reuse)
            ops = E.GateUpOperands(ep, gate, up, dt, n, k, bs)
            fused.append((ops, ep.allocate(m * n * 2)))
        for _ in range(2):                                  # the first call makes the repacked copies, the second is the single launch
            for ops, y in fused:
                ops.run(a, dt, m, y)
        ep.sync()
        variant = fused[0][0].kernel.last_variant()
        graph = capture(ep, lambda: [ops.run(a, dt, m, y) for ops, y in fused])
        us = time_graph(ep, graph, 20, 2) * 1e3 / copies
        graph.release()
        nbytes = 2 * synth.algorithmic_bytes(m, n, k, bs, a_dtype=dt, scale_dtype=dt, zero_points=True) - m * k * 2 - m * n * 2
        for ops, y in fused:
            ep.deallocate(y)
            ops.free()
        plain = [Node(ep, "gate_up.%d" % i, k, 2 * n, bs, 400 + i, dt, m) for i in range(copies)]
        for node in plain:
            node.run(a)
        ep.sync()
        graph = capture(ep, lambda: [node.run(a) for node in plain])
        plain_us = time_graph(ep, graph, 20, 2) * 1e3 / copies
        graph.release()
        for node in plain:
            node.free(ep)
        ep.deallocate(a)
        table.append({"k": k, "n": n, "m": m, "us": round(us, 2), "gbs": round(nbytes / us / 1e3, 1), "hbm_frac": round(nbytes / us / 1e3 / HBM_PEAK_GBS, 4),
                      "variant": variant, "unfused_matmul_us": round(plain_us, 2)})
    return table


def cpu_baseline(seconds_budget=20.0, threads=None):
    """The reference's CPU path (vendored MLAS through its plain-C shim, oracle/_ref) on this host, on a bounded
    sample of the workload: the gate/up projection (3584 -> 37888), bf16 activations widened to f32 before and
    the output narrowed after each call inside the timed region, weights packed once outside it."""
    import oracle
    from concurrent.futures import ThreadPoolExecutor
    if not oracle.Ref.available():
        return None
    ref, port = oracle.Ref(), oracle.Port()
    # the GPU box gives one job the CPU share of one GPU (16 hardware threads), whatever os.cpu_count() shows of the host
    threads = threads or min(16, os.cpu_count() or 1)
    k, n, m = HIDDEN, 2 * INTER, 1
    copies = 3                                         # 3 x 68 MB of packed weights: larger than the last-level cache
    shard = -(-n // threads)
    shard = (shard + 15) // 16 * 16
    packs = []
    for c in range(copies):
        b, s, zp = synth.make_weights(n, k, BS, 300 + c, zero_points=True, scale_lo=0.002, scale_hi=0.01, scale_dtype=A_DT)
        sf = synth.to_f32(s, A_DT)
        shards = []
        for lo in range(0, n, shard):
            hi = min(lo + shard, n)
            pk = ref.pack(b[lo:hi], sf[lo:hi], zp[lo:hi], hi - lo, k, BS, ref.COMP_FP32)
            if pk is None:
                return None
            pk["ws"] = ref.workspace(pk, m)
            pk["lo"], pk["hi"] = lo, hi
            shards.append(pk)
        whole = ref.pack(b, sf, zp, n, k, BS, ref.COMP_FP32)
        whole["ws"] = ref.workspace(whole, m)
        packs.append((shards, whole))
    a16 = synth.make_activation(m, k, 5, A_DT)
    nbytes = synth.algorithmic_bytes(m, n, k, BS, a_dtype=A_DT, scale_dtype=A_DT, zero_points=True)
    out = np.empty((m, n), np.float32)

    def one_thread(i):
        _, whole = packs[i % copies]
        a = port.widen(a16, A_DT)
        ref.gemm(whole, a, out=out, workspace=whole["ws"])
        return port.narrow(out, A_DT)

    pool = ThreadPoolExecutor(max_workers=threads)
    outs = [np.empty((m, pk["hi"] - pk["lo"]), np.float32) for pk in packs[0][0]]

    def all_threads(i):
        shards, _ = packs[i % copies]
        a = port.widen(a16, A_DT)
        list(pool.map(lambda t: ref.gemm(shards[t], a, out=outs[t], workspace=shards[t]["ws"]), range(len(shards))))
        return port.narrow(np.concatenate(outs, axis=1), A_DT)

    result = {}
    for label, fn in (("1", one_thread), (str(threads), all_threads)):
        for i in range(3):
            fn(i)
        t0, calls = time.perf_counter(), 0
        while time.perf_counter() - t0 < seconds_budget / 2:
            fn(calls)
            calls += 1
        dt = (time.perf_counter() - t0) / calls
        result[label] = {"gbs": nbytes / dt / 1e9, "us": dt * 1e6, "calls": calls}
    pool.shutdown()
    cpu_model, cpu_ids = "", {}
    try:
        with open("/proc/cpuinfo") as f:
            for line in f:
                key, _, value = line.partition(":")
                key = key.strip()
                if key == "model name" and not cpu_model:
                    cpu_model = value.strip()
                if key in ("cpu family", "model", "stepping", "cpu MHz") and key not in cpu_ids:
                    cpu_ids[key] = value.strip()
    except OSError:
        pass
    try:
        usable = len(os.sched_getaffinity(0))
    except (AttributeError, OSError):
        usable = os.cpu_count() or 1
    best = result[str(threads)]
    return {"value": round(best["gbs"], 2), "unit": "GB/s", "cores": threads, "kind": "reference",
            "sample": f"MLAS SQNBit CompFp32 (oracle/_ref), gate_up 3584->37888, M=1, bf16 in/out widened+narrowed in the timed region, "
                      f"block 128 with zero points, {best['calls']} calls rotating over {copies} weight copies, N-sharded over {threads} threads",
            "us_per_call": round(best["us"], 1), "single_thread_gbs": round(result["1"]["gbs"], 2),
            "dispatch": ref.dispatch_id(), "cpu": cpu_model, "cpu_ids": cpu_ids, "host_logical_cpus": os.cpu_count(), "usable_cpus": usable,
            "note": "cores = worker threads used: the CPU share a one-GPU job is given on this host (16), not every core of the machine"}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--m", type=int, default=1, help="rows of the decode batch (1..16)")
    ap.add_argument("--layers", type=int, default=LAYERS)
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--no-sweep", action="store_true", help="skip the per-shape sweep and the prefill table")
    ap.add_argument("--cpu-seconds", type=float, default=20.0)
    ap.add_argument("--only-roofline", action="store_true",
                    help="run only the roofline leg (decode kernel on the gate_up shape) and one 256 MiB device copy: the command profiles are taken from")
    ap.add_argument("--only-tables", action="store_true",
                    help="run only the prefill and accuracy_level=4 tables, one JSON line per row (the command their profiles are taken from)")
    ap.add_argument("--traffic-from", nargs=2, metavar=("FETCH_CSV", "WRITE_CSV"),
                    help="no GPU work: turn two rocprofv3 counter files of --only-roofline runs (FETCH_SIZE, WRITE_SIZE) into profiles/decode_gate_up_m1_traffic.txt")
    ap.add_argument("--trace-spread", metavar="KERNEL_TRACE_CSV",
                    help="no GPU work: per call of a layer, the percentiles of the step's launch durations in a rocprofv3 kernel trace and how their spread splits between layers, replays and the rest")
    ap.add_argument("--trace-summary", metavar="KERNEL_TRACE_CSV",
                    help="no GPU work: per kernel and launch shape of a rocprofv3 --kernel-trace file of this benchmark, one JSON line each")
    ap.add_argument("--lds-probe", action="store_true",
                    help="only measure what one CU's LDS moves per clock (reads, writes, global memory straight into LDS, mixed) and print one JSON line")
    ap.add_argument("--read-floor", action="store_true",
                    help="run only the yardstick: a plain read of each decode shape's bytes, one launch per layer buffer in a graph, beside the decode kernel's time on the same buffers")
    ap.add_argument("--row-sweep", action="store_true",
                    help="run only a sweep of the row count M across the dispatch boundaries (1 .. 2048), one JSON line per call shape")
    ap.add_argument("--model-sweep", action="store_true",
                    help="run only a sweep of decoder-model call shapes (Qwen2.5-7B / 0.5B, Llama-3-8B, Phi-3-mini projections) over 1 .. 16 rows, "
                         "block size 32 and 128, accuracy_level 0 and 4; one JSON line per shape and block size")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py: this build runs on one GPU only (no collectives exist on the MatMulNBits path); use --gpus 1")
    if args.traffic_from:
        print(json.dumps(traffic_from_counters(*args.traffic_from)), flush=True)
        return
    if args.trace_spread:
        for row in trace_spread(args.trace_spread, layers=args.layers):
            print(json.dumps(row), flush=True)
        return
    if args.trace_summary:
        for row in trace_summary(args.trace_summary):
            print(json.dumps(row), flush=True)
        return

    ep = E.RocmExecutionProvider(0)
    info = ep.device_info()
    if args.only_roofline:
        return roofline_only(ep, args)
    if args.lds_probe:
        names = {0: "ds_read_b128", 1: "ds_write_b128", 2: "buffer_load_dwordx4 ... lds", 3: "half the waves read, half write"}
        table = [{"access": names[mode], "waves_per_cu": waves, "bytes_per_clock_per_cu": round(ep.lds_probe(mode, waves), 1)}
                 for mode in (0, 1, 2, 3) for waves in (1, 4, 8, 16)]
        print(json.dumps({"lds_probe": table}))
        ep.shutdown()
        return
    if args.read_floor:
        for row in read_floor(ep, args):
            print(json.dumps(row), flush=True)
        return
    if args.row_sweep:
        for row in row_sweep(ep):
            print(json.dumps(row), flush=True)
        return
    if args.model_sweep:
        for row in model_sweep(ep):
            print(json.dumps(row), flush=True)
        return
    if args.only_tables:
        for row in prefill_table(ep) + prefill_7b_table(ep) + acc4_table(ep):
            print(json.dumps(row), flush=True)
        return
    nodes, a_bufs = build_decode_stack(ep, args.m, args.layers)
    step_bytes = sum(n.bytes for n in nodes)
    step_flops = sum(n.flops for n in nodes)

    def one_step():
        for node in nodes:
            node.run(a_bufs[node.k])

    one_step()                       # eager once: every kernel resolves its variant and reports errors here
    ep.sync()
    variants = sorted({n.ops.kernel.last_variant() for n in nodes})
    graph = capture(ep, one_step)
    for _ in range(args.warmup):
        graph.replay()
    ep.sync()
    start, stop = ep.event(), ep.event()
    t0 = time.perf_counter()
    start.record()
    for _ in range(args.steps):
        graph.replay()
    stop.record()
    ms_total = start.elapsed_ms(stop)
    ep.sync()
    wall_ms = (time.perf_counter() - t0) * 1e3
    ms_per_step = ms_total / args.steps
    value = step_bytes / (ms_per_step * 1e-3) / 1e9

    # roofline of the dominant kernel: decode GEMV on the gate/up shape (58% of the step's bytes), one launch
    # per layer buffer, recorded as a graph of `layers` launches and timed with events on the same stream.
    gate_up = [n for n in nodes if n.name.startswith("gate_up")]
    g2 = capture(ep, lambda: [n.run(a_bufs[n.k]) for n in gate_up])
    ms = time_graph(ep, g2, max(10, args.steps // 2), 3)
    launch_us = ms * 1e3 / len(gate_up)
    achieved = gate_up[0].bytes / (launch_us * 1e-6) / 1e9
    roofline = {"bound": "hbm", "kernel": "%s<bf16, block 128> on gate_up 3584->37888, M=%d" % (gate_up[0].ops.kernel.last_variant(), args.m),
                "achieved": round(achieved, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": round(achieved / HBM_PEAK_GBS, 4),
                "bytes_per_launch": gate_up[0].bytes, "us_per_launch": round(launch_us, 2),
                "traffic": measured_traffic("decode_packed_kernel") if args.m == 1 and gate_up[0].ops.kernel.last_variant() == "decode_mfma_packed" else None,
                "traffic_source": os.path.relpath(TRAFFIC_JSON, ROOT)}
    g2.release()

    result = {
        "metric": "int4 MatMulNBits decode GB/s (% HBM peak) + prefill TFLOPS, 7B shapes, 1 GPU",
        "value": round(value, 1), "unit": "GB/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 4), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "bf16", "data": "synthetic",
        "config": {"workload": f"Qwen2.5-7B decode-step MatMulNBits sweep (configs[2]): {args.layers} layers x (qkv, o, gate_up, down) + lm_head, "
                               f"M={args.m}, bf16, block_size 128, zero points; {len(nodes)} calls per step replayed as one HIP graph",
                   "m": args.m, "calls_per_step": len(nodes), "bytes_per_step": step_bytes, "flops_per_step": step_flops},
        "hbm_frac": round(value / HBM_PEAK_GBS, 4), "wall_ms_per_step": round(wall_ms / args.steps, 4),
        "kernel_variants": variants, "device": info, "roofline": roofline,
    }
    graph.release()

    if not args.no_sweep:
        result["sweep"] = sweep(ep, nodes, a_bufs, args)
    for node in nodes:
        node.free(ep)
    for buf in a_bufs.values():
        ep.deallocate(buf)
    if not args.no_sweep:
        result["prefill"] = prefill_table(ep)
        result["prefill_7b_bf16"] = prefill_7b_table(ep)
        result["acc4"] = acc4_table(ep)
        result["gate_up_swiglu"] = swiglu_table(ep)
        result["small_model_step"] = small_model_step(ep)
    ep.shutdown()
    if not args.no_cpu:
        result["cpu_baseline"] = cpu_baseline(args.cpu_seconds)
    print(json.dumps(result), flush=True)


def roofline_only(ep, args):
    """The decode kernel on the gate/up shape over `layers` distinct weight buffers, `steps` times, plus one plain
    256 MiB device copy whose byte counters calibrate FETCH_SIZE / WRITE_SIZE."""
    a = ep.upload(synth.make_activation(args.m, HIDDEN, 5, A_DT))
    nodes, reuse = [], None
    for layer in range(args.layers):
        node = Node(ep, f"gate_up.{layer}", HIDDEN, 2 * INTER, BS, layer, A_DT, args.m, reuse=reuse)
        reuse = node.host_b if reuse is None else reuse
        nodes.append(node)
    for node in nodes:               # eager once: constant weights are repacked here, never inside a capture
        node.run(a)
    ep.sync()
    graph = capture(ep, lambda: [n.run(a) for n in nodes])
    ms = time_graph(ep, graph, args.steps, args.warmup)
    us = ms * 1e3 / len(nodes)
    copy_bytes = 256 << 20
    src, dst = ep.allocate(copy_bytes), ep.allocate(copy_bytes)
    ep.copy(dst, src, copy_bytes)
    ep.sync()
    print(json.dumps({"kernel": nodes[0].ops.kernel.last_variant() + " on gate_up 3584->37888", "m": args.m, "launches": len(nodes) * (args.steps + args.warmup) + 1,
                      "us_per_launch": round(us, 2), "bytes_per_launch": nodes[0].bytes, "achieved_gbs": round(nodes[0].bytes / us / 1e3, 1),
                      "copy_kernel_bytes_read": copy_bytes, "copy_kernel_bytes_written": copy_bytes}), flush=True)


def read_floor(ep, args):
    """What the chain of dependent launches allows at best: for every decode shape, `layers` launches of a kernel that only
    reads the shape's algorithmic bytes (distinct buffers, one HIP graph, the same timing as the decode sweep), beside the
    decode kernel itself over its own `layers` weight buffers. A launch that does nothing but read cannot be beaten, so
    `floor_us` bounds the shape's share of the step; the step's bound is their sum."""
    rows, a_bufs = [], {k: ep.upload(synth.make_activation(args.m, k, 5, A_DT)) for k in (HIDDEN, INTER)}
    for name, k, n in LAYER_SHAPES + [LM_HEAD]:
        copies = args.layers if name != LM_HEAD[0] else 3
        nodes, reuse = [], None
        for i in range(copies):
            node = Node(ep, f"{name}.{i}", k, n, BS, 50 + i, A_DT, args.m, reuse=reuse)
            reuse = node.host_b if reuse is None else reuse
            nodes.append(node)
        for node in nodes:
            node.run(a_bufs[k])
        ep.sync()
        graph = capture(ep, lambda: [node.run(a_bufs[k]) for node in nodes])
        kernel_us = time_graph(ep, graph, args.steps, args.warmup) * 1e3 / copies
        graph.release()
        nbytes = nodes[0].bytes
        bufs = [ep.allocate(nbytes) for _ in range(copies)]
        for b in bufs:
            ep.read_probe(b, nbytes)
        ep.sync()
        graph = capture(ep, lambda: [ep.read_probe(b, nbytes) for b in bufs])
        floor_us = time_graph(ep, graph, args.steps, args.warmup) * 1e3 / copies
        graph.release()
        rows.append({"shape": name, "k": k, "n": n, "m": args.m, "bytes": nbytes, "launches_per_graph": copies, "read_only_us": round(floor_us, 2),
                     "read_only_gbs": round(nbytes / floor_us / 1e3, 1), "decode_kernel_us": round(kernel_us, 2), "decode_over_read_only": round(kernel_us / floor_us, 3),
                     "variant": nodes[0].ops.kernel.last_variant()})
        for b in bufs:
            ep.deallocate(b)
        for node in nodes:
            node.free(ep)
    per_layer = [r for r in rows if r["shape"] != LM_HEAD[0]]
    lm = rows[-1]
    step_floor = args.layers * sum(r["read_only_us"] for r in per_layer) + lm["read_only_us"]
    step_now = args.layers * sum(r["decode_kernel_us"] for r in per_layer) + lm["decode_kernel_us"]
    step_bytes = args.layers * sum(r["bytes"] for r in per_layer) + lm["bytes"]
    rows.append({"step": "%d layers + lm_head" % args.layers, "bytes": step_bytes, "read_only_us": round(step_floor, 1), "read_only_gbs": round(step_bytes / step_floor / 1e3, 1),
                 "read_only_hbm_frac": round(step_bytes / step_floor / 1e3 / HBM_PEAK_GBS, 4), "decode_kernels_us": round(step_now, 1),
                 "decode_hbm_frac": round(step_bytes / step_now / 1e3 / HBM_PEAK_GBS, 4)})
    return rows


def sweep(ep, nodes, a_bufs, args):
    """Per-shape decode figures at M in {1, 4, 8, 16}: the launches of one shape across all layer buffers in one graph."""
    table = []
    by_shape = {}
    for n in nodes:
        by_shape.setdefault(n.name.split(".")[0], []).append(n)
    # A shape with one buffer in the stack (lm_head) gets two more over distinct device memory for this table: replaying
    # one 290 MB buffer would let the 256 MB last-level cache serve part of it.
    extra = []
    for shape, group in by_shape.items():
        while len(group) < 3:
            first = group[0]
            clone = Node(ep, "%s.copy%d" % (shape, len(group)), first.k, first.n, BS, 7000 + len(group), A_DT, first.m)
            clone.host_b = None
            group.append(clone)
            extra.append(clone)
    for m in (1, 4, 8, 16):
        a_m = {k: ep.upload(synth.make_activation(m, k, 6, A_DT)) for k in (HIDDEN, INTER)}
        for shape, group in by_shape.items():
            saved = [(g.m, g.y) for g in group]
            for g in group:
                g.m = m
                g.y = ep.allocate(m * g.n * 2)
            for g in group:
                g.run(a_m[g.k])                    # first call of a kernel object: repacks its weights (never under capture)
            ep.sync()
            graph = capture(ep, lambda: [g.run(a_m[g.k]) for g in group])
            ms = time_graph(ep, graph, 20, 3)
            graph.release()
            us = ms * 1e3 / len(group)
            nbytes = synth.algorithmic_bytes(m, group[0].n, group[0].k, BS, a_dtype=A_DT, scale_dtype=A_DT, zero_points=True)
            table.append({"shape": shape, "k": group[0].k, "n": group[0].n, "m": m, "us": round(us, 2),
                          "gbs": round(nbytes / (us * 1e-6) / 1e9, 1), "hbm_frac": round(nbytes / (us * 1e-6) / 1e9 / HBM_PEAK_GBS, 4),
                          "variant": group[0].ops.kernel.last_variant()})
            for g, (m0, y0) in zip(group, saved):
                ep.deallocate(g.y)
                g.m, g.y = m0, y0
        for buf in a_m.values():
            ep.deallocate(buf)
    for clone in extra:
        clone.free(ep)
    return table


ROW_SWEEP_ROWS = (1, 2, 4, 5, 8, 16, 17, 24, 32, 33, 48, 64, 65, 128, 256, 512, 1023, 1024, 2048)
ROW_SWEEP_SHAPES = (   # block size, K, N, accuracy_level
    (128, 4096, 14336, 0), (32, 4096, 14336, 0), (64, 4096, 14336, 0), (128, 3584, 37888, 0), (32, 3584, 37888, 0), (64, 3584, 37888, 0),
    (128, 4096, 14336, 4), (32, 4096, 14336, 4),
)


def row_sweep(ep):
    """Time per call against the row count M, bf16 with zero points, on the default dispatch: each step in the table should
    cost no more than the rows it adds (a step that does marks a kernel boundary placed at the wrong M). Per graph four
    copies of the weights up to 64 rows (with two, the graph's own launch cost shows in a 10 us call and the figures
    scatter by 10-30 %), two above; replayed after a warm-up."""
    out = []
    for bs, k, n, acc in ROW_SWEEP_SHAPES:
        shape_rows = []
        for m in reversed(ROW_SWEEP_ROWS):      # tallest first: the short calls then follow light work, not 2048-row GEMMs
            nodes = [Node(ep, f"w{i}", k, n, bs, i, E.BF16, m, accuracy_level=acc) for i in range(4 if m <= 64 else 2)]
            a = ep.upload(synth.make_activation(m, k, 5, E.BF16))
            for nd in nodes:
                nd.run(a)
            ep.sync()
            graph = capture(ep, lambda: [nd.run(a) for nd in nodes])
            ms = time_graph(ep, graph, 20, 20) / len(nodes)
            shape_rows.append({"block_size": bs, "k": k, "n": n, "accuracy_level": acc, "m": m, "us": round(ms * 1e3, 1),
                        "tflops": round(nodes[0].flops / ms / 1e9, 1), "gbs": round(nodes[0].bytes / ms / 1e6, 1),
                        "variant": nodes[0].ops.kernel.last_variant()})
            for nd in nodes:
                nd.free(ep)
            ep.deallocate(a)
        out += reversed(shape_rows)
    return out


MODEL_SWEEP_SHAPES = (   # name, K, N
    ("qwen2.5-7b qkv", 3584, 4608), ("qwen2.5-7b o", 3584, 3584), ("qwen2.5-7b gate/up", 3584, 37888), ("qwen2.5-7b down", 18944, 3584),
    ("qwen2.5-7b lm_head", 3584, 152064),
    ("llama-3-8b qkv", 4096, 6144), ("llama-3-8b o", 4096, 4096), ("llama-3-8b gate/up", 4096, 28672), ("llama-3-8b gate", 4096, 14336),
    ("llama-3-8b down", 14336, 4096), ("llama-3-8b lm_head", 4096, 128256),
    ("qwen2.5-0.5b q", 896, 896), ("qwen2.5-0.5b gate/up", 896, 4864), ("qwen2.5-0.5b down", 4864, 896), ("qwen2.5-0.5b lm_head", 896, 151936),
    ("phi-3-mini qkv", 3072, 9216), ("phi-3-mini o", 3072, 3072), ("phi-3-mini gate/up", 3072, 16384), ("phi-3-mini down", 8192, 3072),
    ("phi-3-mini lm_head", 3072, 32064),
    ("qwen2.5-14b gate", 5120, 13824), ("qwen2.5-14b down", 13824, 5120),
)
MODEL_SWEEP_ROWS = (1, 2, 4, 5, 8, 16)


def model_sweep(ep):
    """Time per call (us) of decoder-model projections at 1 .. 16 rows, bf16 with zero points, block size 32 and 128, float and
    accuracy_level = 4, on the default dispatch: the table that calls costing more than a taller or coarser-blocked neighbour
    are read off. Per graph as many weight copies as 600 MB hold (2 .. 8), replayed after a warm-up."""
    out = []
    for acc in (0, 4):
        for name, k, n in MODEL_SWEEP_SHAPES:
            for bs in (32, 128):
                wbytes = n * k // 2 + n * (k // bs) * 2 + n * ((k // bs + 1) // 2)
                copies = max(2, min(8, int(600e6 // wbytes)))
                us = {}
                for m in MODEL_SWEEP_ROWS:
                    nodes = [Node(ep, f"w{i}", k, n, bs, i, E.BF16, m, accuracy_level=acc) for i in range(copies)]
                    a = ep.upload(synth.make_activation(m, k, 5, E.BF16))
                    for nd in nodes:
                        nd.run(a)
                    ep.sync()
                    graph = capture(ep, lambda: [nd.run(a) for nd in nodes])
                    us[m] = round(time_graph(ep, graph, 10, 3) / len(nodes) * 1e3, 2)
                    variant = nodes[0].ops.kernel.last_variant()
                    graph.release()
                    for nd in nodes:
                        nd.free(ep)
                    ep.deallocate(a)
                out.append({"accuracy_level": acc, "shape": name, "k": k, "n": n, "block_size": bs, "us": us,
                            "gbs_one_row": round(wbytes / us[1] / 1e3, 0), "variant_16_rows": variant})
    return out


def prefill_routes(ep):
    """The ways a tall 16-bit call can run, each as its own provider: the default dispatch (this provider's own tiled
    kernel at every height); and, for comparison, the two opt-in forms of the dense route - weights expanded into one
    shared 16-bit buffer per call and then the library GEMM (from 1024 rows), or constant weights keeping a resident
    16-bit copy (the call is the library GEMM alone)."""
    return [("default", ep, False), ("library_transient", E.RocmExecutionProvider(0, {"dense_gemm_min_rows": "1024"}), True),
            ("library_resident", E.RocmExecutionProvider(0, {"dense_weights": "resident"}), True)]


def prefill_table(ep, shapes=((4096, 14336), (14336, 4096)), rows=(512, 2048, 8192), dtype=E.F16, bs=32, zero_points=False):
    """Prefill GEMM. Defaults: Llama-3-8B MLP shapes (configs[3]): fp16, block 32, no zero points. One row per route
    that runs a different kernel sequence for the shape."""
    table = []
    routes = prefill_routes(ep)
    for k, n in shapes:
        for m in rows:
            seen = set()
            for route, provider, _ in routes:
                node = Node(provider, "prefill", k, n, bs, 7, dtype, m, zero_points=zero_points, scale_range=(0.001, 0.01))
                a = provider.upload(synth.make_activation(m, k, 8, dtype))
                node.run(a)
                provider.sync()
                variant = node.ops.kernel.last_variant()
                tall = variant.startswith("prefill") or variant.startswith("dense")
                if variant not in seen and (tall or m <= 512):   # the catch-all kernel is not a prefill path: one row of the table is enough
                    seen.add(variant)
                    graph = capture(provider, lambda: node.run(a))
                    ms = time_graph(provider, graph, 10 if tall else 1, 1)
                    graph.release()
                    tflops = node.flops / (ms * 1e-3) / 1e12
                    table.append({"k": k, "n": n, "m": m, "route": route, "us": round(ms * 1e3, 1), "tflops": round(tflops, 1),
                                  "mfma_frac": round(tflops / MFMA_F16_PEAK_TFLOPS, 4), "variant": variant})
                provider.deallocate(a)
                node.free(provider)
    for _, provider, owned in routes:
        if owned:
            provider.shutdown()
    return table


def prefill_7b_table(ep):
    """The same routes at the Qwen2.5-7B shapes of the decode sweep: bf16, block 128, zero points, M = 4096."""
    return prefill_table(ep, shapes=((3584, 37888), (18944, 3584)), rows=(4096,), dtype=E.BF16, bs=128, zero_points=True)


def acc4_table(ep):
    """accuracy_level=4 at 70B-class shapes (configs[4]): fp16, block 64, zero points, M in {1, 256, 4096}. Each call is
    the activation quantizer plus the int8 MFMA kernel. M=1 rows are priced against HBM, the others against int8 MFMA."""
    table = []
    for k, n in ((8192, 28672), (28672, 8192), (8192, 10240)):
        for m in (1, 256, 4096):
            # One-row calls take tens of microseconds: eight calls over distinct weight buffers per graph, so that the
            # replay's own launch cost does not drown them (the decode step and the roofline leg do the same).
            copies = 8 if m == 1 else 1
            nodes, reuse = [], None
            for i in range(copies):
                node = Node(ep, "acc4.%d" % i, k, n, 64, 9 + i, E.F16, m, accuracy_level=4, reuse=reuse)
                reuse = node.host_b if reuse is None else reuse
                nodes.append(node)
            a = ep.upload(synth.make_activation(m, k, 8, E.F16))
            for node in nodes:
                node.run(a)
            ep.sync()
            graph = capture(ep, lambda: [node.run(a) for node in nodes])
            ms = time_graph(ep, graph, 20 if m == 1 else 3, 2 if m == 1 else 1) / copies
            graph.release()
            node = nodes[0]
            row = {"k": k, "n": n, "m": m, "us": round(ms * 1e3, 1), "variant": node.ops.kernel.last_variant()}
            if m == 1:
                row["gbs"] = round(node.bytes / (ms * 1e-3) / 1e9, 1)
                row["hbm_frac"] = round(node.bytes / (ms * 1e-3) / 1e9 / HBM_PEAK_GBS, 4)
            else:
                row["tops"] = round(node.flops / (ms * 1e-3) / 1e12, 1)
                row["mfma_i8_frac"] = round(node.flops / (ms * 1e-3) / 1e12 / MFMA_I8_PEAK_TOPS, 4)
            table.append(row)
            ep.deallocate(a)
            for node in nodes:
                node.free(ep)
    return table


if __name__ == "__main__":
    main()
