#!/usr/bin/env python3
"""Benchmark of the W4A16 Marlin GEMM hot path on one MI355X.

A step is one GEMM call (marlin.mul -> C ABI -> HIP kernel) on synthetic,
seeded inputs already resident in HBM.  Memory-bound shapes rotate over enough
distinct weight/scale buffers to exceed the 256 MB Infinity Cache, so the
figure is an HBM figure and not a cache figure.  The timed steps are captured in HIP
graphs (kernel launches only) and bracketed by HIP events on the launch stream,
so the host's launch cost is not part of the kernel's number: a graph holds a
whole number of K-step runs, at least 200 launches (the hand-over between two
graphs costs the GPU about 8 us, which is not the kernel's either), and is
replayed until at least 50 ms of GPU time and 20 replays have been timed (when
one graph does not cover the rotated weight buffers, several that continue the
rotation take turns); `ms_per_step` is the median sample, the spread is
reported beside it.  The eager (one host call per step) rate is
reported next to it.

Prints ONE JSON line: the headline workload is the decode configuration (
M=1, N=K=4096, group 128), with `roofline` for its kernel and `cpu_baseline`
from the CPU oracle; `shapes` carries the other points of the metric
(M=16 and M=2048 at N=K=4096) and the MLP-pair and 64-row configurations, measured the same
way.
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.join(ROOT, "awesome-cute_amd"))
sys.path.insert(0, os.path.join(ROOT, "tests"))

HBM_PEAK_GBPS = 8000.0      # MI355X HBM3E, published
MFMA_FP16_PEAK_TFLOPS = 2500.0  # MI355X dense fp16 MFMA, published
MALL_BYTES = 256 << 20

SHAPES = {
    # name: (M, N, K, groupsize, bound)
    "decode": (1, 4096, 4096, 128, "hbm"),          # the configuration the metric is quoted on
    "batch16": (16, 4096, 4096, 128, "hbm"),        # metric's M=16 point
    "prefill": (2048, 4096, 4096, 128, "mfma"),     # the MFMA-bound configuration
    "mlp_up": (16, 11008, 4096, 128, "hbm"),        # configs[2]
    "mlp_down": (16, 4096, 11008, 128, "hbm"),
    "large_g128": (64, 28672, 8192, 128, "hbm"),    # configs[4]
    "large_chan": (64, 28672, 8192, -1, "hbm"),
    # not one of the benchmark's configurations: the decode kernel where the
    # launch and exchange latencies are small beside the weight stream
    "decode_large": (1, 28672, 8192, 128, "hbm"),
    # the row counts between the benchmark's configurations, N = K = 4096 (reported
    # under "m_sweep": which kernel the host picks and what it costs)
    "m32": (32, 4096, 4096, 128, "hbm"),
    "m64": (64, 4096, 4096, 128, "hbm"),
    "m128": (128, 4096, 4096, 128, "hbm"),
    "m256": (256, 4096, 4096, 128, "mfma"),
    "m512": (512, 4096, 4096, 128, "mfma"),
    "m1024": (1024, 4096, 4096, 128, "mfma"),
}
M_SWEEP = ["m32", "m64", "m128", "m256", "m512", "m1024"]

# HBM bytes per launch (read + written) measured with rocprofv3 --pmc FETCH_SIZE /
# WRITE_SIZE (KiB per dispatch) and scaled by what the same counters read for a
# 256 MiB device copy (FETCH_SIZE x 2.0, WRITE_SIZE x 1.0 on this pool); the
# summaries, with the commands, are under profiles/.  Each entry names the plan
# it was measured on (kernel, grid): when the library plans the shape otherwise
# the figure is stale and is reported as null.
MEASURED_TRAFFIC_BYTES = {
    "decode": (("strips", 256), int((4284.5 * 2.0 + 8.0) * 1024)),            # 8.78 MB, 1.01 x algorithmic
    "batch16": (("strips", 256), int((4770.0 * 2.0 + 128.0) * 1024)),         # 9.90 MB, 1.11 x (the rows read by every workgroup)
    "prefill": (("prefill", 256), int((33941.5 * 2.0 + 16389.5) * 1024)),     # 86.3 MB, 2.04 x (A and B read by 16 tiles each)
    "mlp_up": (("strips", 230), int((11930.9 * 2.0 + 356.0) * 1024)),         # 24.8 MB, 1.04 x
    "mlp_down": (("stream", 256), int((13714.5 * 2.0 + 2185.0) * 1024)),      # 30.3 MB, 1.28 x
    "large_g128": (("prefill", 224), int((66886.0 * 2.0 + 17930.5) * 1024)),  # 155.3 MB, 1.23 x
    "large_chan": (("prefill", 224), int((65121.5 * 2.0 + 17930.5) * 1024)),  # 151.7 MB, 1.24 x
    "decode_large": (("stream", 224), int((59281.0 * 2.0 + 56.0) * 1024)),    # 121.5 MB, 1.00 x
}


def algorithmic_bytes(M, N, K, g):
    """weights + scales + activations + result, the bytes one GEMM has to move"""
    return K * N // 2 + 2 * (K // 128 if g != -1 else 1) * N + 2 * M * K + 2 * M * N


def sig(x, n=4):
    """floats rounded to n significant digits (the printed line stays short)"""
    if isinstance(x, float):
        return float(f"{x:.{n}g}")
    if isinstance(x, dict):
        return {k: sig(v, n) for k, v in x.items()}
    if isinstance(x, (list, tuple)):
        return [sig(v, n) for v in x]
    return x


def build_inputs(torch, O, M, N, K, groupsize, nbuf, seed=0):
    import numpy as np
    dev = torch.device("cuda:0")
    A, q, s, B, sp = O.make_problem(M, N, K, groupsize, seed)
    dA = torch.from_numpy(A).to(dev)
    dBs, dSs = [], []
    rng = np.random.default_rng(seed + 1)
    hB = torch.from_numpy(B)
    hS = torch.from_numpy(sp)
    for i in range(nbuf):
        if i == 0:
            dBs.append(hB.to(dev))
            dSs.append(hS.to(dev))
        else:
            # distinct memory with the same value distribution: a row rotation
            # of the packed buffers (uniform nibbles stay uniform)
            dBs.append(torch.roll(dBs[0], shifts=i, dims=0).contiguous())
            dSs.append(torch.roll(dSs[0], shifts=i, dims=1).contiguous())
    dC = torch.zeros((M, N), dtype=torch.half, device=dev)
    ws = torch.zeros(N // 128 * 16, dtype=torch.int, device=dev)
    return (A, B, sp), dA, dBs, dSs, dC, ws


def graph_ms(torch, side, fn, steps, period):
    """Median time (ms) of one step, calls fn(i), over replays of HIP graphs.

    A graph holds a whole number of K-step runs, at least 200 launches: the
    hand-over from one graph to the next costs the GPU about 8 us, which a
    graph of 20 launches would spread over them as 0.4 us each (an empty
    kernel: 1.94 us per launch in graphs of 20, 1.54 us in graphs of 200 or
    2000), and that is the runtime's cost, not the kernel's.  i runs on from
    graph to graph, so `period` distinct buffers are all visited.  Returns
    (median, (min, max, samples))."""
    per_graph = steps * max(1, -(-200 // steps))
    n_graphs = max(1, min(8, -(-period // per_graph)))
    graphs = []
    for g in range(n_graphs):
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=side):
            for i in range(per_graph):
                fn(g * per_graph + i)
        graphs.append(graph)
    cur = torch.cuda.current_stream()
    for g in graphs:  # untimed: uploads the graph, brings the clocks up
        g.replay()
    torch.cuda.synchronize()
    times, total, r = [], 0.0, 0
    while (total < 50.0 or r < 20 or len(times) < 15) and r < 20000:
        batch = []
        for _ in range(5):
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record(cur)
            graphs[r % n_graphs].replay()
            r += 1
            e1.record(cur)
            batch.append((e0, e1))
        torch.cuda.synchronize()
        for e0, e1 in batch:
            t = e0.elapsed_time(e1)
            times.append(t / per_graph)
            total += t
    times.sort()
    return times[len(times) // 2], (times[0], times[-1], len(times))


def time_shape(torch, marlin, O, name, steps, warmup, check=True, with_floor=False):
    M, N, K, g, bound = SHAPES[name]
    weight_bytes = K * N // 2
    nbuf = max(2, -(-2 * MALL_BYTES // weight_bytes)) if bound == "hbm" else 2
    nbuf = min(nbuf, 96)
    host, dA, dBs, dSs, dC, ws = build_inputs(torch, O, M, N, K, g, nbuf)

    def call(i):
        marlin.mul(dA, dBs[i % nbuf], dC, dSs[i % nbuf], ws)

    side = torch.cuda.Stream()
    with torch.cuda.stream(side):
        for i in range(max(warmup, 3)):
            call(i)
        side.synchronize()
        if check:
            import numpy as np
            call(0)
            side.synchronize()
            A, B, sp = host
            rows = slice(0, min(M, 4))
            ref = O.gemm(A[rows], B, sp, N, g)
            r = O.compare(dC[rows].cpu().numpy(), ref)
            assert r.max_abs_err <= 1e-2 * r.max_abs_ref, (name, r.max_abs_err, r.max_abs_ref)
            assert not ws.any().item()
        # eager: one host call per step
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        side.synchronize()
        t0 = time.perf_counter()
        e0.record(side)
        for i in range(steps):
            call(i)
        e1.record(side)
        side.synchronize()
        eager_ms = (time.perf_counter() - t0) * 1e3 / steps
        eager_dev_ms = e0.elapsed_time(e1) / steps

    ms, spread = graph_ms(torch, side, call, steps, nbuf)
    # the same launches over one weight buffer, which then stays in the 256 MB
    # Infinity Cache / L2: the figure kernel timings on other hardware usually are
    resident_ms = (graph_ms(torch, side, lambda i: call(0), steps, 1)[0]
                   if bound == "hbm" and nbuf > 1 else None)
    floor = None
    if with_floor and bound == "hbm":
        # what the launch alone and the weight stream alone cost, measured the same way
        e_ms, _ = graph_ms(torch, side, lambda i: marlin.probe(0, dBs[0], N, K, M), steps, 1)
        r_ms, r_spread = graph_ms(torch, side, lambda i: marlin.probe(1, dBs[i % nbuf], N, K, M),
                                  steps, nbuf)
        floor = {"empty_kernel_us": e_ms * 1e3, "read_kernel_us": r_ms * 1e3,
                 "read_kernel_spread_us": [x * 1e3 for x in r_spread[:2]],
                 "read_GBps": weight_bytes / (r_ms * 1e-3) / 1e9,
                 "what": "same grid and work split as the kernel planned for this launch (for 16 "
                         "rows where that is the prefill kernel); read kernel = the packed weights "
                         "through that kernel's 128-bit loads, no arithmetic, nothing written; same "
                         "buffer rotation and graph timing"}
    elif with_floor:
        # what the matrix pipes sustain on the same count of multiply-adds with
        # nothing beside them (one workgroup of 8 waves per CU, N*K/8192 MFMAs
        # of 16384 flop per wave: the work of 2048 rows, scaled to M)
        cus = marlin.device_info(0)["compute_units"]
        per_wave = (N * K // 8192) // 32 * 32
        probe_flops = cus * 8 * per_wave * 16384.0
        m_ms, m_spread = graph_ms(torch, side, lambda i: marlin.probe(2, dBs[0], N, K), steps, 1)
        sustained = probe_flops / (m_ms * 1e-3) / 1e12
        floor = {"mfma_only_us": m_ms * 1e3, "mfma_only_flop": probe_flops,
                 "sustained_TFLOPs": sustained,
                 "what": "a loop of nothing but v_mfma_f32_16x16x32_f16 on pseudo-random operands, "
                         "8 waves per CU with 32 independent accumulators each, same graph timing"}

    flops = 2.0 * M * N * K
    res = {
        "name": name, "M": M, "N": N, "K": K, "groupsize": g,
        "ms_per_step": ms, "us_per_launch": ms * 1e3,
        "us_per_launch_min_max": [spread[0] * 1e3, spread[1] * 1e3], "graph_replays": spread[2],
        "stream_floor": floor,
        "eager_ms_per_step": eager_ms, "eager_device_ms_per_step": eager_dev_ms,
        "weight_GBps": weight_bytes / (ms * 1e-3) / 1e9,
        "tflops": flops / (ms * 1e-3) / 1e12,
        "weight_buffers_rotated": nbuf,
        "cache_resident_us_per_launch": None if resident_ms is None else resident_ms * 1e3,
    }
    rc, plan = marlin.plan(M, N, K, g, -1, -1, -1, marlin.device_info(0)["compute_units"])
    kernel = {1: "stream", 2: "prefill", 3: "strips"}.get(plan["kernel"])
    res["plan"] = {"kernel": kernel, "grid": plan["grid"], "k_slices": plan["k_slices"],
                   "tile_rows": plan["tile_rows"]}
    measured_on, traffic = MEASURED_TRAFFIC_BYTES.get(name, (None, None))
    if measured_on != (kernel, plan["grid"]):
        traffic = None  # measured on another plan: stale
    if bound == "hbm":
        ach = res["weight_GBps"]
        res["roofline"] = {"bound": "hbm", "achieved": ach, "peak": HBM_PEAK_GBPS, "unit": "GB/s",
                           "frac": ach / HBM_PEAK_GBPS, "traffic": traffic}
        if floor:
            # the floor: a plain read of the same weights, launch included
            res["roofline"]["floor_us"] = floor["read_kernel_us"]
            res["roofline"]["frac_of_floor"] = floor["read_kernel_us"] / (ms * 1e3)
    else:
        ach = res["tflops"]
        res["roofline"] = {"bound": "mfma", "achieved": ach, "peak": MFMA_FP16_PEAK_TFLOPS,
                           "unit": "TFLOP/s", "frac": ach / MFMA_FP16_PEAK_TFLOPS,
                           "traffic": traffic}
        if floor:
            # the floor: the same multiply-adds with nothing beside them
            scaled = floor["mfma_only_us"] * flops / floor["mfma_only_flop"]
            res["roofline"]["floor_us"] = scaled
            res["roofline"]["frac_of_floor"] = scaled / (ms * 1e3)
            res["roofline"]["sustained_peak"] = floor["sustained_TFLOPs"]
    res["roofline"]["algorithmic_bytes"] = algorithmic_bytes(M, N, K, g)
    return res


def cpu_baseline(O, name, budget_s=12.0):
    """The CPU oracle (a port: the reference has no CPU implementation of this
    path) on the same workload, repeated until about budget_s of CPU time."""
    M, N, K, g, _ = SHAPES[name]
    A, q, s, B, sp = O.make_problem(M, N, K, g, 0)
    threads = O.lib.w4a16_ref_max_threads()
    O.gemm(A, B, sp, N, g)  # warm
    reps, t0 = 0, time.perf_counter()
    while True:
        O.gemm(A, B, sp, N, g)
        reps += 1
        dt = time.perf_counter() - t0
        if dt >= budget_s or reps >= 200:
            break
    per = dt / reps
    # the same on one core, a few repetitions
    reps1, t1 = 0, time.perf_counter()
    while reps1 < 3 or (time.perf_counter() - t1 < 3.0 and reps1 < 20):
        O.gemm(A, B, sp, N, g, threads=1)
        reps1 += 1
    per1 = (time.perf_counter() - t1) / reps1
    return {"value": (K * N // 2) / per / 1e9, "unit": "GB/s", "cores": threads, "kind": "port",
            "sample": f"{reps} {name} GEMMs (whole), {per * 1e3:.1f} ms each",
            "tflops": 2.0 * M * N * K / per / 1e12,
            "one_core": {"value": (K * N // 2) / per1 / 1e9, "unit": "GB/s", "cores": 1,
                         "sample": f"{reps1} GEMMs, {per1 * 1e3:.1f} ms each"}}


def compact_row(r):
    """one configuration in the printed line: shape [M, N, K, group], time,
    fraction of the published peak of its roofline (HBM unless "b" says mfma),
    the floor (a plain read of the weights, or the same MFMAs alone) and the
    time's share of it, workgroups, HBM traffic over algorithmic bytes"""
    rf = r["roofline"]
    row = {"n": r["name"], "shape": [r["M"], r["N"], r["K"], r["groupsize"]],
           "us": r["us_per_launch"], "frac": rf["frac"], "floor_us": rf.get("floor_us"),
           "of_floor": rf.get("frac_of_floor"), "grid": r["plan"]["grid"]}
    if rf["bound"] != "hbm":
        row["b"] = rf["bound"]
    if rf.get("traffic"):
        row["traffic_x"] = rf["traffic"] / rf["algorithmic_bytes"]
    return row


def hardware_facts(torch, marlin):
    """The figures of this board that shaped the kernels, each from a probe kernel of the
    probe library (libmarlin_amd_probe.so); shader cycles are the wave's own counter."""
    clock_ghz = marlin.device_info()["clock_khz"] / 1e6
    print(f"device clock {clock_ghz:.2f} GHz (nominal); one workgroup of four waves per CU, "
          "32 independent v_mfma_f32_16x16x32_f16 per turn")
    print("cycles per MFMA of a lone wave per SIMD that also issues ...")
    base = marlin.probe_issue(0)
    rows = [("nothing else", (0, 0, 0)), ("1 packed-fp16 VALU per MFMA", (1, 0, 0)),
            ("2 VALU per MFMA", (2, 0, 0)), ("3 VALU per MFMA", (3, 0, 0)),
            ("4 VALU per MFMA", (4, 0, 0)), ("1 ds_read_b128 per 8 MFMAs", (0, 1, 0)),
            ("2 ds_read_b128 per 8 MFMAs", (0, 2, 0)), ("1 global 16-byte load per 8 MFMAs", (0, 0, 1)),
            ("2 global loads per 8 MFMAs", (0, 0, 2)),
            ("2 VALU per MFMA and 1 ds_read_b128 per 8", (2, 1, 0)),
            ("2 VALU per MFMA and 1 global load per 8", (2, 0, 1))]
    for label, (nv, nl, ng) in rows:
        c = marlin.probe_issue(nv, nl, ng)
        extra = ""
        if nl + ng and nv == 0:
            extra = f"  ({(c - base) * 8 / (nl + ng):.1f} cycles per memory instruction)"
        elif nv and not (nl + ng):
            extra = f"  ({(c - base) / nv:.1f} cycles per VALU operation beyond the MFMA's own time)"
        print(f"  {label:45s} {c:6.2f}{extra}")
    print("what compute units pull from memory (16-byte loads per thread, 256 threads a workgroup; "
          "slowest workgroup, by the kernel's 100 MHz clock):")
    src = torch.empty(1 << 30, dtype=torch.uint8, device="cuda")
    src.random_(0, 255)
    cus = marlin.device_info()["compute_units"]
    for wgs, per_wg in ((1, 16 << 20), (cus, 4 << 20)):
        for depth in (1, 4, 16):
            us = marlin.probe_pull(src, per_wg, depth, wgs)
            gbps = per_wg * wgs / (float(us.max()) * 1e-6) / 1e9
            print(f"  {wgs:4d} workgroup(s) x {per_wg >> 20} MiB, {depth:2d} loads in flight per thread: "
                  f"{gbps / wgs:7.1f} GB/s per CU, {gbps:8.0f} GB/s together")


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=2000)
    ap.add_argument("--warmup", type=int, default=50)
    ap.add_argument("--shape", default="headline",
                    help="headline (decode, then the other benchmark shapes) or one of: " +
                         ", ".join(SHAPES))
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--kernel", type=int, default=0,
                    help="0 (default) = the library's own choice of kernel; 1 streaming, 2 prefill, "
                         "3 column strips, 4 = by cost without the column strips "
                         "(marlin_amd_force_kernel): to time or profile an alternative; such a "
                         "run is not the benchmark")
    ap.add_argument("--extras", action="store_true",
                    help="also time the sibling dense fp16 GEMM (reported with the details)")
    ap.add_argument("--copy-calibration", action="store_true",
                    help="also run a plain 256 MiB device copy (reference point for the "
                         "FETCH_SIZE / WRITE_SIZE counters of a rocprofv3 --pmc run)")
    ap.add_argument("--facts", action="store_true",
                    help="instead of the benchmark: the hardware figures the design leans on, "
                         "measured by the probe library (what one wave issues beside its MFMAs, "
                         "what compute units pull from memory); a table on stdout")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py: this path runs on one GPU; --gpus must be 1 "
                 "(sharding over several GPUs is not built)")

    import torch
    import marlin
    import _oracle as O
    if not torch.cuda.is_available():
        sys.exit("bench.py: no GPU visible")

    if args.facts:
        hardware_facts(torch, marlin)
        return
    if args.kernel:
        marlin.force_kernel(args.kernel)

    if args.shape == "headline":
        main_name, others = "decode", ["prefill", "batch16", "mlp_up", "mlp_down", "large_g128",
                                        "large_chan", "decode_large"]
    else:
        main_name, others = args.shape, []

    def steps_for(name):
        # keep the captured graph and the run time bounded for the big shapes
        M, N, K, g, _ = SHAPES[name]
        gflop = 2.0 * M * N * K / 1e9
        cap = 2000 if gflop < 2 else 400
        return max(1, min(args.steps, cap)) if name != main_name else args.steps

    if args.copy_calibration:
        src = torch.empty(256 << 20, dtype=torch.uint8, device="cuda:0").random_(0, 255)
        dst = torch.empty_like(src)
        for _ in range(3):
            dst.copy_(src)
        torch.cuda.synchronize()
        del src, dst

    prop = torch.cuda.get_device_properties(0)
    info = marlin.device_info(0)  # from the HIP runtime, through the C ABI
    # cross-check of the published matrix peak: CUs x 4 SIMDs x 1024 fp16 flop per clock x clock.
    # (The published 8000 GB/s is 8192 pins x 8 Gb/s; the memory clock the runtime reports is
    # printed as it is, no rate is derived from it.)
    clock_hz = info["clock_khz"] * 1e3
    peaks = {"hbm_GBps": HBM_PEAK_GBPS, "mfma_fp16_TFLOPs": MFMA_FP16_PEAK_TFLOPS,
             "device": prop.name, "compute_units": info["compute_units"],
             "clock_MHz": info["clock_khz"] / 1e3,
             "mfma_fp16_TFLOPs_from_clock": info["compute_units"] * 4 * 1024 * clock_hz / 1e12,
             "memory_clock_MHz": info["memory_clock_khz"] / 1e3,
             "memory_bus_bits": info["bus_width_bits"]}
    head = time_shape(torch, marlin, O, main_name, args.steps, args.warmup, with_floor=True)
    shapes = [time_shape(torch, marlin, O, n, steps_for(n), args.warmup, with_floor=True)
              for n in others]
    for r in [head] + shapes:
        if "sustained_peak" in r["roofline"]:
            peaks["mfma_fp16_TFLOPs_sustained"] = r["roofline"]["sustained_peak"]

    M, N, K, g, bound = SHAPES[main_name]
    # The printed line: the contract's fields, the headline's roofline (with its
    # floor), the CPU baseline, and one short row per configuration -- short
    # enough to survive whole wherever only the end of the output is kept.  The
    # long form (spreads, eager rates, floors' parts, row-count sweep) goes to
    # stderr before it.
    out = {
        "metric": "w4a16_gemm_weight_hbm_GBps" if bound == "hbm" else "w4a16_gemm_tflops",
        "value": head["weight_GBps"] if bound == "hbm" else head["tflops"],
        "unit": "GB/s" if bound == "hbm" else "TFLOP/s",
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": head["ms_per_step"],
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "f16", "data": "synthetic",
        "config": {"workload": f"{main_name}: M={M} N={N} K={K} groupsize={g} W4A16 GEMM"},
        "roofline": head["roofline"],
    }
    details = {"headline": head, "shapes": shapes, "peaks": peaks,
               "timing": "HIP graphs of a whole number of K-step runs (>= 200 launches), replayed "
                         "for >= 50 ms and >= 20 replays, HIP events around each replay, median",
               "reference_published": {"RTX4090_marlin_cute_us": 8.714,
                                       "shape": "M=1 N=4096 K=4096 g=128",
                                       "note": "cache-warm kernel time on other hardware, "
                                               "not comparable"}}
    if args.shape == "headline":
        sweep = []
        for n in M_SWEEP:
            r = time_shape(torch, marlin, O, n, min(args.steps, 400), args.warmup)
            sweep.append({"M": r["M"], "N": r["N"], "K": r["K"], "groupsize": r["groupsize"],
                          "us_per_launch": r["us_per_launch"], "weight_GBps": r["weight_GBps"],
                          "tflops": r["tflops"], **r["plan"]})
        details["m_sweep"] = sweep
        # (decode_large is not one of the benchmark's configurations: details only)
        out["rows"] = [compact_row(r) for r in [head] + shapes if r["name"] != "decode_large"]
        out["m_sweep_us"] = {str(r["M"]): r["us_per_launch"] for r in sweep}
        out["peaks"] = {"hbm_GBps": HBM_PEAK_GBPS, "mfma_TFLOPs": MFMA_FP16_PEAK_TFLOPS,
                        "mfma_sustained_TFLOPs": peaks.get("mfma_fp16_TFLOPs_sustained")}
    if args.extras:
        # the sibling dense fp16 GEMM with its stream-K tail, on the reference's three
        # examples (gemm/readme.md:29-31) and one problem small enough for 128 x 128
        # tiles; its own program is gemm_streamk.py
        import gemm_streamk
        details["dense_streamk"] = [
            {k: v for k, v in gemm_streamk.run(m, n, k, repeat=50, log=lambda *_: None).items()
             if k in ("value", "unit", "ms_per_step", "config", "roofline", "vendor_library_tflops",
                      "cos_similarity", "check")}
            for (m, n, k) in [(4096, 4352, 4096), (4096, 4352, 10240), (1152, 4352, 4096),
                              (2048, 2048, 2048)]]
    if not args.no_cpu:
        cpu = cpu_baseline(O, main_name)
        details["cpu_baseline"] = cpu
        out["cpu_baseline"] = {k: cpu[k] for k in ("value", "unit", "cores", "kind", "sample")}
    print(json.dumps(sig(details)), file=sys.stderr)
    # a table of the rows last on stderr, for whoever reads only its end
    for r in [head] + shapes:
        rf = r["roofline"]
        print(f"{r['name']:12s} M={r['M']:<5d} N={r['N']:<6d} K={r['K']:<6d} g={r['groupsize']:<4d}"
              f"{r['us_per_launch']:8.2f} us  {rf['frac']:.3f} of {rf['bound']} peak"
              + (f"  floor {rf['floor_us']:.2f} us ({rf['frac_of_floor']:.2f})"
                 if rf.get("floor_us") else ""), file=sys.stderr)
    sys.stderr.flush()
    print(json.dumps(sig(out)))


if __name__ == "__main__":
    main()
