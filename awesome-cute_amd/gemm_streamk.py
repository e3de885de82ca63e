"""Counterpart of the reference's `gemm_streamk m n k` program
(gemm/streamk_gemm/gemm_streamk.cu:8-110): runs the dense fp16 GEMM with the
stream-K tail on uniform [-2, 2] inputs, times it, and checks the result against
the vendor library's GEMM by cosine similarity (the reference compares with
cuBLAS, include/reference.h:146-165; here torch.matmul, i.e. rocBLAS/hipBLASLt).

    python awesome-cute_amd/gemm_streamk.py 4096 4352 4096 [--repeat 200]

Prints the human-readable lines of the reference's program and one JSON line
with the roofline fraction against the dense fp16 MFMA peak."""
import argparse
import json
import os
import sys

import torch

sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))
import streamk  # noqa: E402

MFMA_FP16_PEAK_TFLOPS = 2500.0  # MI355X, dense


def _time_us(fn, repeat, stream):
    """Mean device time of `repeat` launches replayed from one HIP graph."""
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=stream):
        for _ in range(repeat):
            fn()
    graph.replay()
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    cur = torch.cuda.current_stream()
    e0.record(cur)
    graph.replay()
    e1.record(cur)
    torch.cuda.synchronize()
    return e0.elapsed_time(e1) * 1e3 / repeat


def run(m, n, k, repeat=200, warmup=5, seed=0, dev="cuda:0", log=print):
    gen = torch.Generator(device=dev)
    gen.manual_seed(seed)
    A = (torch.rand((m, k), device=dev, generator=gen) * 4 - 2).half()
    B = (torch.rand((n, k), device=dev, generator=gen) * 4 - 2).half()
    C = torch.empty((m, n), dtype=torch.half, device=dev)
    _, plan = streamk.plan(m, n, k, torch.cuda.get_device_properties(dev).multi_processor_count)
    log(f"fp16 gemm m:{m} n:{n} k:{k}")
    log(f"output tiles: {plan['dp_tiles'] + plan['sk_tiles']}, dp tiles: {plan['dp_tiles']}, "
        f"sk tiles: {plan['sk_tiles']} x {plan['k_slices']} slices, workgroups: {plan['grid']}")
    side = torch.cuda.Stream()
    with torch.cuda.stream(side):
        for _ in range(max(warmup, 1)):  # the first call on a stream allocates the scratch
            streamk.gemm(A, B, C)
            ref = torch.matmul(A, B.t())
        side.synchronize()
    us = _time_us(lambda: streamk.gemm(A, B, C), repeat, side)
    lib_us = _time_us(lambda: torch.matmul(A, B.t(), out=ref), repeat, side)
    flop = 2.0 * m * n * k
    # in double: fp32 sums over tens of millions of elements are off by more
    # than the margin above one
    cos = torch.nn.functional.cosine_similarity(C.double().flatten(), ref.double().flatten(), dim=0).item()
    ok = 0.999 <= cos <= 1.0 + 1e-6
    log(f"gemm_streamk: {flop / us * 1e-6:.1f} tflops, {us * 1e-3:.6f} ms latency")
    log(f"torch.matmul: {flop / lib_us * 1e-6:.1f} tflops, {lib_us * 1e-3:.6f} ms latency")
    log(("check ok" if ok else "check fail") + f", cos_similarity = {cos:.6f}")
    tf = flop / us * 1e-6
    return {
        "metric": "dense fp16 GEMM (TN) with stream-K tail, TFLOP/s", "value": tf, "unit": "TFLOP/s",
        "n_gpus": 1, "steps": repeat, "warmup": warmup, "ms_per_step": us * 1e-3,
        "higher_is_better": True, "dtype": "f16 (fp32 accumulate)", "data": "synthetic uniform [-2, 2]",
        "config": {"workload": f"gemm_streamk m={m} n={n} k={k}", **plan},
        "roofline": {"bound": "mfma", "achieved": tf, "peak": MFMA_FP16_PEAK_TFLOPS,
                     "unit": "TFLOP/s", "frac": tf / MFMA_FP16_PEAK_TFLOPS, "traffic": None},
        "vendor_library_tflops": flop / lib_us * 1e-6, "cos_similarity": cos, "check": ok,
    }


def main():
    ap = argparse.ArgumentParser(description=__doc__.split("\n")[0])
    ap.add_argument("m", type=int, nargs="?", default=4096)
    ap.add_argument("n", type=int, nargs="?", default=4352)
    ap.add_argument("k", type=int, nargs="?", default=4096)
    ap.add_argument("--repeat", type=int, default=200)
    args = ap.parse_args()
    if not torch.cuda.is_available():
        raise SystemExit("gemm_streamk needs a GPU")
    res = run(args.m, args.n, args.k, args.repeat)
    print(json.dumps(res))
    if not res["check"]:
        raise SystemExit(1)


if __name__ == "__main__":
    main()
