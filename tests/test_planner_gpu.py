"""Guard of the host's kernel choice (marlin_host.hip: make_plan): on two
dozen shapes from the decode to the prefill regime, the planned launch must not
be more than 10 % slower than the best of the forced alternatives -- the
streaming kernel, the prefill kernel on 64-row tiles and on 128-row tiles, each
with the slice count its cost model picks, and for at most 1024 rows the
column-strip kernel with 1 to 4 strips per workgroup (for at most 16 rows
instead of the prefill kernel).  The planner is a fitted cost model;
this test is what fails when a kernel change shifts the costs under it.  (The
dispatch rules it replaces: reference marlin_cute_kernel.cu:39-49.)
"""
import os
import sys

import pytest

pytestmark = pytest.mark.gpu

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
sys.path.insert(0, os.path.join(ROOT, "awesome-cute_amd"))

SHAPES = [(m, n, k) for (n, k) in [(4096, 4096), (4096, 11008), (8192, 8192)]
          for m in (48, 64, 128, 512)]
SHAPES += [(m, n, k) for (n, k) in [(4096, 4096), (11008, 4096), (4096, 11008), (2048, 2048),
                                    (8192, 8192), (1024, 8192)]
           for m in (1, 16)]
# more rows over small weights: column strips, the rows in parts of 16, while the
# parts fill the compute units at most twice
SHAPES += [(32, 1024, 1024), (64, 512, 1024), (32, 2048, 2048), (33, 512, 2048), (32, 2048, 4096),
           (64, 512, 4096), (48, 1024, 4096), (64, 8192, 4096), (128, 512, 1024), (128, 2048, 2048),
           (96, 4096, 2048), (256, 1024, 1024), (1024, 256, 512), (512, 512, 2048)]
SLACK = 1.10


@pytest.fixture(scope="module")
def env():
    import torch
    import marlin
    assert torch.cuda.is_available()
    return torch, marlin


def _us_per_call(torch, fn, reps):
    """fastest of five replays of a HIP graph of `reps` back-to-back calls (launches of a
    few microseconds each are bound by the host when they are issued one by one)"""
    side = torch.cuda.Stream()
    with torch.cuda.stream(side):
        for _ in range(3):
            fn()  # also allocates this stream's scratch, which a capture cannot
        side.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=side):
            for _ in range(reps):
                fn()
        graph.replay()
        side.synchronize()
        best = float("inf")
        for _ in range(5):
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record(side)
            graph.replay()
            e1.record(side)
            side.synchronize()
            best = min(best, e0.elapsed_time(e1) * 1e3 / reps)
    del graph
    return best


def _measure(torch, marlin, m, n, k):
    dev = torch.device("cuda:0")
    # enough distinct weight buffers that the stream comes from HBM, as in bench.py
    nbuf = max(2, min(24, (600 << 20) // (k * n // 2)))
    Bs = [torch.randint(-2**31, 2**31 - 1, (k // 16, 2 * n), dtype=torch.int32, device=dev)
          for _ in range(nbuf)]
    S = (torch.rand((k // 128, n), device=dev) * 0.019 + 0.001).half()
    A = torch.randn((m, k), device=dev).half()
    C = torch.zeros((m, n), dtype=torch.half, device=dev)
    ws = torch.zeros(n // 128 * 16, dtype=torch.int, device=dev)
    turn = [0]

    def call():
        turn[0] += 1
        marlin.mul(A, Bs[turn[0] % nbuf], C, S, ws)

    times = {}
    try:
        times["planned"] = _us_per_call(torch, call, 40)
        marlin.force_kernel(1)
        times["streaming"] = _us_per_call(torch, call, 40)
        if m <= 1024:
            for strips in (1, 2, 3, 4):
                marlin.force_kernel(3)
                marlin.force_strips(strips)
                times[f"column strips, {strips} per workgroup"] = _us_per_call(torch, call, 40)
        if m > 16:
            for rows in (64, 128):
                marlin.force_kernel(2)
                marlin.force_tile_rows(rows)
                times[f"prefill, {rows}-row tiles"] = _us_per_call(torch, call, 40)
    finally:
        marlin.force_kernel(0)
        marlin.force_tile_rows(0)
        marlin.force_strips(0)
    torch.cuda.synchronize()
    assert not ws.any().item()
    return times


@pytest.mark.parametrize("m,n,k", SHAPES)
def test_planned_launch_is_within_ten_percent_of_the_best_alternative(env, m, n, k):
    torch, marlin = env
    print(f"  planner guard m={m} n={n} k={k} plan={marlin.plan(m, n, k, 128)[1]}", flush=True)
    for attempt in range(3):  # re-measured twice at most: timings of 15-60 us launches scatter by a few %
        t = _measure(torch, marlin, m, n, k)
        best = min(v for name, v in t.items() if name != "planned")
        if t["planned"] <= SLACK * best:
            return
    raise AssertionError(f"m={m} n={n} k={k}: planned {t['planned']:.1f} us, alternatives {t}")
