"""GPU test of marlin_gemm_static, the entry point that allocates nothing: its
partial sums and tile counters live in a fixed array inside the library's
device image.  Called through the C ABI and compared, bit for bit, with
marlin_gemm (the same plan gives the same summation order), on two calls in a
row, the second with a smaller input; then on shapes that exercise every kind
of exchange (shared column tiles, straddling runs, prefill k slices), the
oracle's tolerance, the size limit's error and a HIP graph of it.
"""
import os
import sys

import numpy as np
import pytest

import _oracle as O

pytestmark = pytest.mark.gpu

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
sys.path.insert(0, os.path.join(ROOT, "awesome-cute_amd"))

TOL = 1e-2


@pytest.fixture(scope="module")
def env():
    import torch
    import marlin
    assert torch.cuda.is_available()
    return torch, marlin


@pytest.fixture(autouse=True)
def no_strips(env):
    """This file is about the scratch: few rows go through the streaming
    kernel, which exchanges partial sums, not through the column strips, which
    the planner would pick for them and which use no scratch at all."""
    torch, marlin = env
    marlin.force_kernel(4)
    yield
    marlin.force_kernel(0)


def both(env, M, N, K, g, seed, sms=-1):
    """marlin_gemm_static and marlin_gemm on the same device buffers."""
    torch, marlin = env
    dev = torch.device("cuda:0")
    A, q, s, B, sp = O.make_problem(M, N, K, g, seed)
    dA, dB, ds = (torch.from_numpy(x).to(dev) for x in (A, B, sp))
    outs = []
    for entry in ("marlin_gemm_static", "marlin_gemm"):
        dC = torch.full((M, N), 3.0, dtype=torch.half, device=dev)
        ws = torch.zeros(N // 128 * 16, dtype=torch.int, device=dev)
        torch.cuda.synchronize()
        print(f"  {entry} M={M} N={N} K={K} g={g} sms={sms}", flush=True)
        rc = marlin.gemm_raw(entry, dA, dB, dC, ds, ws, g, sms=sms)
        assert rc == 0, marlin.last_error()
        torch.cuda.synchronize()
        assert not ws.any().item()
        outs.append(dC.cpu().numpy())
    return (A, B, sp), outs[0], outs[1]


def test_two_calls_in_a_row_second_smaller(env):
    torch, marlin = env
    before = marlin.scratch_bytes()
    # both exchange partial sums through the scratch: 8 workgroups per column tile
    (A, B, sp), c_static, c_pool = both(env, 16, 4096, 4096, 128, seed=1)
    assert np.array_equal(c_static.view(np.uint16), c_pool.view(np.uint16))
    r = O.compare(c_static, O.gemm(A, B, sp, 4096, 128))
    assert r.max_abs_err <= TOL * r.max_abs_ref
    (A, B, sp), c_static, c_pool = both(env, 3, 1024, 2048, 128, seed=2)
    assert np.array_equal(c_static.view(np.uint16), c_pool.view(np.uint16))
    r = O.compare(c_static, O.gemm(A, B, sp, 1024, 128))
    assert r.max_abs_err <= TOL * r.max_abs_ref
    # the static entry itself left the pool alone (marlin_gemm added one buffer at most)
    after = marlin.scratch_bytes()
    assert after[1] <= before[1] + 1


@pytest.mark.parametrize("M,N,K,g,sms", [
    (1, 4096, 4096, 128, -1),      # decode: every tile shared by 8 workgroups
    (16, 1280, 1152, -1, 7),       # runs that straddle tile boundaries
    (48, 768, 2048, 128, 100),     # LDS-ring variant, shared tiles
    (64, 4096, 4096, 128, -1),
    (256, 4096, 4096, 128, -1),    # prefill kernel, 64-row tiles in k slices
    (1024, 4096, 4096, -1, -1),    # prefill kernel, 128-row tiles in 2 slices: 32 MiB, the limit
    (2048, 1024, 1024, 128, -1),   # no exchange at all
])
def test_static_matches_pool_entry(env, M, N, K, g, sms):
    torch, marlin = env
    (A, B, sp), c_static, c_pool = both(env, M, N, K, g, seed=M + N, sms=sms)
    assert np.array_equal(c_static.view(np.uint16), c_pool.view(np.uint16))
    rows = slice(0, min(M, 8))
    r = O.compare(c_static[rows], O.gemm(A[rows], B, sp, N, g))
    assert r.max_abs_err <= TOL * r.max_abs_ref


def test_static_entry_through_column_strips(env):
    """The planner's own choice for few rows over small weights: no scratch on
    either entry, the same bits."""
    torch, marlin = env
    marlin.force_kernel(0)
    assert marlin.plan(1, 4096, 4096, 128)[1]["kernel"] == 3
    (A, B, sp), c_static, c_pool = both(env, 1, 4096, 4096, 128, seed=77)
    assert np.array_equal(c_static.view(np.uint16), c_pool.view(np.uint16))
    r = O.compare(c_static, O.gemm(A, B, sp, 4096, 128))
    assert r.max_abs_err <= TOL * r.max_abs_ref
    # ... and for more rows in parts of 16 (here seven, the last with four rows)
    p = marlin.plan(100, 1024, 1024, -1)[1]
    assert (p["kernel"], p["row_parts"], p["partial_kib"]) == (3, 7, 0)
    (A, B, sp), c_static, c_pool = both(env, 100, 1024, 1024, -1, seed=78)
    assert np.array_equal(c_static.view(np.uint16), c_pool.view(np.uint16))
    r = O.compare(c_static, O.gemm(A, B, sp, 1024, -1))
    assert r.max_abs_err <= TOL * r.max_abs_ref


def test_rejects_what_does_not_fit(env):
    """Only an explicit grid hint above the device's compute units with more than
    16 rows needs more than the fixed 32 MiB: a clear error, nothing launched."""
    torch, marlin = env
    dev = torch.device("cuda:0")
    assert marlin._lib.marlin_gemm_static_capacity() == 32 << 20
    M, N, K = 64, 4096, 8192
    A, q, s, B, sp = O.make_problem(M, N, K, 128, 9)
    dA, dB, ds = (torch.from_numpy(x).to(dev) for x in (A, B, sp))
    dC = torch.full((M, N), 3.0, dtype=torch.half, device=dev)
    ws = torch.zeros(N // 128 * 16, dtype=torch.int, device=dev)
    marlin.force_kernel(1)
    try:
        rc = marlin.gemm_raw("marlin_gemm_static", dA, dB, dC, ds, ws, 128, sms=1000)
    finally:
        marlin.force_kernel(4)
    assert rc == 3 and "fixed scratch holds 33554432" in marlin.last_error()
    torch.cuda.synchronize()
    assert (dC == 3.0).all().item() and not ws.any().item()


def test_static_entry_in_a_graph(env):
    """Captured without a warm-up call on the capture stream (nothing to allocate), replayed
    several times with eager launches in between: every replay gives the eager result."""
    torch, marlin = env
    dev = torch.device("cuda:0")
    M, N, K, g = 4, 4096, 4096, 128
    A, q, s, B, sp = O.make_problem(M, N, K, g, 12)
    dA, dB, ds = (torch.from_numpy(x).to(dev) for x in (A, B, sp))
    want = torch.zeros((M, N), dtype=torch.half, device=dev)
    ws = torch.zeros(N // 128 * 16, dtype=torch.int, device=dev)
    assert marlin.gemm_raw("marlin_gemm_static", dA, dB, want, ds, ws, g) == 0
    torch.cuda.synchronize()
    fresh = torch.cuda.Stream()
    dC = torch.zeros_like(want)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=fresh):
        rc = marlin.gemm_raw("marlin_gemm_static", dA, dB, dC, ds, ws, g)
    assert rc == 0, marlin.last_error()
    for _ in range(4):
        dC.zero_()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(dC, want) and not ws.any().item()
        other = torch.zeros((16, 4096), dtype=torch.half, device=dev)
        dA16 = torch.randn((16, K), dtype=torch.half, device=dev)
        assert marlin.gemm_raw("marlin_gemm_static", dA16, dB, other, ds, ws, g) == 0
        torch.cuda.synchronize()


def test_static_entry_alone_allocates_nothing(env):
    """Only marlin_gemm_static is called, after the pool has been emptied, on a
    fresh stream: a shape whose column tiles are shared by 8 workgroups, then a
    smaller one.  The pool stays empty and the device's free memory does not
    move; the results are the oracle's."""
    torch, marlin = env
    dev = torch.device("cuda:0")
    probs = []
    for (M, N, K, g, seed) in [(16, 4096, 4096, 128, 21), (5, 1024, 2048, -1, 22)]:
        A, q, s, B, sp = O.make_problem(M, N, K, g, seed)
        dA, dB, ds = (torch.from_numpy(x).to(dev) for x in (A, B, sp))
        dC = torch.full((M, N), 3.0, dtype=torch.half, device=dev)
        ws = torch.zeros(N // 128 * 16, dtype=torch.int, device=dev)
        probs.append(((A, B, sp, N, g), dA, dB, ds, dC, ws))
    fresh = torch.cuda.Stream()
    with torch.cuda.stream(fresh):
        # the runtime sets a stream's queue up at its first launch (4 MiB of
        # device memory on this pool): let a kernel of torch's pay for that
        probs[0][5].add_(0)
    torch.cuda.synchronize()
    marlin.release()
    assert marlin.scratch_bytes() == (0, 0)
    free_before = torch.cuda.mem_get_info()[0]
    for ((_, _, _, _, g), dA, dB, ds, dC, ws) in probs:
        print(f"  marlin_gemm_static alone M={dA.shape[0]} N={dC.shape[1]} K={dA.shape[1]}", flush=True)
        rc = marlin.gemm_raw("marlin_gemm_static", dA, dB, dC, ds, ws, g, stream=fresh.cuda_stream)
        assert rc == 0, marlin.last_error()
    fresh.synchronize()
    assert torch.cuda.mem_get_info()[0] == free_before
    assert marlin.scratch_bytes() == (0, 0)
    for ((A, B, sp, N, g), dA, dB, ds, dC, ws) in probs:
        assert not ws.any().item()
        r = O.compare(dC.cpu().numpy(), O.gemm(A, B, sp, N, g))
        assert r.max_abs_err <= TOL * r.max_abs_ref


_FIRST_CALL_UNDER_CAPTURE = r"""
import sys
sys.path.insert(0, sys.argv[1]); sys.path.insert(0, sys.argv[2])
import numpy as np, torch, marlin, _oracle as O
dev = torch.device("cuda:0")
M, N, K, g = 4, 4096, 4096, 128
A, q, s, B, sp = O.make_problem(M, N, K, g, 12)
dA, dB, ds = (torch.from_numpy(x).to(dev) for x in (A, B, sp))
dC = torch.zeros((M, N), dtype=torch.half, device=dev)
ws = torch.zeros(N // 128 * 16, dtype=torch.int, device=dev)
torch.cuda.synchronize()
free_before = torch.cuda.mem_get_info()[0]
side = torch.cuda.Stream()
graph = torch.cuda.CUDAGraph()
with torch.cuda.graph(graph, stream=side):
    # the first call of this process into the library
    rc = marlin.gemm_raw("marlin_gemm_static", dA, dB, dC, ds, ws, g)
assert rc == 0, marlin.last_error()
assert marlin.scratch_bytes() == (0, 0)
ref = O.gemm(A, B, sp, N, g)
for _ in range(3):
    dC.zero_()
    graph.replay()
    torch.cuda.synchronize()
    r = O.compare(dC.cpu().numpy(), ref)
    assert r.max_abs_err <= 1e-2 * r.max_abs_ref and not ws.any().item()
print("first call under capture: ok")
"""


def test_first_static_call_of_a_process_inside_a_capture(env):
    """The very first call into the library is marlin_gemm_static under stream
    capture (a process of its own, so that nothing has been set up before):
    the device set-up and the symbol lookup must not break the capture, and
    every replay gives the oracle's result."""
    import subprocess
    res = subprocess.run([sys.executable, "-c", _FIRST_CALL_UNDER_CAPTURE,
                          os.path.join(ROOT, "awesome-cute_amd"), os.path.join(ROOT, "tests")],
                         capture_output=True, text=True, timeout=300)
    print(res.stdout[-2000:], res.stderr[-2000:], flush=True)
    assert res.returncode == 0 and "first call under capture: ok" in res.stdout
