"""GPU parity tests: the HIP path, called through the C ABI (marlin.mul ->
marlin_mul -> marlin_gemm), against the CPU oracle on the same seeded inputs.

Acceptance: dequantised weights bit-exact (probed with one-hot activation
rows), outputs within max|C - C_ref| <= 1e-2 * max|C_ref|.  Shapes follow the
reference's own tests (marlin_test.py:78-167) and the benchmark configs.
"""
import os
import sys

import numpy as np
import pytest

import _oracle as O

pytestmark = pytest.mark.gpu

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
sys.path.insert(0, os.path.join(ROOT, "awesome-cute_amd"))

TOL = 1e-2  # max-abs-error <= TOL * max|ref|, fp32 accumulation
REL_MEAN_TOL = 1e-3  # mean|C - C_ref| / mean|C_ref|


@pytest.fixture(scope="module")
def env():
    import torch
    import marlin
    assert torch.cuda.is_available()
    return torch, marlin


@pytest.fixture
def no_strips(env):
    """Up to 16 rows through the streaming kernel, as larger launches go: for
    the tests of what workgroups exchange (partial sums, tickets, scratch),
    which the column-strip kernel, the planner's choice for few rows over small
    weights, does not have."""
    torch, marlin = env
    marlin.force_kernel(4)
    yield
    marlin.force_kernel(0)


def gpu_gemm(env, A, B, sp, N, thread_k=-1, thread_n=-1, sms=-1, max_par=16, C_fill=None):
    torch, marlin = env
    dev = torch.device("cuda:0")
    M = A.shape[0]
    print(f"  gemm M={M} N={N} K={A.shape[1]} groups={sp.shape[0]} hints=({thread_k},{thread_n},{sms})",
          flush=True)
    dA = torch.from_numpy(A).to(dev)
    dB = torch.from_numpy(B).to(dev)
    ds = torch.from_numpy(sp).to(dev)
    dC = torch.zeros((M, N), dtype=torch.half, device=dev)
    if C_fill is not None:
        dC.fill_(C_fill)
    ws = torch.zeros(N // 128 * max_par, dtype=torch.int, device=dev)
    marlin.mul(dA, dB, dC, ds, ws, thread_k, thread_n, sms, max_par)
    torch.cuda.synchronize()
    assert not ws.any().item(), "workspace must be handed back zeroed"
    return dC.cpu().numpy()


def check(env, M, N, K, groupsize, seed=0, **kw):
    A, q, s, B, sp = O.make_problem(M, N, K, groupsize, seed)
    C = gpu_gemm(env, A, B, sp, N, **kw)
    Cref = O.gemm(A, B, sp, N, groupsize)
    r = O.compare(C, Cref)
    assert np.isfinite(r.max_abs_err)
    assert r.max_abs_err <= TOL * r.max_abs_ref, (r.max_abs_err, r.max_abs_ref)
    assert r.cosine >= 0.999
    # the figure the reference test prints (marlin_test.py:74; upstream's threshold).  Oracle
    # and kernel both accumulate in fp32, so they differ by summation order only.
    assert r.rel_mean_abs_err <= REL_MEAN_TOL, r.rel_mean_abs_err
    return r


@pytest.mark.parametrize("groupsize", [128, -1])
def test_dequantized_weights_bit_exact(env, groupsize):
    """One-hot activation rows return rows of the dequantised weight matrix;
    single-term sums leave no room for rounding differences."""
    N, K = 256, 512
    _, q, s, B, sp = O.make_problem(1, N, K, groupsize, seed=3)
    W = O.dequant(B, sp, K, N, groupsize)
    if groupsize == -1:
        W = W * O.unpack_scales(sp, False)  # fp16(q-8) * s, one rounding
    for rows in ([0], [5, 17, 130, 511], list(range(0, 512, 33))[:16],
                 list(range(1, 512, 9))[:48]):
        A = np.zeros((len(rows), K), np.float16)
        for i, r in enumerate(rows):
            A[i, r] = 1.0
        C = gpu_gemm(env, A, B, sp, N)
        assert np.array_equal(C.view(np.uint16), W[rows].view(np.uint16))


def test_all_k_rows_bit_exact_through_identity(env):
    """A = 64 shifted one-hot batches covers every k of a 512-deep weight."""
    N, K = 256, 512
    _, q, s, B, sp = O.make_problem(1, N, K, 128, seed=4)
    W = O.dequant(B, sp, K, N, 128)
    for base in range(0, K, 64):
        A = np.zeros((64, K), np.float16)
        A[np.arange(64), base + np.arange(64)] = 1.0
        C = gpu_gemm(env, A, B, sp, N)
        assert np.array_equal(C.view(np.uint16), W[base:base + 64].view(np.uint16))


def test_config1_reference_case(env):
    # smallest benchmark config == first case of marlin_test.py:123-131
    check(env, 16, 256, 512, 128, thread_k=128, thread_n=128)


def test_closed_forms(env):
    M, N, K = 16, 256, 512
    rng = np.random.default_rng(5)
    A = rng.standard_normal((M, K)).astype(np.float16)
    s = rng.uniform(0.001, 0.02, (K // 128, N)).astype(np.float16)
    q = np.full((K, N), 8, np.uint8)
    C = gpu_gemm(env, A, O.pack_weights(q), O.pack_scales(s, True), N, C_fill=7.0)
    assert not C.view(np.uint16).any()  # zero point everywhere -> exact zero
    Ai = rng.integers(-3, 4, (M, K)).astype(np.float16)
    q = rng.integers(0, 16, (K, N), dtype=np.uint8)
    ones = np.ones((K // 128, N), np.float16)
    C = gpu_gemm(env, Ai, O.pack_weights(q), O.pack_scales(ones, True), N)
    want = Ai.astype(np.int64) @ (q.astype(np.int64) - 8)
    assert np.abs(want).max() < 2048
    assert np.array_equal(C.astype(np.int64), want)  # exact integers


@pytest.mark.parametrize("m", [1, 2, 3, 4, 8, 12, 16, 24, 32, 48, 64, 118, 128, 152, 768, 1024])
def test_tiles(env, m):
    # marlin_test.py:78-84
    for thread_k, thread_n in [(64, 256), (128, 128)]:
        if m > 16 and thread_k == 128:
            continue
        check(env, m, 512, 1024, -1, seed=m, thread_k=thread_k, thread_n=thread_n)


@pytest.mark.parametrize("k", [768, 832, 896, 64, 128, 192])
def test_k_divisibility_and_few_stages(env, k):
    # marlin_test.py:86-94
    check(env, 16, 512, k, -1, seed=k, thread_k=64, thread_n=256)


@pytest.mark.parametrize("groupsize", [128, -1])
@pytest.mark.parametrize("n,k", [(256, 512), (256, 1024), (256 * 128, 1024)])
def test_groups(env, groupsize, n, k):
    # marlin_test.py:123-131
    check(env, 16, n, k, groupsize, seed=n + k, thread_k=128, thread_n=128)


@pytest.mark.parametrize("sms", [1, 3, 7, 31, 100, 255, 256, 333, 512, 1024])
@pytest.mark.parametrize("groupsize", [128, -1])
def test_partition_sweep(env, sms, groupsize):
    """Odd workgroup counts put tile boundaries in the middle of workgroups and
    make many workgroups share a tile: exercises the fixup."""
    check(env, 16, 1280, 1152, groupsize, seed=sms, sms=sms)
    check(env, 48, 768, 2048, groupsize, seed=sms + 1, sms=sms)


def test_deterministic(env, no_strips):
    A, q, s, B, sp = O.make_problem(16, 4096, 4096, 128, seed=9)
    c1 = gpu_gemm(env, A, B, sp, 4096)
    c2 = gpu_gemm(env, A, B, sp, 4096)
    assert np.array_equal(c1.view(np.uint16), c2.view(np.uint16))


def test_partition_does_not_change_the_bits(env, no_strips):
    """Partial sums are added in workgroup order by whoever arrives last, so a
    given partition always gives the same bits; different partitions differ
    only by fp32 reassociation (inside the tolerance)."""
    A, q, s, B, sp = O.make_problem(16, 1024, 2048, 128, seed=21)
    for sms in (24, 40, 256):
        runs = [gpu_gemm(env, A, B, sp, 1024, sms=sms) for _ in range(3)]
        assert all(np.array_equal(runs[0].view(np.uint16), r.view(np.uint16)) for r in runs[1:])


@pytest.mark.parametrize("max_par", [1, 2, 5, 8, 16, 64])
def test_workspace_stride_follows_max_par(env, max_par):
    """The tile counters sit max_par ints apart (capped at 16) inside the
    n/128*max_par ints the reference asks for (marlin_gemm.cpp:29-31): the
    smallest legal workspace works and comes back zeroed."""
    check(env, 16, 1024, 2048, 128, seed=max_par, max_par=max_par, sms=40)
    check(env, 33, 512, 1024, -1, seed=max_par + 1, max_par=max_par, sms=24)


def test_back_to_back_launches_share_scratch(env, no_strips):
    """Launches on one stream reuse the partial-sum slots: different inputs of
    one shape, and then another shape, must not see each other's partial sums."""
    torch, marlin = env
    dev = torch.device("cuda:0")
    probs = [O.make_problem(m, n, k, 128, seed) for (m, n, k, seed) in
             [(4, 4096, 4096, 31), (4, 4096, 4096, 32), (4, 4096, 4096, 33), (40, 1024, 4096, 34),
              (4, 4096, 4096, 35)]]
    outs = []
    for A, q, s, B, sp in probs:
        n = B.shape[1] // 2
        dC = torch.zeros((A.shape[0], n), dtype=torch.half, device=dev)
        ws = torch.zeros(n // 128 * 16, dtype=torch.int, device=dev)
        marlin.mul(torch.from_numpy(A).to(dev), torch.from_numpy(B).to(dev), dC,
                   torch.from_numpy(sp).to(dev), ws)
        outs.append((dC, ws))  # no synchronisation between the launches
    torch.cuda.synchronize()
    for (A, q, s, B, sp), (dC, ws) in zip(probs, outs):
        n = B.shape[1] // 2
        r = O.compare(dC.cpu().numpy(), O.gemm(A, B, sp, n, 128))
        assert r.max_abs_err <= TOL * r.max_abs_ref
        assert not ws.any().item()


def test_two_streams_run_side_by_side(env, no_strips):
    """GEMMs on two streams at the same time: each stream has its own partial-sum
    scratch, so neither sees the other's.  Shared column tiles (streaming kernel)
    and k slices (prefill kernel) on both; every result equals the one the same
    call gives alone, bit for bit."""
    torch, marlin = env
    dev = torch.device("cuda:0")
    shapes = [(4, 4096, 4096, 41), (100, 1024, 2048, 42), (16, 2048, 8192, 43), (300, 512, 4096, 44)]
    probs = []
    for (m, n, k, seed) in shapes:
        A, q, s, B, sp = O.make_problem(m, n, k, 128, seed)
        probs.append((n, torch.from_numpy(A).to(dev), torch.from_numpy(B).to(dev),
                      torch.from_numpy(sp).to(dev)))

    def run_all(stream, rounds):
        outs = []
        with torch.cuda.stream(stream):
            for r in range(rounds):
                for n, dA, dB, ds in probs:
                    dC = torch.zeros((dA.shape[0], n), dtype=torch.half, device=dev)
                    ws = torch.zeros(n // 128 * 16, dtype=torch.int, device=dev)
                    marlin.mul(dA, dB, dC, ds, ws)
                    outs.append((dC, ws))
        return outs

    torch.cuda.synchronize()
    s1, s2 = torch.cuda.Stream(), torch.cuda.Stream()
    alone = run_all(s1, 1)
    torch.cuda.synchronize()
    a = run_all(s1, 6)  # no synchronisation: the two streams' launches overlap
    b = run_all(s2, 6)
    torch.cuda.synchronize()
    for outs in (a, b):
        for i, (dC, ws) in enumerate(outs):
            want = alone[i % len(probs)][0]
            assert torch.equal(dC, want), (i, shapes[i % len(probs)])
            assert not ws.any().item()


def test_kernels_of_other_streams_beside_do_not_change_the_result(env, no_strips):
    """A launch gives the same bits whatever else runs on the GPU: kernels of another
    stream that keep LDS and memory busy stretch every latency inside the GEMM, which
    must not matter (shared column tiles of the streaming kernel with 1, 16 and 64 rows,
    k slices of the prefill kernel)."""
    torch, marlin = env
    dev = torch.device("cuda:0")
    shapes = [(1, 4096, 4096, 51), (16, 2048, 8192, 52), (64, 4096, 4096, 53), (128, 4096, 4096, 54)]
    x = torch.randn(4096, 4096, device=dev)
    beside, main = torch.cuda.Stream(), torch.cuda.Stream()
    for (m, n, k, seed) in shapes:
        A, q, s, B, sp = O.make_problem(m, n, k, 128, seed)
        dA, dB, ds = (torch.from_numpy(v).to(dev) for v in (A, B, sp))

        def run():
            dC = torch.zeros((m, n), dtype=torch.half, device=dev)
            ws = torch.zeros(n // 128 * 16, dtype=torch.int, device=dev)
            marlin.mul(dA, dB, dC, ds, ws)
            return dC

        alone = run()
        torch.cuda.synchronize()
        outs = []
        for it in range(20):
            with torch.cuda.stream(beside):
                if it % 2:
                    torch.sort(x[:512], dim=1)
                else:
                    for _ in range(3):
                        torch.softmax(x, dim=1)
            with torch.cuda.stream(main):
                outs.append(run())
        torch.cuda.synchronize()
        assert all(torch.equal(c, alone) for c in outs), (m, n, k)


def test_two_host_threads_two_streams(env, no_strips):
    """Two host threads, each with a stream of its own, call the library at the same time
    (ctypes releases the interpreter lock during a call): the per-device state behind the
    C ABI is locked, and both get the results a single thread gets."""
    import threading
    torch, marlin = env
    dev = torch.device("cuda:0")
    A, q, s, B, sp = O.make_problem(8, 2048, 4096, 128, 51)
    dA, dB, ds = (torch.from_numpy(x).to(dev) for x in (A, B, sp))
    want = torch.zeros((8, 2048), dtype=torch.half, device=dev)
    ws0 = torch.zeros(2048 // 128 * 16, dtype=torch.int, device=dev)
    marlin.mul(dA, dB, want, ds, ws0)
    torch.cuda.synchronize()
    errors = []

    def worker():
        try:
            marlin.force_kernel(4)  # kept per host thread
            st = torch.cuda.Stream()
            with torch.cuda.stream(st):
                ws = torch.zeros(2048 // 128 * 16, dtype=torch.int, device=dev)
                outs = [torch.zeros((8, 2048), dtype=torch.half, device=dev) for _ in range(40)]
                for dC in outs:
                    marlin.mul(dA, dB, dC, ds, ws)
                st.synchronize()
                for dC in outs:
                    assert torch.equal(dC, want)
                assert not ws.any().item()
        except Exception as e:  # surfaced in the main thread
            errors.append(e)

    threads = [threading.Thread(target=worker) for _ in range(2)]
    for t in threads:
        t.start()
    for t in threads:
        t.join()
    assert not errors, errors


@pytest.mark.parametrize("m", [17, 31, 32, 33, 47, 48, 49, 63, 64])
@pytest.mark.parametrize("groupsize", [128, -1])
def test_lds_ring_row_counts(env, m, groupsize):
    """2-4 row blocks take their activations through the LDS ring; ragged row
    counts, a deep k (many ring turns) and a shallow one (ring never full; one
    scale row would mean per-channel scales, so two groups at least)."""
    check(env, m, 512, 4096, groupsize, seed=m)
    check(env, m, 256, 256, groupsize, seed=m + 100)


@pytest.mark.parametrize("which", [1, 2])
@pytest.mark.parametrize("m", [65, 100, 128, 200, 257])
def test_either_kernel_above_64_rows(env, which, m):
    """Above 64 rows the host picks the streaming kernel (64 rows per launch,
    the reference's own scheme, marlin_cute_kernel.cu:70-93) or the prefill
    kernel by cost; both must give the reference's result for any row count."""
    torch, marlin = env
    marlin.force_kernel(which)
    try:
        assert marlin.plan(m, 512, 1024, 128)[1]["kernel"] == which
        check(env, m, 512, 1024, 128, seed=m + which)
        check(env, m, 256, 768, -1, seed=m + which + 7)
    finally:
        marlin.force_kernel(0)


@pytest.mark.parametrize("slices", [1, 2, 3, 4, 8])
@pytest.mark.parametrize("m", [1, 16, 40, 64, 65, 128, 200, 384])
def test_prefill_kernel_k_slices(env, m, slices):
    """The prefill kernel at both tile heights (64 and 128 rows; up to 64 rows
    the planner only uses the first) and with its k range cut into slices that
    meet through the ticketed exchange; the same slicing gives the same bits
    every time."""
    torch, marlin = env
    rows = 64 if m <= 64 or (m + slices) % 2 else 128
    marlin.force_kernel(2)
    marlin.force_k_slices(slices)
    marlin.force_tile_rows(rows)
    try:
        rc, plan = marlin.plan(m, 512, 2048, 128)
        assert rc == 0 and plan["kernel"] == 2 and plan["k_slices"] == slices
        assert plan["tile_rows"] == rows
        check(env, m, 512, 2048, 128, seed=m + slices)
        check(env, m, 256, 1024, -1, seed=m + slices + 3)  # at most 4 slices of 256
        A, q, s, B, sp = O.make_problem(m, 768, 1536, 128, seed=5)
        c1 = gpu_gemm(env, A, B, sp, 768)
        c2 = gpu_gemm(env, A, B, sp, 768)
        assert np.array_equal(c1.view(np.uint16), c2.view(np.uint16))
    finally:
        marlin.force_kernel(0)
        marlin.force_k_slices(0)
        marlin.force_tile_rows(0)


@pytest.mark.parametrize("rows", [64, 128])
@pytest.mark.parametrize("m,n,k,g", [(130, 1024, 1024, 128), (300, 512, 2304, -1), (1000, 768, 512, 128),
                                     (33, 512, 1024, 128), (300, 2048, 512, 128), (520, 4096, 256, -1)])
def test_prefill_kernel_tile_rows(env, rows, m, n, k, g):
    """Both tile heights on ragged row counts, several row tiles per column."""
    torch, marlin = env
    marlin.force_kernel(2)
    marlin.force_tile_rows(rows)
    try:
        rc, plan = marlin.plan(m, n, k, g)
        assert rc == 0 and plan["kernel"] == 2 and plan["tile_rows"] == rows
        assert plan["grid"] == -(-m // rows) * (n // 256) * plan["k_slices"]
        check(env, m, n, k, g, seed=m + rows)
    finally:
        marlin.force_kernel(0)
        marlin.force_tile_rows(0)


@pytest.mark.parametrize("m,n,k,g,slices", [
    (128, 256, 64, -1, 0),      # one stage: the second k half has none
    (129, 512, 192, -1, 0),     # three stages: halves of two and one
    (256, 256, 320, -1, 0),     # five stages, leaves in the middle of the first turn
    (100, 256, 384, 128, 0),
    (128, 256, 512, 128, 2),    # two stages per half and slice
    (1, 256, 256, 128, 0),      # one row of a 128-row tile
    (127, 768, 640, 128, 0),    # a group's scales straddle the k halves
    (128, 256, 1024, 128, 4),
    (333, 1024, 4096, 128, 0),
    (2048, 256, 8192, 128, 0),  # one column tile, many row tiles
    (128, 256, 24576, 128, 0),  # a long k range per workgroup
    (128, 256, 24576, 128, 8),
])
def test_four_wave_kernel_short_and_uneven_k_ranges(env, m, n, k, g, slices):
    """The 128-row kernel's assembly loop at its ends: fewer stages than a turn
    of the loop, odd counts (the k halves differ by a stage that reads zeros),
    ranges that end inside the first turn, and long ones."""
    torch, marlin = env
    marlin.force_kernel(2)
    marlin.force_tile_rows(128)
    marlin.force_k_slices(slices)
    try:
        rc, plan = marlin.plan(m, n, k, g)
        assert rc == 0 and plan["kernel"] == 2 and plan["tile_rows"] == 128
        if slices:
            assert plan["k_slices"] == slices
        check(env, m, n, k, g, seed=m + k)
    finally:
        marlin.force_kernel(0)
        marlin.force_tile_rows(0)
        marlin.force_k_slices(0)


@pytest.mark.parametrize("groupsize", [128, -1])
@pytest.mark.parametrize("m", [17, 32, 33, 48, 49, 64])
def test_several_row_blocks_over_long_runs(env, m, groupsize):
    """Two to four row blocks where every wave of the streaming kernel sees more
    granules than its ring holds (the two-slot instance is only for runs of at
    most two granules per wave; longer ones take the three-slot loop)."""
    torch, marlin = env
    for n, k in ((2048, 11008), (4096, 11008)):
        rc, plan = marlin.plan(m, n, k, groupsize)
        assert rc == 0 and plan["kernel"] == 1 and plan["granules_per_wg"] >= 9, plan
        check(env, m, n, k, groupsize, seed=m + n)


@pytest.mark.parametrize("groupsize", [128, -1])
@pytest.mark.parametrize("m", [17, 18, 31, 32, 33, 40, 48, 49, 63, 64])
def test_rows_cut_in_two_halves(env, m, groupsize):
    """17 to 64 rows on the streaming kernel, whole and cut into two halves that
    separate workgroups compute (each half its own ticket and partial sums):
    both within the tolerance of the oracle, C written everywhere (it starts at
    9), the same bits on a second call; the smallest legal workspace (one
    counter per tile) has no room for the second ticket and is never cut."""
    torch, marlin = env
    marlin.force_kernel(1)
    try:
        for n, k in ((512, 2048), (2048, 4096), (1280, 1152)):
            A, q, s, B, sp = O.make_problem(m, n, k, groupsize, seed=m + n)
            ref = O.gemm(A, B, sp, n, groupsize)
            for mode in (1, 2):
                marlin.force_row_halves(mode)
                rc, plan = marlin.plan(m, n, k, groupsize)
                assert rc == 0 and plan["kernel"] == 1
                c1 = gpu_gemm(env, A, B, sp, n, C_fill=9.0)
                c2 = gpu_gemm(env, A, B, sp, n, C_fill=9.0)
                assert np.array_equal(c1.view(np.uint16), c2.view(np.uint16))
                r = O.compare(c1, ref)
                assert r.max_abs_err <= TOL * r.max_abs_ref, (mode, n, k, r.max_abs_err)
                assert r.rel_mean_abs_err <= REL_MEAN_TOL
            c3 = gpu_gemm(env, A, B, sp, n, max_par=1, C_fill=9.0)  # mode 2 still set
            r = O.compare(c3, ref)
            assert r.max_abs_err <= TOL * r.max_abs_ref
    finally:
        marlin.force_kernel(0)
        marlin.force_row_halves(0)


@pytest.mark.parametrize("groupsize", [128, -1])
@pytest.mark.parametrize("m", [65, 96, 100, 128, 129, 200, 256, 300, 511])
def test_more_than_64_rows_in_one_streaming_launch(env, m, groupsize):
    """More than 64 rows on the streaming kernel as one launch whose rows are
    cut into parts of 32, every (column tile, part) with its own workgroups,
    ticket and partial sums -- where there is a CU per (tile, part) and a
    counter per part in the workspace; otherwise a launch per 64 rows.  Against
    the oracle, C written everywhere, the same bits twice."""
    torch, marlin = env
    marlin.force_kernel(1)
    marlin.force_row_halves(2)
    try:
        for n, k, max_par in ((512, 2048, 16), (1024, 1152, 16), (256, 4096, 16), (512, 1024, 4),
                              (512, 1024, 1)):
            parts = -(-m // 32)
            fits = parts <= min(max_par, 16) and (n // 128) * parts <= 256
            rc, plan = marlin.plan(m, n, k, groupsize)
            assert rc == 0 and plan["kernel"] == 1
            if max_par == 16:
                assert plan["launches"] == (1 if fits else -(-m // 64)), plan
                assert plan["row_parts"] == (parts if fits else 1)
            A, q, s, B, sp = O.make_problem(m, n, k, groupsize, seed=m + n + max_par)
            ref = O.gemm(A, B, sp, n, groupsize)
            c1 = gpu_gemm(env, A, B, sp, n, max_par=max_par, C_fill=9.0)
            c2 = gpu_gemm(env, A, B, sp, n, max_par=max_par, C_fill=9.0)
            assert np.array_equal(c1.view(np.uint16), c2.view(np.uint16))
            r = O.compare(c1, ref)
            assert r.max_abs_err <= TOL * r.max_abs_ref, (n, k, max_par, r.max_abs_err)
            assert r.rel_mean_abs_err <= REL_MEAN_TOL
    finally:
        marlin.force_kernel(0)
        marlin.force_row_halves(0)


STRIP_SHAPES = [
    # (m, n, k, groupsize): rows for every count of staged rows (2, 4, 8, 16), one chunk
    # and a ragged last one, runs of more chunks than the ring holds, both scale modes
    (1, 256, 256, 128), (2, 128, 128, -1), (3, 512, 2304, -1), (4, 2048, 1408, 128),
    (5, 768, 512, 128), (8, 640, 13824, 128), (9, 1280, 1152, 128), (13, 896, 384, -1),
    (16, 256, 4096, 128), (16, 128, 128, -1), (7, 384, 640, -1), (16, 2048, 128 * 37, 128),
    (11, 1152, 64 * 2 * 51, -1), (1, 1024, 8192, -1), (16, 4096, 4096, -1), (1, 11008, 4096, 128),
    # more rows in parts of 16, a workgroup per strip set and part: whole and ragged
    # last parts, more workgroups than compute units, the most rows the kernel takes
    (17, 256, 256, 128), (32, 1024, 1024, 128), (33, 512, 2304, -1), (48, 768, 512, 128),
    (64, 1024, 4096, 128), (40, 1280, 1152, 128), (64, 256, 128, -1), (50, 512, 640, -1),
    (64, 2048, 128 * 37, 128), (31, 1280, 64 * 2 * 51, -1), (128, 512, 1024, 128),
    (97, 768, 640, -1), (250, 2048, 512, 128), (513, 512, 640, -1), (1024, 256, 512, 128),
]


@pytest.mark.parametrize("strips", [1, 2, 3, 4])
@pytest.mark.parametrize("m,n,k,g", STRIP_SHAPES)
def test_column_strip_kernel(env, strips, m, n, k, g):
    """The kernel whose workgroups own 16, 32, 48 or 64 columns (and 16 rows) over
    the whole k range and exchange nothing: every strip width on every shape,
    C overwritten everywhere (it starts at 9)."""
    torch, marlin = env
    marlin.force_kernel(3)
    marlin.force_strips(strips)
    try:
        rc, p = marlin.plan(m, n, k, g)
        parts = -(-m // 16)
        assert (rc, p["kernel"], p["strips"], p["row_parts"]) == (0, 3, strips, parts)
        assert p["grid"] == -(-(n // 16) // strips) * parts  # (of three strips the last workgroup has fewer)
        assert p["launches"] == 1 and p["partial_kib"] == 0
        A, q, s, B, sp = O.make_problem(m, n, k, g, seed=m + n + k)
        C = gpu_gemm(env, A, B, sp, n, C_fill=9.0)
    finally:
        marlin.force_kernel(0)
        marlin.force_strips(0)
    r = O.compare(C, O.gemm(A, B, sp, n, -1 if g == k else g))
    assert r.max_abs_err <= TOL * r.max_abs_ref, (r.max_abs_err, r.max_abs_ref)
    assert r.rel_mean_abs_err <= REL_MEAN_TOL, r.rel_mean_abs_err


@pytest.mark.parametrize("strips", [1, 2, 3, 4])
@pytest.mark.parametrize("groupsize", [128, -1])
def test_column_strip_kernel_dequantized_weights_bit_exact(env, strips, groupsize):
    """One-hot rows through the column strips return the dequantised weights bit
    for bit: every k of a 1024-deep weight (16 rows at a time: all staged-row
    counts' widest instance), then single rows and short batches (the narrower
    instances) and batches of several 16-row parts, for every strip width and
    both scale modes."""
    torch, marlin = env
    N, K = 256, 1024
    _, q, s, B, sp = O.make_problem(1, N, K, groupsize, seed=13)
    W = O.dequant(B, sp, K, N, groupsize)
    if groupsize == -1:
        W = W * O.unpack_scales(sp, False)  # fp16(q-8) * s, one rounding
    marlin.force_kernel(3)
    marlin.force_strips(strips)
    try:
        for base in range(0, K, 16):
            A = np.zeros((16, K), np.float16)
            A[np.arange(16), base + np.arange(16)] = 1.0
            C = gpu_gemm(env, A, B, sp, N)
            assert np.array_equal(C.view(np.uint16), W[base:base + 16].view(np.uint16)), base
        for rows in ([0], [1023], [5, 700], [17, 130, 511], [3, 64, 65, 1000], list(range(2, 1024, 171))[:6],
                     list(range(1, 1024, 41))[:24], list(range(3, 1024, 19))[:45], list(range(0, 1024, 16)),
                     list(range(1, 1024, 5))[:200]):
            A = np.zeros((len(rows), K), np.float16)
            for i, r in enumerate(rows):
                A[i, r] = 1.0
            C = gpu_gemm(env, A, B, sp, N)
            assert np.array_equal(C.view(np.uint16), W[rows].view(np.uint16)), rows
    finally:
        marlin.force_kernel(0)
        marlin.force_strips(0)


@pytest.mark.parametrize("M", [16, 64, 200])
@pytest.mark.parametrize("strips", [1, 2, 3, 4])
def test_column_strip_kernel_closed_forms(env, strips, M):
    """Zero point everywhere gives exact zeros; small integers times unit scales
    give exact integers (every product and every partial sum is exact in fp32)."""
    torch, marlin = env
    N, K = 256, 768
    rng = np.random.default_rng(50 + strips + M)
    marlin.force_kernel(3)
    marlin.force_strips(strips)
    try:
        A = rng.standard_normal((M, K)).astype(np.float16)
        s = rng.uniform(0.001, 0.02, (K // 128, N)).astype(np.float16)
        q = np.full((K, N), 8, np.uint8)
        C = gpu_gemm(env, A, O.pack_weights(q), O.pack_scales(s, True), N, C_fill=7.0)
        assert not C.view(np.uint16).any()
        Ai = rng.integers(-3, 4, (M, K)).astype(np.float16)
        q = rng.integers(0, 16, (K, N), dtype=np.uint8)
        ones = np.ones((K // 128, N), np.float16)
        C = gpu_gemm(env, Ai, O.pack_weights(q), O.pack_scales(ones, True), N)
        want = Ai.astype(np.int64) @ (q.astype(np.int64) - 8)
        assert np.abs(want).max() < 2048
        assert np.array_equal(C.astype(np.int64), want)
    finally:
        marlin.force_kernel(0)
        marlin.force_strips(0)


@pytest.mark.parametrize("M", [1, 5, 8])
@pytest.mark.parametrize("strips", [1, 2, 3, 4])
def test_column_strip_kernel_scales_the_sums_of_a_group(env, strips, M):
    """Up to 8 rows the column strips multiply the sum of a group by its scale
    (fp32) instead of every weight (fp16): with small integer activations the
    result is sum_g s_g * (integer), exact in fp32 up to the order of the adds,
    so C is within one fp16 step of the exactly computed value -- nearer than
    the per-weight rounding of the scaled weights would be."""
    torch, marlin = env
    N, K = 256, 1024
    rng = np.random.default_rng(70 + strips + M)
    A = rng.integers(-3, 4, (M, K)).astype(np.float16)
    q = rng.integers(0, 16, (K, N), dtype=np.uint8)
    s = rng.uniform(0.001, 0.02, (K // 128, N)).astype(np.float16)
    marlin.force_kernel(3)
    marlin.force_strips(strips)
    try:
        C = gpu_gemm(env, A, O.pack_weights(q), O.pack_scales(s, True), N).astype(np.float64)
    finally:
        marlin.force_kernel(0)
        marlin.force_strips(0)
    want = np.zeros((M, N))
    for g in range(K // 128):
        rows = slice(128 * g, 128 * g + 128)
        want += s[g].astype(np.float64) * (A[:, rows].astype(np.int64) @ (q[rows].astype(np.int64) - 8))
    step = np.maximum(np.abs(want), 2.0 ** -14) * 2.0 ** -10  # one step of fp16 at |want|
    assert (np.abs(C - want) <= step).all(), np.abs((C - want) / step).max()


def test_few_rows_through_either_kernel_agree_with_the_oracle(env):
    """The shapes the planner gives to the column strips, through the streaming
    kernel as well: both inside the tolerance, on the same inputs."""
    torch, marlin = env
    for (m, n, k, g) in [(1, 4096, 4096, 128), (8, 2048, 2048, -1), (16, 1280, 1152, 128),
                         (64, 1024, 1024, 128), (200, 512, 1024, -1)]:
        assert marlin.plan(m, n, k, g)[1]["kernel"] == 3
        for which in (0, 4):
            marlin.force_kernel(which)
            try:
                check(env, m, n, k, g, seed=m + k)
            finally:
                marlin.force_kernel(0)


@pytest.mark.parametrize("tag,groupsize", [("g128", 128), ("chan", -1)])
def test_frozen_known_answers(env, tag, groupsize):
    """The committed known answers (tests/golden): dequantised weights bit for
    bit through one-hot rows, the GEMM inside the tolerance."""
    g = np.load(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden",
                             "w4a16_known_answers.npz"))
    B, sp = g[f"{tag}_B"], g[f"{tag}_s_packed"].view(np.float16)
    A, Cref = g[f"{tag}_A"].view(np.float16), g[f"{tag}_C"].view(np.float16)
    K, N = A.shape[1], Cref.shape[1]
    r = O.compare(gpu_gemm(env, A, B, sp, N), Cref)
    assert r.max_abs_err <= TOL * r.max_abs_ref
    rows = list(range(0, K, 7))[:16]
    onehot = np.zeros((len(rows), K), np.float16)
    for i, k in enumerate(rows):
        onehot[i, k] = 1.0
    W = g[f"{tag}_W"].view(np.float16)
    if groupsize == -1:
        W = W * O.unpack_scales(sp, False)
    assert np.array_equal(gpu_gemm(env, onehot, B, sp, N).view(np.uint16),
                          W[rows].view(np.uint16))


def _force(marlin, kernel=0, slices=0, rows=0):
    marlin.force_kernel(kernel)
    marlin.force_k_slices(slices)
    marlin.force_tile_rows(rows)


@pytest.mark.parametrize("slices", [1, 2, 4])
@pytest.mark.parametrize("groupsize", [128, -1])
@pytest.mark.parametrize("rows", [64, 128])
def test_prefill_kernel_dequantized_weights_bit_exact(env, rows, groupsize, slices):
    """The prefill kernel unpacks with its own interleaved copy of the dequant
    sequence and adds k halves and k slices: one-hot rows over every k of a
    1024-deep weight must return the dequantised rows bit for bit (all other
    halves and slices contribute exact zeros), at both tile heights, in both
    scale modes, unsliced and in 2 and 4 slices."""
    torch, marlin = env
    N, K, M = 512, 1024, 128
    _, q, s, B, sp = O.make_problem(1, N, K, groupsize, seed=11 + slices)
    W = O.dequant(B, sp, K, N, groupsize)
    if groupsize == -1:
        W = W * O.unpack_scales(sp, False)  # fp16(q-8) * s, one rounding
    _force(marlin, 2, slices, rows)
    try:
        rc, plan = marlin.plan(M, N, K, groupsize)
        assert rc == 0 and plan["kernel"] == 2 and plan["k_slices"] == slices
        assert plan["tile_rows"] == rows
        for base in range(0, K, M):
            A = np.zeros((M, K), np.float16)
            A[np.arange(M), base + np.arange(M)] = 1.0
            C = gpu_gemm(env, A, B, sp, N, C_fill=3.0)
            assert np.array_equal(C.view(np.uint16), W[base:base + M].view(np.uint16)), base
        # ragged: 70 one-hot rows at scattered k, rows past M never written
        ks = (np.arange(70) * 37 + 5) % K
        A = np.zeros((70, K), np.float16)
        A[np.arange(70), ks] = 1.0
        C = gpu_gemm(env, A, B, sp, N)
        assert np.array_equal(C.view(np.uint16), W[ks].view(np.uint16))
    finally:
        _force(marlin)


@pytest.mark.parametrize("rows,slices", [(64, 1), (128, 1), (64, 2), (128, 4)])
def test_prefill_kernel_closed_forms(env, rows, slices):
    """Zero point everywhere gives exact zeros and unit scales with small
    integer activations give exact integers, on the prefill kernel."""
    torch, marlin = env
    M, N, K = 200, 512, 1024
    rng = np.random.default_rng(rows + slices)
    _force(marlin, 2, slices, rows)
    try:
        assert marlin.plan(M, N, K, 128)[1]["kernel"] == 2
        A = rng.standard_normal((M, K)).astype(np.float16)
        q = np.full((K, N), 8, np.uint8)
        for g in (128, -1):
            s = rng.uniform(0.001, 0.02, (K // 128 if g == 128 else 1, N)).astype(np.float16)
            C = gpu_gemm(env, A, O.pack_weights(q), O.pack_scales(s, g == 128), N, C_fill=7.0)
            assert not C.view(np.uint16).any(), g
        Ai = rng.integers(-2, 3, (M, K)).astype(np.float16)
        q = rng.integers(0, 16, (K, N), dtype=np.uint8)
        want = Ai.astype(np.int64) @ (q.astype(np.int64) - 8)
        assert np.abs(want).max() < 2048
        for g in (128, -1):
            ones = np.ones((K // 128 if g == 128 else 1, N), np.float16)
            C = gpu_gemm(env, Ai, O.pack_weights(q), O.pack_scales(ones, g == 128), N)
            assert np.array_equal(C.astype(np.int64), want)
    finally:
        _force(marlin)


@pytest.mark.parametrize("groupsize", [128, -1])
def test_metric_batch16_point(env, groupsize):
    """M=16, N=K=4096: the middle point of the benchmark's metric, against the oracle."""
    check(env, 16, 4096, 4096, groupsize, seed=16)


@pytest.mark.parametrize("entry", ["marlin_gemm", "marlin_cute", "marlin_official"])
def test_fifteen_argument_entries_directly(env, entry):
    """The entries a relinked reference binding calls (marlin_gemm.cpp:6-14,
    34-46), with the 15 arguments in the reference's order: an explicit stream
    handle as argument 11 and an explicit device index, while another stream is
    current; return codes 0 / 1 / 2 straight from the entry."""
    torch, marlin = env
    dev = torch.device("cuda:0")
    st = torch.cuda.Stream()
    for (M, N, K, g) in [(16, 256, 512, 128), (1, 4096, 4096, 128), (40, 512, 2048, -1),
                         (300, 512, 1024, 128)]:
        A, q, s, B, sp = O.make_problem(M, N, K, g, seed=M + N)
        dA, dB, ds = (torch.from_numpy(x).to(dev) for x in (A, B, sp))
        dC = torch.full((M, N), 5.0, dtype=torch.half, device=dev)
        ws = torch.zeros(N // 128 * 16, dtype=torch.int, device=dev)
        torch.cuda.synchronize()
        print(f"  {entry} M={M} N={N} K={K} g={g} stream={st.cuda_stream:#x}", flush=True)
        rc = marlin.gemm_raw(entry, dA, dB, dC, ds, ws, g, stream=st.cuda_stream)
        assert rc == 0, marlin.last_error()
        st.synchronize()
        r = O.compare(dC.cpu().numpy(), O.gemm(A, B, sp, N, g))
        assert r.max_abs_err <= TOL * r.max_abs_ref and r.rel_mean_abs_err <= REL_MEAN_TOL
        assert not ws.any().item()
        # the default stream (null handle), as the reference's default argument
        dC.fill_(5.0)
        torch.cuda.synchronize()
        assert marlin.gemm_raw(entry, dA, dB, dC, ds, ws, g, stream=0) == 0
        torch.cuda.synchronize()
        r = O.compare(dC.cpu().numpy(), O.gemm(A, B, sp, N, g))
        assert r.max_abs_err <= TOL * r.max_abs_ref
    # error codes come back as integers (marlin_cute_kernel.cu:4-5)
    A = torch.zeros((16, 64), dtype=torch.half, device=dev)
    B = torch.zeros((4, 512), dtype=torch.int, device=dev)
    s1 = torch.ones((1, 256), dtype=torch.half, device=dev)
    C = torch.zeros((16, 256), dtype=torch.half, device=dev)
    ws = torch.zeros(32, dtype=torch.int, device=dev)
    assert marlin.gemm_raw(entry, A, B, C, s1, ws, -1, thread_k=128, thread_n=128) == 1
    assert marlin.gemm_raw(entry, A, B, C, s1, ws, 32, thread_k=64, thread_n=256) == 2
    assert marlin.gemm_raw(entry, A, B, C, s1, ws, -1, thread_k=64, thread_n=256, max_par=0) == 5
    assert marlin.gemm_raw(entry, A, B, C, s1, ws, -1, thread_k=64, thread_n=256) == 0
    torch.cuda.synchronize()


def test_marlin_lib_binding_module(env):
    """`marlin_lib.mul` with the reference's positional call
    (marlin.py:24: A, B, C, s, workspace, thread_k, thread_n, sms, max_par,
    cute_version) and with the pybind defaults (max_par = 8, marlin_gemm.cpp:21)."""
    torch, marlin = env
    import marlin_lib
    dev = torch.device("cuda:0")
    M, N, K, g = 16, 512, 1024, 128
    A, q, s, B, sp = O.make_problem(M, N, K, g, seed=77)
    dA, dB, ds = (torch.from_numpy(x).to(dev) for x in (A, B, sp))
    Cref = O.gemm(A, B, sp, N, g)
    for cute_version in (True, False):
        dC = torch.zeros((M, N), dtype=torch.half, device=dev)
        ws = torch.zeros(N // 128 * 16, dtype=torch.int, device=dev)
        marlin_lib.mul(dA, dB, dC, ds, ws, -1, -1, -1, 16, cute_version)
        torch.cuda.synchronize()
        r = O.compare(dC.cpu().numpy(), Cref)
        assert r.max_abs_err <= TOL * r.max_abs_ref and not ws.any().item()
    dC = torch.zeros((M, N), dtype=torch.half, device=dev)
    ws8 = torch.zeros(N // 128 * 8, dtype=torch.int, device=dev)  # enough for the default max_par
    marlin_lib.mul(dA, dB, dC, ds, ws8)
    torch.cuda.synchronize()
    assert O.compare(dC.cpu().numpy(), Cref).max_abs_err <= TOL * np.abs(Cref.astype(np.float32)).max()
    with pytest.raises(RuntimeError, match="workspace must be of size at least 32"):
        marlin_lib.mul(dA, dB, dC, ds, ws8[:16])


@pytest.mark.parametrize("m", [65, 128, 600])
@pytest.mark.parametrize("sms", [7, 100, 256, 1000])
def test_sms_hint_above_64_rows(env, m, sms):
    """An explicit `sms` (the reference's grid size, marlin_cute_kernel.cu:37-38,54)
    with more than 64 rows: whichever kernel the host falls to, the result is the
    reference's; with the streaming kernel forced the hint sets its grid."""
    torch, marlin = env
    check(env, m, 512, 2048, 128, seed=m + sms, sms=sms)
    marlin.force_kernel(1)
    try:
        rc, plan = marlin.plan(m, 512, 2048, 128, sms=sms)
        assert rc == 0 and plan["kernel"] == 1 and plan["grid"] <= min(sms, 4 * 32)
        check(env, m, 512, 2048, -1, seed=m + sms + 1, sms=sms)
    finally:
        marlin.force_kernel(0)


LLAMA_LARGER = {  # marlin_test.py:145-160: (k, n) of the four linear layers
    "13B": [(5120, 3 * 5120), (5120, 5120), (5120, 2 * 13568), (13568, 5120)],
    "33B": [(6656, 3 * 6656), (6656, 6656), (6656, 2 * 17664), (17664, 6656)],
    "70B": [(8192, 3 * 8192), (8192, 8192), (8192, 2 * 21760), (21760, 8192)],
}


@pytest.mark.parametrize("model,layer", [(m, i) for m in LLAMA_LARGER for i in range(4)])
def test_llama_larger_shapes(env, model, layer):
    """marlin_test.py:133-167, the 13B / 33B / 70B rows at batch 1 and 16 with
    per-channel scales as the reference test runs them.  GPU on the whole
    shape; oracle on three 256-column slices (columns are independent and a
    slice of the packed buffers on 128-column boundaries is a problem of its
    own)."""
    k, n = LLAMA_LARGER[model][layer]
    A16, q, s, B, sp = O.make_problem(16, n, k, -1, seed=k + n)
    del q
    for batch in (1, 16):
        A = np.ascontiguousarray(A16[:batch])
        C = gpu_gemm(env, A, B, sp, n, thread_k=128, thread_n=128)
        for c0 in (0, 256 * ((n // 256) // 2), n - 256):
            Bs = np.ascontiguousarray(B[:, 2 * c0:2 * (c0 + 256)])
            ss = np.ascontiguousarray(sp[:, c0:c0 + 256])
            r = O.compare(C[:, c0:c0 + 256], O.gemm(A, Bs, ss, 256, -1))
            assert r.max_abs_err <= TOL * r.max_abs_ref, (batch, c0, r.max_abs_err, r.max_abs_ref)
            assert r.rel_mean_abs_err <= REL_MEAN_TOL


def test_scratch_is_sized_by_the_plan_and_can_be_released(env, no_strips):
    """Partial-sum scratch: nothing for a launch that exchanges nothing, whole MiB
    sized by the plan per (device, stream) otherwise, shared with the dense
    GEMM, grown on demand, freed by release(); a first call under graph capture
    that would have to allocate fails with code 3 and leaves the capture usable."""
    torch, marlin = env
    import streamk
    dev = torch.device("cuda:0")
    torch.cuda.synchronize()
    marlin.release()
    assert marlin.scratch_bytes() == (0, 0)
    MiB = 1 << 20
    A, q, s, B, sp = O.make_problem(1, 4096, 4096, 128, seed=3)
    dA, dB, ds = (torch.from_numpy(x).to(dev) for x in (A, B, sp))
    want = None
    streams = [torch.cuda.Stream() for _ in range(8)]
    for i, st in enumerate(streams):
        with torch.cuda.stream(st):
            dC = torch.zeros((1, 4096), dtype=torch.half, device=dev)
            ws = torch.zeros(4096 // 128 * 16, dtype=torch.int, device=dev)
            marlin.mul(dA, dB, dC, ds, ws)
            st.synchronize()
            want = dC if want is None else want
            assert torch.equal(dC, want)
        held, bufs = marlin.scratch_bytes(0)
        # decode: 256 workgroups x 2 slots of 8 KiB = 4 MiB of partial sums, + 64 KiB of counters
        assert bufs == i + 1 and held == (i + 1) * (4 * MiB + 65536), (held, bufs)
    rc, plan = marlin.plan(1, 4096, 4096, 128)
    assert plan["partial_kib"] == 4096
    # one tile per workgroup exchanges nothing: no buffer for a new stream
    st = torch.cuda.Stream()
    with torch.cuda.stream(st):
        assert marlin.plan(16, 256 * 128, 1024, 128, thread_k=128, thread_n=128)[1]["partial_kib"] == 0
        check(env, 16, 256 * 128, 1024, 128, seed=5, thread_k=128, thread_n=128)
    assert marlin.scratch_bytes(0)[1] == 8
    # growth on one stream: a sliced prefill launch needs more than decode did
    with torch.cuda.stream(streams[0]):
        rc, plan = marlin.plan(512, 4096, 4096, 128)
        assert plan["k_slices"] > 1 and plan["partial_kib"] > 4096
        check(env, 512, 4096, 4096, 128, seed=6)
        held, bufs = marlin.scratch_bytes(0)
        assert bufs == 9  # the smaller buffer stays until release (graphs may name it)
        assert held <= 8 * (4 * MiB + 65536) + 2 * plan["partial_kib"] * 1024 + 65536 + MiB
        # the dense GEMM's stream-K tiles use the same buffer of this stream
        a = torch.randn((256, 2048), dtype=torch.half, device=dev)
        b = torch.randn((512, 2048), dtype=torch.half, device=dev)
        c = streamk.gemm(a, b)
        streams[0].synchronize()
        assert marlin.scratch_bytes(0)[1] == 9
        assert torch.allclose(c.float(), a.float() @ b.float().t(), rtol=2e-2, atol=0.5)
    # capture on a stream that has no scratch yet: refused, not allocated
    fresh = torch.cuda.Stream()
    dC = torch.zeros((1, 4096), dtype=torch.half, device=dev)
    ws = torch.zeros(4096 // 128 * 16, dtype=torch.int, device=dev)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=fresh):
        with pytest.raises(RuntimeError, match="captured"):
            marlin.mul(dA, dB, dC, ds, ws)
        dC.zero_()  # the capture is still alive
    graph.replay()
    torch.cuda.synchronize()
    assert marlin.scratch_bytes(0)[1] == 9
    del graph
    freed = marlin.release(0)
    assert freed == held and marlin.scratch_bytes() == (0, 0)
    with torch.cuda.stream(streams[3]):  # allocates again after a release
        dC = torch.zeros((1, 4096), dtype=torch.half, device=dev)
        marlin.mul(dA, dB, dC, ds, ws)
        streams[3].synchronize()
        assert torch.equal(dC, want)
    assert marlin.scratch_bytes(0) == (4 * MiB + 65536, 1)



def test_config2_decode(env):
    check(env, 1, 4096, 4096, 128, seed=2)


def test_config3_mlp_pair(env):
    check(env, 16, 11008, 4096, 128, seed=31)
    check(env, 16, 4096, 11008, 128, seed=32)


@pytest.mark.parametrize("m", [1, 16])
@pytest.mark.parametrize("k,n", [(4096, 3 * 4096), (4096, 4096), (4096, 2 * 10752), (10752, 4096)])
def test_llama7b_shapes(env, m, k, n):
    # marlin_test.py:133-167 (7B rows; per-channel as in the reference test)
    check(env, m, n, k, -1, seed=k + n + m, thread_k=128, thread_n=128)


@pytest.mark.parametrize("seed", [0, 1, 2])
def test_random_shapes_kernels_and_knobs(env, seed):
    """Seeded random draws over row counts around every row-block and tile
    boundary, widths, depths, both scale modes, either kernel, both tile
    heights and odd workgroup hints: each within tolerance of the oracle, C
    overwritten everywhere (it starts at 9), workspace handed back zeroed."""
    torch, marlin = env
    rng = np.random.default_rng(seed)
    for case in range(14):
        g = int(rng.choice([128, -1]))
        M = int(rng.choice([1, 2, 5, 15, 16, 17, 31, 32, 33, 47, 48, 49, 63, 64, 65, 70, 100, 128,
                            129, 200, 300, 513]))
        N = (256 * int(rng.integers(1, 20)) if M > 16 or rng.random() < 0.5
             else 128 * int(rng.integers(1, 40)))
        K = 128 * int(rng.integers(1, 40))
        if K == 128 and g == 128:
            K = 256
        forced = int(rng.choice([0, 0, 1, 2, 3, 4])) if N % 256 == 0 else int(rng.choice([0, 3, 4]))
        rows = int(rng.choice([0, 64, 128]))
        sms = int(rng.choice([-1, -1, -1, 7, 64, 100, 256, 300, 1000]))
        assert marlin.check(M, N, K, g) == 0
        print(f"  case {seed}/{case}: forced kernel {forced}, tile rows {rows}", flush=True)
        marlin.force_kernel(forced)
        marlin.force_tile_rows(rows)
        try:
            A, q, s, B, sp = O.make_problem(M, N, K, g, 1000 * seed + case)
            C = gpu_gemm(env, A, B, sp, N, sms=sms, C_fill=9.0)
        finally:
            marlin.force_kernel(0)
            marlin.force_tile_rows(0)
        r = O.compare(C, O.gemm(A, B, sp, N, g))
        assert r.max_abs_err <= TOL * r.max_abs_ref, (M, N, K, g, forced, rows, sms, r.max_abs_err)


@pytest.mark.parametrize("m,n,k,g", [(128, 4096, 11008, 128), (160, 4096, 11008, -1),
                                     (96, 5120, 13568, 128), (320, 4096, 11008, 128)])
def test_mid_rows_deep_k_planned_slices(env, m, n, k, g):
    """Between decode and prefill over a deep k range the prefill kernel's
    tiles are cut into more than four k slices (or three, not a power of two)
    by the host's cost model (the kernel is pinned: some of these shapes stream
    with their rows in parts otherwise); oracle on a column slice, GPU on the
    whole shape, and twice the same bits."""
    torch, marlin = env
    marlin.force_kernel(2)
    try:
        rc, plan = marlin.plan(m, n, k, g)
        assert rc == 0 and plan["kernel"] == 2 and plan["k_slices"] in (3, 5, 6), plan
        A, q, s, B, sp = O.make_problem(m, n, k, g, seed=m + k)
        C = gpu_gemm(env, A, B, sp, n)
        for c0 in (0, n - 256):
            Bs = np.ascontiguousarray(B[:, 2 * c0:2 * (c0 + 256)])
            ss = np.ascontiguousarray(sp[:, c0:c0 + 256])
            r = O.compare(C[:, c0:c0 + 256], O.gemm(A, Bs, ss, 256, g))
            assert r.max_abs_err <= TOL * r.max_abs_ref, (c0, r.max_abs_err, r.max_abs_ref)
        assert np.array_equal(gpu_gemm(env, A, B, sp, n).view(np.uint16), C.view(np.uint16))
    finally:
        marlin.force_kernel(0)


def test_config4_prefill_rows_sample(env):
    """M=2048, N=K=4096: the oracle checks a sample of rows (the full product
    is 69 GFLOP on the CPU); the GPU computes all of them."""
    M, N, K = 2048, 4096, 4096
    A, q, s, B, sp = O.make_problem(M, N, K, 128, seed=4)
    C = gpu_gemm(env, A, B, sp, N)
    rows = np.r_[0:8, 63:66, 127:130, 1000:1008, 2040:2048]
    Cref = O.gemm(A[rows], B, sp, N, 128)
    r = O.compare(C[rows], Cref)
    assert r.max_abs_err <= TOL * r.max_abs_ref
    # linearity across the whole output: rows are independent, so a second
    # call on a row permutation must give the permuted result bit for bit
    perm = np.random.default_rng(0).permutation(M)
    C2 = gpu_gemm(env, A[perm], B, sp, N)
    assert np.array_equal(C2.view(np.uint16), C[perm].view(np.uint16))


@pytest.mark.parametrize("groupsize", [128, -1])
def test_config5_large_uneven(env, groupsize):
    """M=64, N=28672, K=8192.  Oracle on a column slice (columns are
    independent; a slice of the packed buffers on 128-column boundaries is a
    valid problem of its own), GPU on the full shape."""
    M, N, K = 64, 28672, 8192
    A, q, s, B, sp = O.make_problem(M, N, K, groupsize, seed=5)
    C = gpu_gemm(env, A, B, sp, N)
    for c0 in (0, 128 * 111, N - 256):
        Bs = np.ascontiguousarray(B[:, 2 * c0:2 * (c0 + 256)])
        ss = np.ascontiguousarray(sp[:, c0:c0 + 256])
        Cref = O.gemm(A, Bs, ss, 256, groupsize)
        r = O.compare(C[:, c0:c0 + 256], Cref)
        assert r.max_abs_err <= TOL * r.max_abs_ref, (c0, r.max_abs_err, r.max_abs_ref)
    # zero-point weights in half of the k range must not change anything when
    # the matching activations are garbage-free zeros: C(A) == C(A with k<4096
    # zeroed) + C(A with k>=4096 zeroed) up to fp16 rounding of the two halves
    A1 = A.copy(); A1[:, K // 2:] = 0
    A2 = A.copy(); A2[:, :K // 2] = 0
    Cs = gpu_gemm(env, A1, B, sp, N).astype(np.float32) + gpu_gemm(env, A2, B, sp, N).astype(np.float32)
    assert np.abs(Cs - C.astype(np.float32)).max() <= TOL * np.abs(C.astype(np.float32)).max()


def test_binding_errors_raise(env):
    # marlin_test.py:96-121
    torch, marlin = env
    dev = torch.device("cuda:0")
    m, n, k = 16, 256, 64
    A = torch.zeros((m, k), dtype=torch.half, device=dev)
    B = torch.zeros((k // 16, 2 * n), dtype=torch.int, device=dev)
    s = torch.ones((1, n), dtype=torch.half, device=dev)
    C = torch.zeros((m, n), dtype=torch.half, device=dev)
    small_ws = torch.zeros(n // 128, dtype=torch.int, device=dev)
    ws = torch.zeros(n // 128 * 16, dtype=torch.int, device=dev)
    with pytest.raises(RuntimeError, match="workspace"):
        marlin.mul(A, B, C, s, small_ws, 128, 128, -1)
    with pytest.raises(RuntimeError, match="not compatible with thread_k=128"):
        marlin.mul(A, B, C, s, ws, 128, 128, -1)
    with pytest.raises(RuntimeError, match="not compatible with thread_k=256"):
        marlin.mul(A, B, C, s, ws, 256, 256, -1)
    s2 = torch.zeros((2, n), dtype=torch.half, device=dev)
    with pytest.raises(RuntimeError):
        marlin.mul(A, B, C, s2, ws, 256, 256, -1)
    with pytest.raises(RuntimeError, match="No kernel"):
        marlin.mul(A, B, C, s2, ws, 64, 256, -1)  # groupsize 32
    s3 = torch.zeros((3, n), dtype=torch.half, device=dev)
    with pytest.raises(RuntimeError, match="groups"):
        marlin.mul(A, B, C, s3, ws, 64, 256, -1)


def test_layer_forward_matches_oracle(env):
    torch, marlin = env
    dev = torch.device("cuda:0")
    k, n, m = 512, 256, 8
    rng = np.random.default_rng(21)
    w = rng.standard_normal((k, n)).astype(np.float16)
    for groupsize in (128, -1):
        q, s, ref = O.gen_quant4(w, groupsize)
        linear = torch.nn.Linear(k, n, bias=False)
        linear.weight.data = torch.from_numpy(ref).t().contiguous()
        layer = marlin.Layer(k, n, groupsize=groupsize)
        layer.pack(linear, torch.from_numpy(s).t().contiguous())
        assert np.array_equal(layer.B.numpy(), O.pack_weights(q))
        layer = layer.to(dev)
        A = rng.standard_normal((2, m // 2, k)).astype(np.float16)
        out = layer(torch.from_numpy(A).to(dev))
        torch.cuda.synchronize()
        assert out.shape == (2, m // 2, n)
        Cref = O.gemm(A.reshape(m, k), O.pack_weights(q), O.pack_scales(s, groupsize != -1), n,
                      groupsize)
        r = O.compare(out.cpu().numpy().reshape(m, n), Cref)
        assert r.max_abs_err <= TOL * r.max_abs_ref


@pytest.mark.parametrize("groupsize", [128, -1])
def test_profiling_row(env, groupsize):
    """One case of the LLaMA sweep harness at a small size: it checks the result
    against torch's fp32 product itself and reports both times."""
    import marlin_profiling as mp
    print(f"  run_profiling m=16 n=512 k=1024 group={groupsize}", flush=True)
    row = mp.run_profiling(16, 512, 1024, groupsize, iters=5, model="t")
    assert row['shape(m_n_k_group)'] == f"t_16_512_1024_{groupsize}"
    assert float(row['resident_us']) > 0 and float(row['hbm_us']) > 0
    assert float(row['max_rel_err']) <= TOL


@pytest.mark.parametrize("m,n,k,which", [(1, 4096, 4096, 4), (1, 4096, 4096, 3), (48, 1024, 4096, 0),
                                         (200, 2048, 2048, 0)])
def test_graph_replays_match_eager(env, m, n, k, which):
    """A captured launch (streaming kernel with shared tiles, column strips, LDS-ring
    variant, prefill kernel with k slices) replayed several times, with eager launches and
    synchronisations in between, gives the eager result every time and leaves the
    workspace zero: the counters are reset by the kernels, nothing is a memset."""
    torch, marlin = env
    dev = torch.device("cuda:0")
    marlin.force_kernel(which)
    try:
        _graph_replays(torch, marlin, dev, m, n, k)
    finally:
        marlin.force_kernel(0)


def _graph_replays(torch, marlin, dev, m, n, k):
    A, q, s, B, sp = O.make_problem(m, n, k, 128, 41)
    A2, q2, s2, B2, sp2 = O.make_problem(16, 512, 1024, 128, 42)
    d = [torch.from_numpy(x).to(dev) for x in (A, B, sp, A2, B2, sp2)]
    ws = torch.zeros(n // 128 * 16, dtype=torch.int, device=dev)
    ws2 = torch.zeros(512 // 128 * 16, dtype=torch.int, device=dev)
    side = torch.cuda.Stream()
    with torch.cuda.stream(side):
        want = torch.zeros((m, n), dtype=torch.half, device=dev)
        marlin.mul(d[0], d[1], want, d[2], ws)  # also allocates this stream's scratch
        other = torch.zeros((16, 512), dtype=torch.half, device=dev)
        marlin.mul(d[3], d[4], other, d[5], ws2)
        side.synchronize()
        C = torch.zeros_like(want)
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=side):
            marlin.mul(d[0], d[1], C, d[2], ws)
    for _ in range(4):
        C.zero_()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(C, want) and not ws.any().item()
        with torch.cuda.stream(side):
            C2 = torch.zeros_like(other)
            marlin.mul(d[3], d[4], C2, d[5], ws2)
            side.synchronize()
            assert torch.equal(C2, other)


def test_mul_under_torch_compile(env):
    """`marlin.mul` inside a function compiled with torch.compile(fullgraph=True)
    (the reference advertises use within torch.compile, marlin.py:12): the call
    is traced as the registered operator marlin_amd::mul, which mutates C and
    the workspace, and the compiled function gives the oracle's result and the
    eager call's bits, for a decode-sized and a prefill-sized problem."""
    torch, marlin = env
    dev = torch.device("cuda:0")

    def linear(A, B, s, ws):
        C = torch.empty((A.shape[0], s.shape[1]), dtype=torch.half, device=A.device)
        marlin.mul(A, B, C, s, ws)
        return C * 2

    compiled = torch.compile(linear, fullgraph=True, backend="aot_eager")
    for (M, N, K, g) in [(4, 512, 1024, 128), (200, 768, 512, -1)]:
        A, q, s, B, sp = O.make_problem(M, N, K, g, seed=M)
        dA, dB, ds = (torch.from_numpy(x).to(dev) for x in (A, B, sp))
        ws = torch.zeros(N // 128 * 16, dtype=torch.int, device=dev)
        print(f"  torch.compile M={M} N={N} K={K} g={g}", flush=True)
        got = compiled(dA, dB, ds, ws)
        want = linear(dA, dB, ds, ws)
        torch.cuda.synchronize()
        assert torch.equal(got, want) and not ws.any().item()
        r = O.compare((got / 2).cpu().numpy(), O.gemm(A, B, sp, N, g))
        assert r.max_abs_err <= TOL * r.max_abs_ref
    layer = marlin.Layer(512, 256, groupsize=128).to(dev)
    A, q, s, B, sp = O.make_problem(8, 256, 512, 128, seed=5)
    layer.B.copy_(torch.from_numpy(B))
    layer.s.copy_(torch.from_numpy(sp))
    got = torch.compile(layer, fullgraph=True, backend="aot_eager")(torch.from_numpy(A).to(dev))
    torch.cuda.synchronize()
    r = O.compare(got.cpu().numpy(), O.gemm(A, B, sp, 256, 128))
    assert r.max_abs_err <= TOL * r.max_abs_ref


@pytest.mark.parametrize("k", [8192, 21760])
@pytest.mark.parametrize("kind", ["mean one", "all positive"])
def test_per_channel_64_row_tiles_with_activations_of_one_sign(env, k, kind):
    """Per-channel scales on 64-row prefill tiles accumulate biased integers
    (1024 + n, 64 + n) and remove the bias, 1032 or 72 times the sum of the
    activations, at the end: with activations of one sign that sum grows with
    k, and so does the fp32 rounding it carries.  The result must stay inside
    the mean-error bound (and far inside the max-error bound) all the same."""
    torch, marlin = env
    M, N = 64, 512
    A, q, s, B, sp = O.make_problem(M, N, k, -1, seed=k)
    rng = np.random.default_rng(k)
    if kind == "mean one":
        A = (1.0 + 0.25 * rng.standard_normal((M, k))).astype(np.float16)
    else:
        A = np.abs(rng.standard_normal((M, k))).astype(np.float16)
    _force(marlin, kernel=2, rows=64)
    try:
        assert marlin.plan(M, N, k, -1)[1]["tile_rows"] == 64
        C = gpu_gemm(env, A, B, sp, N)
    finally:
        _force(marlin)
    r = O.compare(C, O.gemm(A, B, sp, N, -1))
    print(f"  k={k} {kind}: max_abs_err {r.max_abs_err:.3e} of {r.max_abs_ref:.3e}, "
          f"rel mean {r.rel_mean_abs_err:.2e}", flush=True)
    assert r.max_abs_err <= TOL * r.max_abs_ref
    assert r.rel_mean_abs_err <= REL_MEAN_TOL
