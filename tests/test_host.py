"""CPU-only tests of the host side: the C ABI library loads and exports what
include/marlin_amd.h declares, the argument contract matches the reference
launcher's return codes, the stream-K partition covers every granule exactly
once, and the Python mirror of the reference's `marlin` module packs the way
the oracle does.  No GPU work is launched here.
"""
import ctypes
import os
import re
import sys

import numpy as np
import pytest

import _oracle as O

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
sys.path.insert(0, os.path.join(ROOT, "awesome-cute_amd"))
LIB = os.path.join(ROOT, "awesome-cute_amd", "libmarlin_amd.so")


@pytest.fixture(scope="module")
def marlin():
    if not os.path.exists(LIB):
        pytest.fail("libmarlin_amd.so is not built; run `python __graft_entry__.py build`")
    import marlin as m
    return m


def test_library_exports_every_declared_symbol(marlin):
    header = open(os.path.join(ROOT, "include", "marlin_amd.h")).read()
    tools = open(os.path.join(ROOT, "include", "marlin_amd_tools.h")).read()
    probe = open(os.path.join(ROOT, "include", "marlin_amd_probe.h")).read()
    # the drop-in boundary carries no planner knob and no probe
    boundary = re.findall(r"\b(marlin_\w+)\s*\(", re.sub(r"/\*.*?\*/", "", header, flags=re.S))
    assert set(boundary) == {"marlin_gemm", "marlin_cute", "marlin_official", "marlin_mul",
                             "marlin_gemm_static", "marlin_gemm_static_capacity",
                             "marlin_amd_scratch_bytes", "marlin_amd_release",
                             "marlin_amd_last_error", "marlin_amd_version"}
    header = re.sub(r"/\*.*?\*/", "", header + tools, flags=re.S)
    names = re.findall(r"\b(marlin_\w+)\s*\(", header)
    assert {"marlin_gemm", "marlin_cute", "marlin_official", "marlin_mul", "marlin_amd_check",
            "marlin_amd_plan", "marlin_amd_work_order", "marlin_amd_force_kernel",
            "marlin_amd_force_k_slices", "marlin_amd_force_tile_rows",
            "marlin_amd_last_error", "marlin_gemm_static", "marlin_gemm_static_capacity",
            "marlin_amd_scratch_bytes", "marlin_amd_release", "marlin_amd_device_info",
            "marlin_amd_version"} <= set(names)
    lib = ctypes.CDLL(LIB)
    for n in set(names):
        assert hasattr(lib, n), n
    # the probes are a library of their own; the product library has none
    probe_names = set(re.findall(r"\b(marlin_\w+)\s*\(", re.sub(r"/\*.*?\*/", "", probe, flags=re.S)))
    assert probe_names == {"marlin_amd_probe", "marlin_amd_probe_issue", "marlin_amd_probe_pull",
                           "marlin_amd_probe_last_error"}
    assert not any(hasattr(lib, n) for n in probe_names)
    assert b"probe" not in open(LIB, "rb").read()
    plib = ctypes.CDLL(os.path.join(ROOT, "awesome-cute_amd", "libmarlin_amd_probe.so"))
    for n in probe_names:
        assert hasattr(plib, n), n
    assert b"gfx950" in marlin._lib.marlin_amd_version()


def test_oracle_is_not_linked_into_the_product():
    out = os.popen(f"ldd {LIB}").read()
    assert "w4a16_ref" not in out
    src = os.path.join(ROOT, "awesome-cute_amd")
    for dirpath, _, files in os.walk(src):
        for f in files:
            if f.endswith((".py", ".hip", ".hpp", ".h", ".cpp")):
                text = open(os.path.join(dirpath, f), errors="ignore").read()
                assert "oracle" not in text.lower() or f == "build.py", (dirpath, f)


# return codes of the reference launcher (marlin_cute_kernel.cu:39-60,95-107)
@pytest.mark.parametrize("args,want", [
    ((16, 256, 512, 128, -1, -1), 0),      # smallest benchmark config
    ((1, 4096, 4096, 128, -1, -1), 0),
    ((2048, 4096, 4096, 128, -1, -1), 0),
    ((64, 28672, 8192, -1, -1, -1), 0),
    ((0, 256, 512, 128, -1, -1), 0),       # empty problem is fine
    ((16, 0, 512, -1, -1, -1), 0),
    ((16, 256, 64, -1, 128, 128), 1),      # marlin_test.py:105 (k=64, thread_k=128)
    ((16, 256, 64, -1, 256, 256), 1),      # marlin_test.py:111
    ((16, 256, 64, 32, 256, 256), 1),      # marlin_test.py:118 (shape check comes first)
    ((16, 256, 64, 32, 64, 256), 2),       # groupsize 32: no kernel
    ((16, 128, 512, 128, -1, -1), 0),      # n=128 only with the small tile
    ((17, 128, 512, 128, -1, -1), 1),      # auto tile is (64,256) above 16 rows
    ((32, 256, 512, 128, 128, 128), 2),    # small tile has no kernel for 32 rows
    ((16, 256, 512, 128, 64, 128), 2),     # unknown tile
    ((16, 256, 192, -1, 64, 256), 0),      # marlin_test.py:93 (k=192, per-channel)
    ((16, 256, 192, 128, 64, 256), 1),     # k not a multiple of the group
    ((16, 256, 512, 128, 0, 128), 1),
    ((16, 256, 512, 0, -1, -1), 2),
])
def test_shape_contract(marlin, args, want):
    assert marlin.check(*args) == want


def test_binding_level_errors_without_gpu(marlin):
    """marlin_mul rejects bad group counts and short workspaces before any
    device work (marlin_gemm.cpp:27-31); null pointers are never touched."""
    err = ctypes.create_string_buffer(256)
    f = marlin._lib.marlin_mul
    rc = f(None, None, None, None, 16, 256, 64, 3, None, 32, 0, None, -1, -1, -1, 16, 1, err, 256)
    assert rc == 4 and b"not compatible with 3 groups" in err.value
    rc = f(None, None, None, None, 16, 256, 64, 1, None, 2, 0, None, 128, 128, -1, 16, 1, err, 256)
    assert rc == 5 and b"workspace must be of size at least 32" in err.value
    rc = f(None, None, None, None, 16, 256, 64, 1, None, 32, 0, None, 128, 128, -1, 16, 1, err, 256)
    assert rc == 1 and b"thread_k=128" in err.value
    rc = f(None, None, None, None, 16, 256, 64, 2, None, 32, 0, None, 64, 256, -1, 16, 1, err, 256)
    assert rc == 2 and b"groupsize=32" in err.value
    # an empty problem is accepted and does nothing
    rc = f(None, None, None, None, 0, 256, 128, 1, None, 32, 0, None, -1, -1, -1, 16, 1, err, 256)
    assert rc == 0
    # operands beyond the kernels' 32-bit byte offsets are refused before any device work
    n, k = 65536, 131072
    rc = f(None, None, None, None, 16, n, k, k // 128, None, n // 128 * 16, 0, None,
           -1, -1, -1, 16, 1, err, 256)
    assert rc == 3 and b"2 GiB" in err.value


def _partition(plan):
    """Re-derivation of the stream-K ownership from the plan's four numbers."""
    NT, KG, gpb, grid, wpt = (plan[k] for k in ("col_tiles", "granules_per_tile",
                                                "granules_per_wg", "grid", "wgs_per_tile"))
    total = NT * KG
    owner = np.full(total, -1)
    for b in range(grid):
        if wpt:  # every tile cut into wpt nearly equal runs
            t, j = divmod(b, wpt)
            lo, hi = t * KG + j * KG // wpt, t * KG + (j + 1) * KG // wpt
            assert hi - lo <= gpb
        else:    # the tile-major sequence cut into runs of gpb
            lo, hi = b * gpb, min(total, (b + 1) * gpb)
        assert lo < hi, "every launched workgroup owns at least one granule"
        assert (owner[lo:hi] == -1).all()
        owner[lo:hi] = b
    assert (owner >= 0).all(), "every granule has exactly one owner"
    return owner.reshape(NT, KG)


@pytest.mark.parametrize("n,k", [(4096, 4096), (11008, 4096), (4096, 11008), (28672, 8192),
                                 (128, 128), (256, 192), (512, 1024), (1280, 1152)])
@pytest.mark.parametrize("sms", [1, 2, 3, 7, 31, 100, 255, 256, 304, 512, 1024, 5000])
def test_stream_partition_properties(marlin, n, k, sms):
    m = 16 if n % 256 else 48
    rc, plan = marlin.plan(m, n, k, -1, -1, -1, sms, 256)
    assert rc == 0 and plan["kernel"] == 1
    assert plan["grid"] <= min(max(sms, 1), 1024)
    owner = _partition(plan)
    gpb = plan["granules_per_wg"]
    slots = set()
    for t in range(owner.shape[0]):
        sharers = sorted(set(owner[t].tolist()))
        # contributors of a tile are consecutive workgroups
        assert sharers == list(range(sharers[0], sharers[-1] + 1))
        assert sharers[0] == (t * owner.shape[1]) // gpb
        assert sharers[-1] == ((t + 1) * owner.shape[1] - 1) // gpb
        if len(sharers) > 1:
            for b in sharers:
                first_tile = (b * gpb) // owner.shape[1]
                slot = 2 * b + (1 if t != first_tile else 0)
                assert slot not in slots, "partial-sum slots never collide"
                slots.add(slot)
    # a workgroup shares at most its first and its last tile
    for b in range(plan["grid"]):
        tiles = np.unique(np.nonzero(owner == b)[0])
        for t in tiles[1:-1]:
            assert (owner[t] == b).all()


@pytest.mark.parametrize("grid", [1, 2, 7, 8, 9, 15, 16, 100, 172, 224, 251, 256, 1000, 1024])
def test_work_order_is_an_xcd_blocked_permutation(marlin, grid):
    """Workgroup b runs on XCD b % 8; the work indices of one XCD's workgroups
    form one run of consecutive numbers, so that the consecutive work indices
    that share a column tile meet behind one L2."""
    order = marlin.work_order(grid)
    assert sorted(order) == list(range(grid))
    start = 0
    for x in range(8):
        mine = [order[b] for b in range(x, grid, 8)]
        assert mine == list(range(start, start + len(mine)))
        start += len(mine)


@pytest.mark.parametrize("m,n,k", [(1, 4096, 4096), (16, 11008, 4096), (16, 4096, 11008),
                                   (32, 28672, 8192), (16, 256, 512), (16, 1280, 1152),
                                   (4, 12288, 4096), (16, 4096, 10752), (8, 4096, 14336),
                                   (48, 5120, 13824), (16, 128, 128), (16, 32768, 4096)])
def test_default_stream_plans_stay_inside_tiles(marlin, m, n, k):
    """Without an `sms` hint the planner picks splits whose workgroups never
    straddle a column-tile boundary (one exchange per workgroup at most) and
    never launches more workgroups than CUs."""
    marlin.force_kernel(1)  # the streaming kernel's plan, also where column strips would be cheaper
    try:
        rc, plan = marlin.plan(m, n, k, -1, -1, -1, -1, 256)
    finally:
        marlin.force_kernel(0)
    assert rc == 0 and plan["kernel"] == 1 and plan["grid"] <= 256
    owner = _partition(plan)
    KG = plan["granules_per_tile"]
    for b in range(plan["grid"]):
        tiles = np.unique(np.nonzero(owner == b)[0])
        assert len(tiles) >= 1
        if plan["wgs_per_tile"]:
            assert len(tiles) == 1
        else:  # whole tiles per workgroup
            assert plan["granules_per_wg"] % KG == 0
            for t in tiles:
                assert (owner[t] == b).all()


def test_kernel_choice_by_cost(marlin):
    """Up to 16 rows over a few MiB of weights, and more rows (in parts of 16,
    a workgroup each) while the parts fill the compute units at most twice, go
    through the column-strip kernel, few rows otherwise through the streaming
    kernel, many through the prefill kernel, whose k range is cut into slices (the cheapest count, at most eight)
    while tiles alone would leave CUs idle; 49-64 rows over big weights take 64-row prefill tiles, and
    so do more rows while twice as many tiles save k slices; up to a few hundred
    rows over small weights stream in one launch with the rows cut into parts of
    32.  The knobs override the choice."""
    for m, n, k, kernel, slices, rows in [
            (1, 4096, 4096, 3, 1, 0), (16, 4096, 11008, 1, 1, 0), (48, 28672, 8192, 1, 1, 0),
            (1, 11008, 4096, 3, 1, 0), (1, 28672, 8192, 1, 1, 0), (17, 4096, 4096, 3, 1, 0),
            (8, 2048, 2048, 3, 1, 0), (16, 8192, 8192, 1, 1, 0), (32, 1024, 1024, 3, 1, 0),
            (64, 512, 1024, 3, 1, 0), (32, 2048, 4096, 3, 1, 0), (64, 512, 4096, 3, 1, 0),
            (64, 4096, 4096, 3, 1, 0), (64, 8192, 4096, 1, 1, 0), (64, 28672, 8192, 2, 2, 64),
            (96, 4096, 4096, 1, 1, 0), (128, 4096, 4096, 1, 1, 0), (128, 512, 1024, 3, 1, 0),
            (1024, 256, 512, 3, 1, 0), (1040, 256, 512, 2, 1, 64), (512, 4096, 4096, 2, 2, 64),
            (128, 8192, 8192, 2, 4, 64), (640, 4096, 11008, 2, 3, 128),
            (512, 4096, 11008, 2, 4, 128), (1024, 4096, 4096, 2, 2, 128),
            (1536, 4096, 4096, 2, 1, 128), (2048, 4096, 4096, 2, 1, 128)]:
        rc, p = marlin.plan(m, n, k, 128)
        assert rc == 0 and (p["kernel"], p["k_slices"], p["tile_rows"]) == (kernel, slices, rows), \
            (m, n, k, p)
        if kernel == 2:
            assert p["grid"] == -(-m // rows) * (n // 256) * slices
    # rows in parts: one launch, a workgroup set per (tile, part)
    rc, p = marlin.plan(128, 4096, 4096, 128)
    assert (p["launches"], p["row_parts"], p["part_rows"], p["wgs_per_tile"]) == (1, 4, 32, 2)
    assert p["grid"] == 32 * 4 * 2
    rc, p = marlin.plan(64, 8192, 4096, 128)
    assert (p["launches"], p["row_parts"], p["part_rows"], p["wgs_per_tile"]) == (1, 2, 32, 2)
    rc, p = marlin.plan(16, 4096, 11008, 128)
    assert (p["kernel"], p["row_parts"], p["wgs_per_tile"], p["strips"]) == (1, 1, 8, 0)
    # column strips: a workgroup per 16, 32 or 64 columns, nothing exchanged, one launch
    rc, p = marlin.plan(1, 4096, 4096, 128)
    assert (p["kernel"], p["strips"], p["grid"], p["launches"], p["partial_kib"]) == (3, 1, 256, 1, 0)
    rc, p = marlin.plan(1, 8192, 1024, 128)
    assert (p["kernel"], p["strips"], p["grid"]) == (3, 2, 256)
    # ... and per 16 rows: strip sets x parts
    rc, p = marlin.plan(64, 4096, 4096, 128)
    assert (p["kernel"], p["strips"], p["row_parts"], p["part_rows"], p["grid"]) == (3, 4, 4, 16, 256)
    rc, p = marlin.plan(100, 512, 1024, 128)
    assert (p["kernel"], p["strips"], p["row_parts"], p["grid"], p["launches"]) == (3, 2, 7, 16 * 7, 1)
    assert marlin.plan(1, 4096, 4096, 128, sms=64)[1]["kernel"] == 1  # a hint asks for the streaming split
    try:
        marlin.force_kernel(3)
        for strips in (1, 2, 3, 4):
            marlin.force_strips(strips)
            rc, p = marlin.plan(16, 28672, 8192, 128)
            assert (p["kernel"], p["strips"], p["grid"]) == (3, strips, -(-28672 // (16 * strips)))
        marlin.force_strips(4)
        rc, p = marlin.plan(16, 128 * 3, 512, 128, 128, 128)  # 24 strips
        assert (p["kernel"], p["strips"]) == (3, 4) and p["grid"] == 6
        marlin.force_strips(0)
        rc, p = marlin.plan(1024, 4096, 4096, 128)  # up to 1024 rows
        assert (p["kernel"], p["row_parts"], p["grid"]) == (3, 64, 64 * 4096 // (16 * p["strips"]))
        assert marlin.plan(1025, 4096, 4096, 128)[1]["kernel"] == 2  # more: as by cost
        assert marlin.plan(2048, 4096, 4096, 128)[1]["kernel"] == 2
    finally:
        marlin.force_kernel(0)
        marlin.force_strips(0)
    try:
        marlin.force_kernel(1)
        rc, p = marlin.plan(2048, 4096, 4096, 128)
        assert rc == 0 and p["kernel"] == 1 and p["launches"] == 32 and p["row_parts"] == 1
        marlin.force_kernel(2)
        rc, p = marlin.plan(100, 512, 1024, 128)
        assert rc == 0 and p["kernel"] == 2 and p["row_parts"] == 1
        assert p["grid"] == -(-100 // p["tile_rows"]) * 2 * p["k_slices"]
        marlin.force_tile_rows(128)
        assert marlin.plan(100, 512, 1024, 128)[1]["tile_rows"] == 128
        assert marlin.plan(40, 512, 1024, 128)[1]["tile_rows"] == 128
        marlin.force_tile_rows(64)
        rc, p = marlin.plan(2048, 4096, 4096, 128)
        assert rc == 0 and p["tile_rows"] == 64 and p["grid"] == 32 * 16 * p["k_slices"]
        marlin.force_tile_rows(0)
        marlin.force_k_slices(3)
        assert marlin.plan(100, 512, 1024, 128)[1]["k_slices"] == 3
        assert marlin.plan(100, 512, 512, 128)[1]["k_slices"] == 2  # slices are >= 256 deep
        assert marlin.plan(16, 128, 512, 128)[1]["kernel"] == 1  # n = 128: no 256-wide tile
    finally:
        marlin.force_kernel(0)
        marlin.force_k_slices(0)
        marlin.force_tile_rows(0)


def test_plan_costs_are_what_the_choice_compares(marlin):
    """marlin_amd_plan_costs: the fitted costs behind the choice of kernel --
    positive microseconds, -1 where a kernel cannot run the shape, and the plan
    is the cheapest of them where no rule of the planner says otherwise."""
    rc, c = marlin.plan_costs(1, 4096, 4096, 128)
    assert rc == 0 and 3.0 < c["strips"] < c["stream"] < 8.0 and c["strips_per_wg"] == 1
    assert marlin.plan(1, 4096, 4096, 128)[1]["kernel"] == 3
    rc, c = marlin.plan_costs(2048, 4096, 4096, 128)
    assert rc == 0 and c["strips"] == -1 and 40.0 < c["prefill"] < c["stream"]
    rc, c = marlin.plan_costs(16, 128 * 5, 1024, 128)
    assert rc == 0 and c["prefill"] == -1 and c["strips"] > 0      # n no multiple of 256
    rc, c = marlin.plan_costs(32, 28672, 512, 128)
    assert rc == 0 and c["strips"] == -1 and c["strips_per_wg"] == 0  # no width the rules allow:
    # parts of 16 rows may fill the compute units twice, no more (2 x 448 workgroups with four strips)
    assert marlin.plan(32, 28672, 512, 128)[1]["kernel"] == 1
    assert marlin.plan_costs(16, 100, 512, 128)[0] == 1 and marlin.plan_costs(0, 256, 512, 128)[0] == 0
    # a short k range never takes the prefill kernel up to 64 rows, whatever the fits say
    assert marlin.plan(64, 11008, 2048, 128)[1]["kernel"] == 1
    for m, n, k in [(1, 11008, 4096), (16, 4096, 11008), (32, 1024, 1024), (48, 4096, 4096),
                    (64, 8192, 4096), (32, 4096, 8192), (128, 2048, 2048), (256, 512, 4096)]:
        rc, c = marlin.plan_costs(m, n, k, 128)
        margin = 1.05 if m > 16 else 1.0
        want = 3 if c["strips"] > 0 and c["strips"] * margin < c["stream"] else 1
        assert marlin.plan(m, n, k, 128)[1]["kernel"] == want, (m, n, k, c)


def test_planned_column_strips_obey_the_planner_s_rules(marlin):
    """Over random shapes: a planned column-strip launch has strip sets x 16-row
    parts workgroups in one launch without scratch; more than 16 rows only while
    the parts fill 256 compute units at most twice; three strips per workgroup
    only up to 16 rows and from K = 1024 on; two and four only where they divide
    N's strips; nothing beyond 1024 rows or with an `sms` hint."""
    rng = np.random.default_rng(5)
    seen = 0
    for _ in range(3000):
        m = int(rng.choice([1, 2, 5, 8, 9, 16, 17, 33, 64, 100, 256, 700, 1024, 1025, 3000]))
        n = 256 * int(rng.integers(1, 120)) if m > 16 or rng.random() < 0.5 else 128 * int(rng.integers(1, 240))
        k = 128 * int(rng.integers(1, 100))
        sms = int(rng.choice([-1, -1, -1, 64]))
        rc, p = marlin.plan(m, n, k, 128, sms=sms)
        assert rc == 0, (m, n, k)
        if p["kernel"] != 3:
            assert p["strips"] == 0
            continue
        seen += 1
        cs, parts = p["strips"], -(-m // 16)
        assert sms < 0 and m <= 1024 and cs in (1, 2, 3, 4)
        assert p["row_parts"] == parts and p["part_rows"] == (16 if m > 16 else 0)
        assert p["grid"] == -(-(n // 16) // cs) * parts
        assert p["launches"] == 1 and p["partial_kib"] == 0
        if m > 16:
            assert p["grid"] <= 2 * 256, (m, n, k, p)
        if cs == 3:
            assert m <= 16 and k >= 1024
        else:
            assert n % (16 * cs) == 0
    assert seen > 300


def test_plan_picks_kernels(marlin):
    assert marlin.plan(1, 4096, 4096, 128)[1]["kernel"] == 3
    assert marlin.plan(32, 28672, 8192, 128)[1]["kernel"] == 1
    rc, p = marlin.plan(2048, 4096, 4096, 128)
    assert rc == 0 and p["kernel"] == 2 and p["grid"] == 16 * 16
    assert marlin.plan(16, 256, 64, -1, 128, 128)[0] == 1


# ------------------------------------------------------------ Python mirror

def test_perms_match_oracle(marlin):
    perm, sp, sps = O.get_perms()
    assert np.array_equal(marlin._perm.numpy(), perm)
    assert marlin._scale_perm == sp.tolist()
    assert marlin._scale_perm_single == sps.tolist()


@pytest.mark.parametrize("k,n", [(16, 64), (128, 256), (512, 768)])
def test_pack_weights_matches_oracle(marlin, k, n):
    import torch
    q = np.random.default_rng(k + n).integers(0, 16, (k, n), dtype=np.uint8)
    B = marlin.pack_weights(torch.from_numpy(q.astype(np.int32)))
    assert B.dtype == torch.int32
    assert np.array_equal(B.numpy(), O.pack_weights(q))


@pytest.mark.parametrize("groupwise", [True, False])
def test_pack_scales_matches_oracle(marlin, groupwise):
    import torch
    s = np.random.default_rng(7).uniform(0.001, 0.02, (4 if groupwise else 1, 512)).astype(np.float16)
    got = marlin.pack_scales(torch.from_numpy(s), groupwise).numpy()
    assert np.array_equal(got.view(np.uint16), O.pack_scales(s, groupwise).view(np.uint16))


@pytest.mark.parametrize("groupsize", [128, -1])
def test_layer_pack_on_cpu(marlin, groupsize):
    """Layer.pack (marlin.py:92-131) from a fake-quantised Linear: the packed
    buffers decode back to the quantiser's integers and scales."""
    import torch
    k, n = 256, 256
    w = np.random.default_rng(3).standard_normal((k, n)).astype(np.float16)
    q, s, ref = O.gen_quant4(w, groupsize)
    linear = torch.nn.Linear(k, n, bias=False)
    linear.weight.data = torch.from_numpy(ref).t().contiguous()
    layer = marlin.Layer(k, n, groupsize=groupsize)
    layer.pack(linear, torch.from_numpy(s).t().contiguous())
    assert np.array_equal(O.unpack_weights(layer.B.numpy(), k, n), q)
    assert np.array_equal(O.unpack_scales(layer.s.numpy(), groupsize != -1).view(np.uint16),
                          s.view(np.uint16))
    assert layer.workspace.numel() == n // 128 * 16 and not layer.workspace.any()


def test_quantize_matches_oracle_quantiser(marlin):
    import torch
    w = np.random.default_rng(5).standard_normal((256, 128)).astype(np.float16)
    for g in (128, -1):
        ref, q, s = marlin.quantize(torch.from_numpy(w), g)
        q0, s0, ref0 = O.gen_quant4(w, g)
        assert np.array_equal(q.numpy(), q0)
        assert np.array_equal(s.numpy().view(np.uint16), s0.view(np.uint16))
        assert np.array_equal(ref.numpy().view(np.uint16), ref0.view(np.uint16))


def test_layer_rejects_what_the_reference_rejects(marlin):
    with pytest.raises(ValueError):
        marlin.Layer(256, 256, groupsize=64)
    with pytest.raises(ValueError):
        marlin.Layer(192, 256)
    with pytest.raises(ValueError):
        marlin.Layer(256, 128)


def test_replace_linear(marlin):
    import torch.nn as nn
    model = nn.Sequential(nn.Linear(256, 512), nn.ReLU(), nn.Sequential(nn.Linear(512, 256)))
    marlin.replace_linear(model, groupsize=128)
    assert isinstance(model[0], marlin.Layer) and isinstance(model[2][0], marlin.Layer)
    assert model[0].k == 256 and model[0].n == 512 and model[0].groupsize == 128
    marlin.replace_linear(model)  # Layers are left alone


def test_mul_refuses_cpu_tensors(marlin):
    import torch
    A = torch.zeros((1, 128), dtype=torch.half)
    with pytest.raises(RuntimeError, match="GPU tensor"):
        marlin.mul(A, A, A, A, A)


def test_profiling_sweep_shapes_are_accepted(marlin):
    """The sweep's layer table is the reference's (marlin_profiling.py:88-113) and
    every case of it passes the shape contract."""
    import marlin_profiling as mp
    assert mp.MODELS['7B'] == [(4096, 12288), (4096, 4096), (4096, 21504), (10752, 4096)]
    assert mp.MODELS['70B'][2:] == [(8192, 43520), (21760, 8192)]
    assert len(mp.MODELS) == 4 and all(len(v) == 4 for v in mp.MODELS.values())
    for layers in mp.MODELS.values():
        for k, n in layers:
            for g in mp.GROUP_SIZES:
                for m in mp.BATCHES:
                    assert marlin.check(m, n, k, g) == 0, (m, n, k, g)


@pytest.mark.parametrize("groupsize", [128, -1])
def test_profiling_gen_quant4_on_cpu(marlin, groupsize):
    """gen_quant4 of the sweep: the packed buffers decode (through the oracle's
    unpackers) to a weight equal to the fake-quantised one it returns."""
    import marlin_profiling as mp
    k, n = 256, 128
    ref, B, sp = mp.gen_quant4(k, n, groupsize, dev='cpu', seed=1)
    q = O.unpack_weights(B.numpy(), k, n)
    s = O.unpack_scales(sp.numpy(), groupsize != -1)
    gs = k if groupsize == -1 else groupsize
    want = (q.astype(np.float32) - 8).astype(np.float16) * np.repeat(s, gs, axis=0)
    assert np.array_equal(want.view(np.uint16), ref.numpy().view(np.uint16))


def test_scratch_accounting_and_plan_sizes_without_gpu(marlin):
    """Nothing is held before any GEMM ran; the plan reports what a launch would
    exchange through the scratch: two 8 KiB slots per workgroup and row block
    for the streaming kernel when column tiles are shared, tile bytes per k
    slice for the prefill kernel, nothing otherwise."""
    assert marlin.scratch_bytes() == (0, 0)
    assert marlin.release() == 0
    rc, p = marlin.plan(1, 4096, 4096, 128)  # column strips: nothing exchanged
    assert rc == 0 and p["kernel"] == 3 and p["partial_kib"] == 0
    rc, p = marlin.plan(16, 4096, 11008, 128)
    assert rc == 0 and p["wgs_per_tile"] == 8 and p["grid"] == 256 and p["partial_kib"] == 2 * 256 * 8
    rc, p = marlin.plan(64, 4096, 4096, 128, sms=100)  # forced uniform runs, four row blocks
    assert p["kernel"] == 1 and p["wgs_per_tile"] == 0
    assert p["partial_kib"] == 2 * p["grid"] * 4 * 8
    marlin.force_kernel(1)
    try:
        rc, p = marlin.plan(16, 256 * 128, 1024, 128, 128, 128)  # one whole tile per workgroup
    finally:
        marlin.force_kernel(0)
    assert p["kernel"] == 1 and p["partial_kib"] == 0
    rc, p = marlin.plan(2048, 4096, 4096, 128)
    assert p["kernel"] == 2 and p["k_slices"] == 1 and p["partial_kib"] == 0
    rc, p = marlin.plan(512, 4096, 4096, 128)
    assert p["kernel"] == 2 and p["k_slices"] > 1
    assert p["partial_kib"] == p["grid"] * p["tile_rows"] * 256 * 4 // 1024
    rc, p = marlin.plan(128, 4096, 4096, 128)  # rows in parts of 32: two row blocks per slot
    assert p["kernel"] == 1 and p["row_parts"] == 4 and p["partial_kib"] == 2 * p["grid"] * 2 * 8
    rc, p = marlin.plan(256, 4096, 4096, 128)  # a workgroup per tile and part: no exchange
    assert p["kernel"] == 1 and p["wgs_per_tile"] == 1 and p["partial_kib"] == 0
    assert marlin._lib.marlin_gemm_static_capacity() == 32 << 20


def test_streaming_grid_stays_within_the_slot_limit(marlin):
    """However many compute units a device reports, the streaming launch has at
    most 1024 workgroups (the bound its partial-sum slots are sized for)."""
    for cus in (256, 1000, 2000, 5000):
        for (m, n, k) in [(16, 4096, 4096), (1, 28672, 8192), (64, 32768, 4096)]:
            marlin.force_kernel(1)
            try:
                rc, p = marlin.plan(m, n, k, 128, cus=cus)
            finally:
                marlin.force_kernel(0)
            assert rc == 0 and p["grid"] <= 1024, (cus, m, n, k, p)
            _partition(p)


def test_planner_overrides_are_per_thread(marlin):
    """force_kernel and friends change the plans of the calling thread only."""
    import threading
    seen = {}
    marlin.force_kernel(1)
    try:
        def other():
            seen["other"] = marlin.plan(2048, 4096, 4096, 128)[1]["kernel"]
        t = threading.Thread(target=other)
        t.start()
        t.join()
        seen["mine"] = marlin.plan(2048, 4096, 4096, 128)[1]["kernel"]
    finally:
        marlin.force_kernel(0)
    assert seen == {"other": 2, "mine": 1}


def test_max_par_below_one(marlin):
    """max_par < 1 cannot size the tile counters: marlin_gemm refuses it, and the
    binding asks for one counter per tile at least (the reference's comparison,
    marlin_gemm.cpp:29-31, would let an empty workspace through)."""
    err = ctypes.create_string_buffer(256)
    f = marlin._lib.marlin_mul
    rc = f(None, None, None, None, 16, 256, 128, 1, None, 0, 0, None, -1, -1, -1, 0, 1, err, 256)
    assert rc == 5 and b"workspace must be of size at least 2" in err.value
    g = marlin._lib.marlin_gemm
    assert g(None, None, None, None, 16, 256, 128, None, -1, 0, None, -1, -1, -1, 0) == 5
    assert g(None, None, None, None, 16, 256, 128, None, -1, 0, None, -1, -1, -1, -3) == 5


def test_marlin_lib_module_signature(marlin):
    """The module the reference imports as marlin_lib (marlin.py:5-8) with the
    pybind defaults of marlin_gemm.cpp:58-60."""
    import inspect
    import marlin_lib
    sig = inspect.signature(marlin_lib.mul)
    assert list(sig.parameters) == ["A", "B", "C", "s", "workspace", "thread_k", "thread_n", "sms",
                                    "max_par", "cute_version"]
    d = {k: v.default for k, v in sig.parameters.items() if v.default is not inspect.Parameter.empty}
    assert d == {"thread_k": -1, "thread_n": -1, "sms": -1, "max_par": 8, "cute_version": True}


def test_header_compiles_as_c_and_links(tmp_path):
    """A consumer written in C: the headers under include/ compiled with gcc
    -std=c11 -Wall -Werror (and as C++ with g++), linked against libmarlin_amd.so
    (and the probe library beside it), the way
    the reference's binding would be relinked (marlin_gemm.cpp:6-14, 34-46).
    It asks marlin_amd_check for the reference's error codes and calls
    marlin_gemm on an empty problem, which returns before touching a GPU."""
    import shutil
    import subprocess
    if shutil.which("gcc") is None:
        pytest.skip("no C compiler")
    src = tmp_path / "consumer.c"
    src.write_text(r'''
#include <stdio.h>
#include "marlin_amd_tools.h"
#include "marlin_amd_probe.h"
int main(void) {
  /* k = 64 with thread_k = 128: the problem does not fit the tile */
  if (marlin_amd_check(16, 256, 64, -1, 128, 128) != MARLIN_ERR_PROB_SHAPE) return 1;
  /* group size 32: no kernel */
  if (marlin_amd_check(16, 256, 512, 32, -1, -1) != MARLIN_ERR_KERN_SHAPE) return 2;
  if (marlin_amd_check(16, 256, 512, 128, -1, -1) != MARLIN_OK) return 3;
  /* an empty problem is fine and launches nothing (reference marlin_cute_kernel.cu:56-60) */
  if (marlin_gemm(0, 0, 0, 0, 0, 256, 512, 0, 128, 0, 0, -1, -1, -1, 16) != MARLIN_OK) return 4;
  if (marlin_cute(0, 0, 0, 0, 16, 0, 512, 0, -1, 0, 0, -1, -1, -1, 16) != MARLIN_OK) return 5;
  if (marlin_official(0, 0, 0, 0, 16, 256, 0, 0, -1, 0, 0, -1, -1, -1, 16) != MARLIN_OK) return 6;
  if (marlin_gemm_static(0, 0, 0, 0, 0, 256, 512, 0, 128, 0, 0, -1, -1, -1, 16) != MARLIN_OK) return 7;
  /* the probe library beside it: an unknown kind is refused before any GPU call */
  if (marlin_amd_probe(7, 0, 1, 256, 512, 0, 0) != MARLIN_ERR_PROB_SHAPE) return 8;
  if (marlin_amd_probe_last_error()[0] != 0) return 9;
  printf("%s\n", marlin_amd_version());
  return 0;
}
''')
    libdir = os.path.join(ROOT, "awesome-cute_amd")
    inc = os.path.join(ROOT, "include")
    for cc, std in (("gcc", "-std=c11"), ("g++", "-std=c++11")):
        exe = tmp_path / f"consumer_{cc}"
        cmd = [cc, std, "-Wall", "-Werror", "-pedantic", "-I", inc]
        cmd += ["-x", "c++"] if cc == "g++" else []
        cmd += [str(src), "-o", str(exe), "-L", libdir, "-lmarlin_amd_probe", "-lmarlin_amd",
                "-Wl,-rpath," + libdir, "-Wl,--allow-shlib-undefined"]
        res = subprocess.run(cmd, capture_output=True, text=True)
        assert res.returncode == 0, res.stderr
        run = subprocess.run([str(exe)], capture_output=True, text=True)
        assert run.returncode == 0, (run.returncode, run.stdout, run.stderr)
        assert "marlin_amd" in run.stdout
