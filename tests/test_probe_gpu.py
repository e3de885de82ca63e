"""The probe library beside the product library (libmarlin_amd_probe.so,
include/marlin_amd_probe.h): its launches run, refuse what they do not support,
and give figures of the right order.  The probes have no counterpart in the
reference; bench.py uses them for the floor beside every row and for
`--facts`, so a broken probe would silently spoil the evidence.
"""
import os
import sys

import numpy as np
import pytest

pytestmark = pytest.mark.gpu

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
sys.path.insert(0, os.path.join(ROOT, "awesome-cute_amd"))


@pytest.fixture(scope="module")
def env():
    import torch
    import marlin
    assert torch.cuda.is_available()
    return torch, marlin


def test_launch_probes_run_and_refuse_bad_arguments(env):
    torch, marlin = env
    n, k = 1024, 1024
    B = torch.randint(-2**31, 2**31 - 1, (k // 16, 2 * n), dtype=torch.int32, device="cuda")
    assert marlin.plan(1, n, k, 128)[1]["kernel"] == 3
    for kind in (0, 1, 2):
        marlin.probe(kind, B, n, k)         # the column-strip kernel's split
        marlin.probe(kind, B, n, k, m=2048)  # prefill rows: the split of 16 rows
        assert marlin.plan(64, n, k, 128)[1]["row_parts"] == 4
        marlin.probe(kind, B, n, k, m=64)   # column strips, the rows in four parts
        marlin.force_kernel(4)              # (the probe library asks with the thread's overrides)
        try:
            assert marlin.plan(64, n, k, 128)[1]["kernel"] == 1
            marlin.probe(kind, B, n, k, m=64)   # the streaming kernel's split
        finally:
            marlin.force_kernel(0)
    for strips in (2, 4):
        marlin.force_strips(strips)
        try:
            marlin.probe(1, B, n, k)
        finally:
            marlin.force_strips(0)
    torch.cuda.synchronize()
    with pytest.raises(RuntimeError):
        marlin.probe(3, B, n, k)        # no such kind
    with pytest.raises(RuntimeError):
        marlin.probe(1, B, 1000, k)     # not a shape the GEMM accepts


def test_issue_probe_orders_the_mixes(env):
    """An MFMA of this shape takes 16-17 cycles of a lone wave; two VALU
    operations behind it cost (next to) nothing, a third and fourth do; a
    memory instruction per eight MFMAs costs less than a cycle per MFMA."""
    torch, marlin = env
    alone = marlin.probe_issue(0, iters=500, workgroups=64)
    assert 15.0 < alone < 19.0, alone
    two = marlin.probe_issue(2, iters=500, workgroups=64)
    four = marlin.probe_issue(4, iters=500, workgroups=64)
    assert alone - 0.2 <= two < alone + 2.5, (alone, two)
    assert four > two + 3.0, (two, four)
    lds = marlin.probe_issue(0, 1, 0, iters=500, workgroups=64)
    assert alone < lds < alone + 3.0, (alone, lds)
    with pytest.raises(RuntimeError):
        marlin.probe_issue(5)           # unsupported mix
    with pytest.raises(RuntimeError):
        marlin.probe_issue(1, 1, 1)


def test_pull_probe_scales_with_loads_in_flight(env):
    torch, marlin = env
    src = torch.empty(64 << 20, dtype=torch.uint8, device="cuda").random_(0, 255)
    one = marlin.probe_pull(src, 4 << 20, 1, 1)
    many = marlin.probe_pull(src, 4 << 20, 16, 1)
    assert one.shape == (1,) and many.shape == (1,)
    gbps_one = (4 << 20) / (float(one[0]) * 1e-6) / 1e9
    gbps_many = (4 << 20) / (float(many[0]) * 1e-6) / 1e9
    assert 2.0 < gbps_one < 40.0, gbps_one
    assert gbps_many > 2.0 * gbps_one, (gbps_one, gbps_many)
    us = marlin.probe_pull(src, 1 << 20, 4, 64)
    assert us.shape == (64,) and np.all(us > 0)
    with pytest.raises(RuntimeError):
        marlin.probe_pull(src, 4 << 20, 16, 17)      # 68 MiB of a 64 MiB buffer
    with pytest.raises(RuntimeError):
        marlin.probe_pull(src, 4 << 20, 3, 1)        # depth 3 is not built
