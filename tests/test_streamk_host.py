"""CPU-side tests of the dense stream-K GEMM: the C ABI is exported, the shape
contract, the split of the tiles into data-parallel and stream-K parts
(counterpart of dp_sk_block.h:82-128), the tile numbering, and the dense oracle
against numpy.  No kernel is launched here."""
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
def streamk():
    if not os.path.exists(LIB):
        pytest.fail("libmarlin_amd.so is not built; run `python __graft_entry__.py build`")
    import streamk as s
    return s


def test_library_exports_every_declared_symbol():
    text = open(os.path.join(ROOT, "include", "streamk_amd.h")).read()
    names = re.findall(r"\b(streamk_\w+)\s*\(", text)
    assert {"streamk_gemm_tn", "streamk_amd_plan", "streamk_amd_check"} <= set(names)
    lib = ctypes.CDLL(LIB)
    for n in set(names):
        assert hasattr(lib, n), n


@pytest.mark.parametrize("args,want", [
    ((4096, 4352, 4096), 0), ((1152, 4352, 4096), 0), ((1, 256, 64), 0), ((0, 256, 64), 0),
    ((16, 256, 0), 0), ((16, 0, 64), 0),
    ((16, 128, 64), 1), ((16, 4352 + 64, 4096), 1), ((16, 256, 32), 1), ((16, 256, 96), 1),
    ((-1, 256, 64), 1), ((16, -256, 64), 1),
])
def test_shape_contract(streamk, args, want):
    assert streamk.check(*args) == want


@pytest.mark.parametrize("cus", [256, 304, 64, 8])
def test_tile_split_properties(streamk, cus):
    rng = np.random.default_rng(cus)
    cases = [(4096, 4352, 4096), (4096, 4352, 10240), (1152, 4352, 4096), (4096, 4096, 4096),
             (2048, 2048, 2048), (8192, 8192, 8192), (300, 512, 320), (1, 256, 64)]
    cases += [(int(rng.integers(1, 9000)), 256 * int(rng.integers(1, 40)), 64 * int(rng.integers(1, 200)))
              for _ in range(200)]
    for m, n, k in cases:
        rc, p = streamk.plan(m, n, k, cus)
        assert rc == 0
        # 256 x 256 tiles; 128 x 256 when those would fill at most half the CUs; 128 x 128
        # when the 128 x 256 ones would, too
        large = -(-m // 256) * (n // 256)
        half = -(-m // 128) * (n // 256)
        assert p["tile_rows"] == (128 if 2 * large <= cus else 256)
        assert p["tile_cols"] == (128 if 2 * large <= cus and 2 * half <= cus else 256)
        tiles = -(-m // p["tile_rows"]) * (n // p["tile_cols"])
        assert p["tiles_m"] * p["tiles_n"] == tiles
        assert p["dp_tiles"] + p["sk_tiles"] == tiles
        assert p["grid"] == p["dp_tiles"] + p["sk_tiles"] * p["k_slices"]
        assert 1 <= p["k_slices"] <= 4
        if p["sk_tiles"]:
            # the stream-K part is the partial last wave, cut into at least two slices of
            # at least 256 k each, and fits the compute units and the partial-sum slots
            assert p["k_slices"] >= 2 and k // p["k_slices"] >= 256
            assert p["sk_tiles"] == tiles % cus and p["dp_tiles"] % cus == 0
            assert p["sk_tiles"] * p["k_slices"] <= min(cus, 256)
        else:
            assert p["k_slices"] == 1
            # nothing is split only when the tiles fill whole waves, a split cannot pay,
            # or two slices per tile would not fit the partial-sum slots
            rem = tiles % cus
            assert rem == 0 or cus // rem < 2 or k < 512 or rem * 2 > 256


def test_reference_shapes_use_the_stream_k_tail(streamk):
    """The reference's stream-K examples (gemm/readme.md:27-31) have tile counts that
    do not fill the compute units.  On 256 CUs the two with 272 large tiles get a
    stream-K part; the third has so few large tiles that it runs on 128-row tiles."""
    for m, n, k in [(4096, 4352, 4096), (4096, 4352, 10240)]:
        rc, p = streamk.plan(m, n, k, 256)
        assert rc == 0 and p["tile_rows"] == 256
        assert p["dp_tiles"] == 256 and p["sk_tiles"] == 16 and p["k_slices"] == 4, (m, n, k, p)
    rc, p = streamk.plan(1152, 4352, 4096, 256)
    assert rc == 0 and (p["tile_rows"], p["tile_cols"]) == (128, 256)
    assert p["dp_tiles"] + p["sk_tiles"] == 9 * 17
    # so few tiles that 128 x 128 ones fill the compute units without any k slices
    rc, p = streamk.plan(2048, 2048, 2048, 256)
    assert rc == 0 and (p["tile_rows"], p["tile_cols"]) == (128, 128)
    assert p["dp_tiles"] == 256 and p["sk_tiles"] == 0
    rc, p = streamk.plan(4096, 4096, 4096, 256)
    assert p["sk_tiles"] == 0 and p["dp_tiles"] == 256 and p["tile_rows"] == 256


@pytest.mark.parametrize("tm,tn", [(16, 17), (5, 17), (1, 1), (3, 8), (7, 9), (32, 32), (2, 40)])
def test_tile_numbering_is_a_bijection_in_panels(streamk, tm, tn):
    seen = set()
    for t in range(tm * tn):
        r, c = streamk.tile_coord(t, tm, tn)
        assert 0 <= r < tm and 0 <= c < tn
        seen.add((r, c))
    assert len(seen) == tm * tn
    # a run of 8 * tm numbers is one panel: all rows, 8 (or the last few) columns
    first = [streamk.tile_coord(t, tm, tn) for t in range(min(8, tn) * tm)]
    assert {c for _, c in first} == set(range(min(8, tn)))
    assert {r for r, _ in first} == set(range(tm))


def test_dense_oracle_against_numpy():
    """f16_gemm_tn_ref is pinned by an independent routine: exact equality with numpy's
    float64 product where every sum is exactly representable (small integers), and
    agreement to fp16 rounding for random inputs.  A transposed operand or a
    dropped k term fails both."""
    rng = np.random.default_rng(0)
    for m, n, k in [(3, 5, 7), (17, 32, 64), (64, 48, 96)]:
        A = rng.integers(-4, 5, (m, k)).astype(np.float16)
        B = rng.integers(-4, 5, (n, k)).astype(np.float16)
        want = (A.astype(np.float64) @ B.astype(np.float64).T)
        assert np.abs(want).max() < 2048
        got = O.dense_gemm_tn(A, B)
        assert np.array_equal(got.astype(np.float64), want)
    A = rng.standard_normal((33, 200)).astype(np.float16)
    B = rng.standard_normal((40, 200)).astype(np.float16)
    want = A.astype(np.float64) @ B.astype(np.float64).T
    got = O.dense_gemm_tn(A, B).astype(np.float64)
    # one fp16 rounding (2^-11 relative) plus fp32 accumulation error
    assert np.all(np.abs(got - want) <= np.abs(want) * 2.0 ** -10 + 1e-2)
    assert O.dense_gemm_tn(np.zeros((4, 0), np.float16), np.zeros((8, 0), np.float16)).any() == False


def test_gemm_refuses_cpu_tensors(streamk):
    import torch
    with pytest.raises(ValueError):
        streamk.gemm(torch.zeros((16, 64), dtype=torch.half), torch.zeros((256, 64), dtype=torch.half))


def test_dense_oracle_reproduces_frozen_known_answers():
    """tests/golden/f16_gemm_known_answers.npz (this repository's own known answers, the
    reference program keeps none): the oracle still gives every bit of them."""
    z = np.load(os.path.join(ROOT, "tests", "golden", "f16_gemm_known_answers.npz"))
    for tag in ("a", "b"):
        A, B = z[f"{tag}_A"].view(np.float16), z[f"{tag}_B"].view(np.float16)
        assert np.array_equal(O.dense_gemm_tn(A, B).view(np.uint16), z[f"{tag}_C"])
