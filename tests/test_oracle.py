"""Pins the CPU oracle (oracle/w4a16_ref.c) without using its own formulae.

The reference holds no golden vectors for the W4A16 path, so each oracle
function is checked against numpy's independent fp16 arithmetic, against a
second derivation of the same quantity, or against closed forms.
"""
import os

import numpy as np
import pytest

import _oracle as O


# ------------------------------------------------------------------ soft fp16

def test_f16_to_f32_exhaustive():
    bits = np.arange(65536, dtype=np.uint16)
    want = bits.view(np.float16).astype(np.float32)
    got = np.array([O.lib.ref_f16_to_f32(int(b)) for b in bits], np.float32)
    nan = np.isnan(want)
    assert nan.sum() == 2 * 1023 and np.isnan(got[nan]).all()
    # signalling NaNs are quieted on the way back through the C float ABI
    assert np.array_equal(got.view(np.uint32)[~nan], want.view(np.uint32)[~nan])


def test_f32_to_f16_against_numpy():
    rng = np.random.default_rng(1)
    # every half, every midpoint between adjacent halves, and their neighbours
    halves = np.arange(0x7c00, dtype=np.uint16).view(np.float16).astype(np.float64)
    mids = (halves[:-1] + halves[1:]) / 2
    cases = np.concatenate([
        halves, mids, np.nextafter(mids.astype(np.float32), np.float32(np.inf)),
        np.nextafter(mids.astype(np.float32), np.float32(-np.inf)),
        [65504.0, 65519.9, 65520.0, 70000.0, 1e-8, 2.0 ** -25, 2.0 ** -24 * 1.5,
         np.inf, 0.0],
        rng.standard_normal(20000) * 10.0 ** rng.integers(-8, 5, 20000),
    ]).astype(np.float32)
    cases = np.concatenate([cases, -cases])
    with np.errstate(over="ignore"):
        want = cases.astype(np.float16).view(np.uint16)
    got = np.array([O.lib.ref_f32_to_f16(float(x)) for x in cases], np.uint16)
    assert np.array_equal(got, want)
    assert O.lib.ref_f32_to_f16(float("nan")) & 0x7c00 == 0x7c00
    assert O.lib.ref_f32_to_f16(float("nan")) & 0x03ff != 0


def test_f64_to_f16_single_rounding():
    # 1 + 2^-11 + 2^-30 lies just above a tie: rounding through float32 first
    # would land on the tie and round to even (1.0); one rounding gives 1+2^-10
    x = 1.0 + 2.0 ** -11 + 2.0 ** -30
    assert O.lib.ref_f64_to_f16(x) == 0x3c01
    assert O.lib.ref_f64_to_f16(1.0 + 2.0 ** -11) == 0x3c00
    assert O.lib.ref_f64_to_f16(1.0 + 3 * 2.0 ** -11) == 0x3c02


def test_f16_mul_against_numpy():
    rng = np.random.default_rng(2)
    a = rng.integers(0, 0x7c00, 50000).astype(np.uint16)
    b = rng.integers(0, 0x7c00, 50000).astype(np.uint16)
    a[::3] |= 0x8000
    with np.errstate(over="ignore"):
        want = (a.view(np.float16).astype(np.float64) * b.view(np.float16).astype(np.float64))
        want = want.astype(np.float16).view(np.uint16)
    got = np.array([O.lib.ref_f16_mul(int(x), int(y)) for x, y in zip(a, b)], np.uint16)
    assert np.array_equal(got, want)


# --------------------------------------------------------------- permutations

def test_perm_is_bijection_and_spot_value():
    perm, sp, sps = O.get_perms()
    assert sorted(perm.tolist()) == list(range(1024))
    assert sorted(sp.tolist()) == list(range(64))
    assert sorted(sps.tolist()) == list(range(32))
    # lane 5 = (t=1, c=1): rows 2,3,10,11 of columns 1 and 9, low nibble first
    # in the order the dequantiser consumes them (nibble e <-> e&1: +8 rows,
    # e>>1&1: +8 columns, e>>2: odd row); derived by hand from marlin.py:29-48
    assert perm[5 * 32:5 * 32 + 8].tolist() == [33, 161, 41, 169, 49, 177, 57, 185]
    assert sp[:10].tolist() == [0, 8, 16, 24, 32, 40, 48, 56, 1, 9]
    assert sps[:10].tolist() == [0, 1, 8, 9, 16, 17, 24, 25, 2, 3]


def test_perm_matches_closed_form_everywhere():
    """Transcribed permutation (marlin.py) == layout the kernels consume."""
    perm, _, _ = O.get_perms()
    import ctypes
    k = ctypes.c_int()
    n = ctypes.c_int()
    for p in range(1024):
        word, e = divmod(p, 8)
        O.lib.marlin_weight_coord(0, word, e, ctypes.byref(k), ctypes.byref(n))
        # perm indexes a row of four 16x16 tiles stored tile after tile
        tile, col = divmod(n.value, 16)
        assert perm[p] == 256 * tile + 16 * k.value + col, p


def _numpy_pack(q):
    """numpy restatement of the tiling / gather / nibble packing, written
    against the closed-form coordinates only."""
    K, N = q.shape
    B = np.zeros((K // 16, 2 * N), np.uint32)
    kt = np.arange(K // 16)[:, None]
    w = np.arange(2 * N)[None, :]
    n64, lane, j = w // 128, (w % 128) // 4, w % 4
    t, c = lane % 4, lane // 4
    for e in range(8):
        k = 16 * kt + 2 * t + ((e >> 2) & 1) + 8 * (e & 1)
        n = 64 * n64 + 16 * j + c + 8 * ((e >> 1) & 1)
        B |= q[k, n].astype(np.uint32) << np.uint32(4 * e)
    return B.view(np.int32)


@pytest.mark.parametrize("K,N", [(16, 64), (64, 128), (128, 256), (512, 256)])
def test_pack_two_derivations_agree(K, N):
    rng = np.random.default_rng(K * 1000 + N)
    q = rng.integers(0, 16, (K, N), dtype=np.uint8)
    B = O.pack_weights(q)
    assert np.array_equal(B, _numpy_pack(q))
    assert np.array_equal(O.unpack_weights(B, K, N), q)


def test_pack_single_weight_lands_where_dequant_reads_it():
    # one non-zero weight at (k=10, n=9): Marlin lane t=1 (rows 2,3,10,11),
    # c=1, tile j=0, +8 rows -> e&1, +8 cols -> e>>1&1  => nibble 3 of word
    # (4c+t)*4 + j = 20
    q = np.zeros((16, 64), np.uint8)
    q[10, 9] = 0xF
    B = O.pack_weights(q)
    assert B.shape == (1, 128)
    nz = np.nonzero(B[0])[0].tolist()
    assert nz == [20]
    assert (int(B[0, 20]) & 0xFFFFFFFF) == 0xF << 12


@pytest.mark.parametrize("groupwise", [True, False])
def test_scale_perm_two_derivations_agree(groupwise):
    rng = np.random.default_rng(3)
    G, N = (4, 256) if groupwise else (1, 256)
    s = rng.uniform(0.001, 0.02, (G, N)).astype(np.float16)
    sp = O.pack_scales(s, groupwise)
    assert np.array_equal(O.unpack_scales(sp, groupwise).view(np.uint16), s.view(np.uint16))
    # what a reader sees: groupwise lane c of block b reads 8 consecutive
    # halves = columns c + 8j; single: lane t reads columns 2t+{0,1,8,9,...}
    if groupwise:
        for b in range(N // 64):
            for c in range(8):
                got = sp[1, 64 * b + 8 * c:64 * b + 8 * c + 8]
                want = s[1, [64 * b + c + 8 * j for j in range(8)]]
                assert np.array_equal(got, want)
    else:
        offs = [0, 1, 8, 9, 16, 17, 24, 25]
        for b in range(N // 32):
            for t in range(4):
                got = sp[0, 32 * b + 8 * t:32 * b + 8 * t + 8]
                want = s[0, [32 * b + 2 * t + o for o in offs]]
                assert np.array_equal(got, want)


# ------------------------------------------------------------- dequantisation

def test_dequant_magic_exhaustive():
    out = (np.zeros(4, np.uint16))
    for lo0 in range(16):
        for hi0 in range(16):
            for lo1 in range(16):
                # nibbles 0,1 (low half) and 4,5 (high half); others = noise
                q = lo0 | (hi0 << 4) | (0xA5 << 8) | (lo1 << 16) | ((15 - hi0) << 20) | (0x5A << 24)
                qs = q - (1 << 32) if q >= 1 << 31 else q
                O.lib.marlin_dequant_magic(qs, O._p(out))
                want = np.array([lo0 - 8, lo1 - 8, hi0 - 8, (15 - hi0) - 8], np.float16)
                assert np.array_equal(out, want.view(np.uint16)), hex(q)


@pytest.mark.parametrize("groupsize", [128, -1])
def test_dequant_ref_against_numpy(groupsize):
    K, N = 256, 128
    A, q, s, B, sp = O.make_problem(1, N, K, groupsize, seed=5)
    W = O.dequant(B, sp, K, N, groupsize)
    base = (q.astype(np.int32) - 8).astype(np.float16)
    if groupsize > 0:
        want = base * np.repeat(s, groupsize, axis=0)  # numpy: float16 RN multiply
        assert want.dtype == np.float16
    else:
        want = base
    assert np.array_equal(W.view(np.uint16), want.view(np.uint16))


def test_scale_multiply_exhaustive_single_rounding():
    """RN_fp16((q-8)*s) for all 16 q and every finite positive fp16 scale."""
    s_bits = np.arange(1, 0x7c00, dtype=np.uint16)
    s = s_bits.view(np.float16)
    for qv in range(16):
        v = np.float16(qv - 8)
        with np.errstate(over="ignore"):
            want = (np.float64(v) * s.astype(np.float64)).astype(np.float16).view(np.uint16)
        vb = int(np.array([v]).view(np.uint16)[0])
        got = np.array([O.lib.ref_f16_mul(vb, int(b)) for b in s_bits[::7]], np.uint16)
        assert np.array_equal(got, want[::7])


# ----------------------------------------------------------------------- GEMM

@pytest.mark.parametrize("groupsize", [128, -1])
def test_gemm_ref_against_f64_bruteforce(groupsize):
    M, N, K = 5, 64, 256
    A, q, s, B, sp = O.make_problem(M, N, K, groupsize, seed=7)
    C = O.gemm(A, B, sp, N, groupsize).astype(np.float64)
    C64 = O.gemm_f64(A, B, sp, N, groupsize)
    # independent numpy float64 evaluation from the logical q / s
    W = (q.astype(np.float64) - 8)
    if groupsize > 0:
        W = (W.astype(np.float16) * np.repeat(s, groupsize, axis=0)).astype(np.float64)
        want = A.astype(np.float64) @ W
    else:
        want = (A.astype(np.float64) @ W) * s.astype(np.float64)
    assert np.allclose(C64, want, rtol=1e-12, atol=1e-12)
    # fp32 accumulation + fp16 rounding error budget
    tol = 2e-3 * np.abs(want).max()
    assert np.abs(C - want).max() <= tol


def test_gemm_ref_closed_forms():
    M, N, K = 16, 128, 256
    rng = np.random.default_rng(11)
    A = rng.standard_normal((M, K)).astype(np.float16)
    # all weights at the zero point -> exactly zero
    q = np.full((K, N), 8, np.uint8)
    s = rng.uniform(0.001, 0.02, (K // 128, N)).astype(np.float16)
    C = O.gemm(A, O.pack_weights(q), O.pack_scales(s, True), N, 128)
    assert not C.view(np.uint16).any()
    # unit scales and small-integer activations -> exact integers
    Ai = rng.integers(-3, 4, (M, K)).astype(np.float16)
    q = rng.integers(0, 16, (K, N), dtype=np.uint8)
    ones = np.ones((K // 128, N), np.float16)
    C = O.gemm(Ai, O.pack_weights(q), O.pack_scales(ones, True), N, 128)
    want = Ai.astype(np.int64) @ (q.astype(np.int64) - 8)
    assert np.abs(want).max() < 2048  # exactly representable in fp16
    assert np.array_equal(C.astype(np.int64), want)


@pytest.mark.parametrize("groupsize", [128, -1])
def test_gemm_ref_one_hot_rows_return_weights_bit_exact(groupsize):
    N, K = 128, 256
    _, q, s, B, sp = O.make_problem(1, N, K, groupsize, seed=13)
    rows = [0, 1, 9, 127, 128, 255]
    A = np.zeros((len(rows), K), np.float16)
    for i, r in enumerate(rows):
        A[i, r] = 1.0
    C = O.gemm(A, B, sp, N, groupsize)
    base = (q.astype(np.int32) - 8).astype(np.float16)
    if groupsize > 0:
        W = base * np.repeat(s, groupsize, axis=0)
    else:
        W = base * s  # fp16(fp16(q-8)) * s == one RN multiply
    assert np.array_equal(C.view(np.uint16), W[rows].view(np.uint16))


def test_gemm_ref_threads_do_not_change_bits():
    M, N, K = 3, 512, 256
    A, q, s, B, sp = O.make_problem(M, N, K, 128, seed=17)
    c1 = O.gemm(A, B, sp, N, 128, threads=1)
    c8 = O.gemm(A, B, sp, N, 128, threads=0)
    assert np.array_equal(c1.view(np.uint16), c8.view(np.uint16))


def test_config1_shape_runs():
    # smallest benchmark config: M=16, N=256, K=512, group 128 (marlin_test.py:123-131)
    A, q, s, B, sp = O.make_problem(16, 256, 512, 128, seed=0)
    assert B.shape == (32, 512) and sp.shape == (4, 256)
    C = O.gemm(A, B, sp, 256, 128)
    want = A.astype(np.float64) @ ((q.astype(np.int32) - 8).astype(np.float16)
                                   * np.repeat(s, 128, axis=0)).astype(np.float64)
    r = O.compare(C, want.astype(np.float16))
    assert r.max_abs_err <= 1e-2 * r.max_abs_ref


# ------------------------------------------------------------------ quantiser

@pytest.mark.parametrize("groupsize", [128, -1])
def test_gen_quant4_invariants(groupsize):
    K, N = 256, 64
    rng = np.random.default_rng(19)
    w = rng.standard_normal((K, N)).astype(np.float16)
    q, s, ref = O.gen_quant4(w, groupsize)
    gs = groupsize if groupsize > 0 else K
    sfull = np.repeat(s.astype(np.float64), gs, axis=0)
    assert q.min() >= 0 and q.max() <= 15
    assert np.array_equal(ref.view(np.uint16),
                          ((q.astype(np.int32) - 8).astype(np.float16)
                           * np.repeat(s, gs, axis=0)).view(np.uint16))
    # inside the clamp range the error is at most half a step (+ fp16 slack)
    inside = (q > 0) & (q < 15)
    err = np.abs(ref.astype(np.float64) - w.astype(np.float64))
    assert (err[inside] <= 0.5 * sfull[inside] * 1.01 + 1e-3).all()
    # the group maximum maps to +7 or -7.5 -> q in {15, 0 or 1}
    for g in range(K // gs):
        blk = np.abs(w[g * gs:(g + 1) * gs].astype(np.float64))
        k = blk.argmax(axis=0) + g * gs
        qq = q[k, np.arange(N)]
        assert np.isin(qq, [0, 1, 15]).all()


def test_compare_helper():
    a = np.array([1.0, 2.0, -3.0], np.float16)
    b = np.array([1.0, 2.5, -3.0], np.float16)
    r = O.compare(a, b)
    assert r.max_abs_err == 0.5 and r.max_abs_ref == 3.0
    assert r.mismatched_bits == 1
    assert abs(r.rel_mean_abs_err - 0.5 / 6.5) < 1e-12
    a[0] = np.nan
    assert np.isnan(O.compare(a, b).max_abs_err)


# ---------------------------------------------------------------- frozen known answers

def _golden():
    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden",
                        "w4a16_known_answers.npz")
    return np.load(path)  # allow_pickle stays False


@pytest.mark.parametrize("tag,groupsize", [("g128", 128), ("chan", -1)])
def test_oracle_reproduces_frozen_known_answers(tag, groupsize):
    """tests/golden/w4a16_known_answers.npz (written by tests/golden/make_fixtures.py
    from this oracle once pinned): packers, dequantiser and GEMM still give the
    same bits."""
    g = _golden()
    q, s = g[f"{tag}_q"], g[f"{tag}_s"].view(np.float16)
    K, N = q.shape
    B = O.pack_weights(q)
    sp = O.pack_scales(s, groupsize != -1)
    assert np.array_equal(B, g[f"{tag}_B"])
    assert np.array_equal(sp.view(np.uint16), g[f"{tag}_s_packed"])
    assert np.array_equal(O.dequant(B, sp, K, N, groupsize).view(np.uint16), g[f"{tag}_W"])
    A = g[f"{tag}_A"].view(np.float16)
    assert np.array_equal(O.gemm(A, B, sp, N, groupsize).view(np.uint16), g[f"{tag}_C"])
    perm, scale_perm, scale_perm_single = O.get_perms()
    assert np.array_equal(perm, g["perm"]) and np.array_equal(scale_perm, g["scale_perm"])
    assert np.array_equal(scale_perm_single, g["scale_perm_single"])
