#!/usr/bin/env python3
"""Writes tests/golden/w4a16_known_answers.npz and tests/golden/f16_gemm_known_answers.npz.

The reference keeps no golden vectors for this path, and nothing of it was
imported or run to make these: they are known answers produced by this
repository's own CPU oracle (oracle/w4a16_ref.c) after it had been pinned by
tests/test_oracle.py, frozen here so that a later change to the oracle, the
packers or the kernels that alters any bit shows up as a diff against data
instead of passing silently.  Two small problems (group 128 and per-channel
scales): logical int4 weights and scales, their packed forms, activations, the
dequantised weight matrix, the fp32-accumulate GEMM result, and the three
layout permutations.  For the dense fp16 GEMM (whose reference program keeps
no vectors either): two small problems with their fp32-accumulate results.

Run from the repository root:  python tests/golden/make_fixtures.py
"""
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(HERE))
import _oracle as O  # noqa: E402


def problem(M, N, K, groupsize, seed):
    rng = np.random.default_rng(seed)
    A = rng.standard_normal((M, K)).astype(np.float16)
    q = rng.integers(0, 16, (K, N), dtype=np.uint8)
    groups = K // groupsize if groupsize != -1 else 1
    s = rng.uniform(0.001, 0.02, (groups, N)).astype(np.float16)
    B = O.pack_weights(q)
    sp = O.pack_scales(s, groupsize != -1)
    W = O.dequant(B, sp, K, N, groupsize)
    C = O.gemm(A, B, sp, N, groupsize)
    return {"A": A.view(np.uint16), "q": q, "s": s.view(np.uint16), "B": B,
            "s_packed": sp.view(np.uint16), "W": W.view(np.uint16), "C": C.view(np.uint16)}


def main():
    out = {}
    for tag, (M, N, K, g, seed) in {"g128": (5, 256, 256, 128, 11),
                                    "chan": (3, 256, 128, -1, 12)}.items():
        for k, v in problem(M, N, K, g, seed).items():
            out[f"{tag}_{k}"] = v
    perm, sp, sps = O.get_perms()
    out["perm"], out["scale_perm"], out["scale_perm_single"] = perm, sp, sps
    path = os.path.join(HERE, "w4a16_known_answers.npz")
    np.savez_compressed(path, **out)
    print(path, os.path.getsize(path), "bytes")

    dense = {}
    for tag, (M, N, K, seed) in {"a": (40, 256, 192, 21), "b": (130, 256, 320, 22)}.items():
        rng = np.random.default_rng(seed)
        A = (rng.random((M, K)) * 4 - 2).astype(np.float16)
        B = (rng.random((N, K)) * 4 - 2).astype(np.float16)
        dense[f"{tag}_A"], dense[f"{tag}_B"] = A.view(np.uint16), B.view(np.uint16)
        dense[f"{tag}_C"] = O.dense_gemm_tn(A, B).view(np.uint16)
    path = os.path.join(HERE, "f16_gemm_known_answers.npz")
    np.savez_compressed(path, **dense)
    print(path, os.path.getsize(path), "bytes")


if __name__ == "__main__":
    main()
