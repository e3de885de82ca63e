"""ctypes face of the CPU oracle (oracle/libw4a16_ref.so).  Test helper only."""
import ctypes
import os
import subprocess

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
_SO = os.path.join(ROOT, "oracle", "libw4a16_ref.so")


def _load():
    if not os.path.exists(_SO):
        subprocess.check_call(["make", "-C", os.path.join(ROOT, "oracle")])
    lib = ctypes.CDLL(_SO)
    c = ctypes
    P = c.c_void_p
    lib.ref_f16_to_f32.restype = c.c_float
    lib.ref_f16_to_f32.argtypes = [c.c_uint16]
    lib.ref_f32_to_f16.restype = c.c_uint16
    lib.ref_f32_to_f16.argtypes = [c.c_float]
    lib.ref_f64_to_f16.restype = c.c_uint16
    lib.ref_f64_to_f16.argtypes = [c.c_double]
    for name in ("ref_f16_mul", "ref_f16_sub"):
        getattr(lib, name).restype = c.c_uint16
        getattr(lib, name).argtypes = [c.c_uint16, c.c_uint16]
    lib.ref_f16_fma.restype = c.c_uint16
    lib.ref_f16_fma.argtypes = [c.c_uint16] * 3
    lib.marlin_get_perms.argtypes = [P, P, P]
    lib.marlin_pack_weights.argtypes = [P, c.c_int, c.c_int, P]
    lib.marlin_pack_scales.argtypes = [P, c.c_int, c.c_int, c.c_int, P]
    lib.marlin_weight_coord.argtypes = [c.c_int, c.c_int, c.c_int, P, P]
    lib.marlin_unpack_weights.argtypes = [P, c.c_int, c.c_int, P]
    lib.marlin_scale_index_group.restype = c.c_int
    lib.marlin_scale_index_group.argtypes = [c.c_int]
    lib.marlin_scale_index_single.restype = c.c_int
    lib.marlin_scale_index_single.argtypes = [c.c_int]
    lib.marlin_unpack_scales.argtypes = [P, c.c_int, c.c_int, c.c_int, P]
    lib.marlin_dequant_magic.argtypes = [c.c_int32, P]
    lib.w4a16_dequant_ref.argtypes = [P, P, c.c_int, c.c_int, c.c_int, P]
    lib.w4a16_gemm_ref.restype = c.c_int
    lib.w4a16_gemm_ref.argtypes = [P, P, P, P] + [c.c_int] * 5
    lib.w4a16_gemm_ref_f64.argtypes = [P, P, P, P] + [c.c_int] * 4
    lib.gen_quant4_ref.argtypes = [P, c.c_int, c.c_int, c.c_int, P, P, P]
    lib.w4a16_compare.argtypes = [P, P, c.c_size_t, P]
    lib.w4a16_ref_max_threads.restype = c.c_int
    lib.f16_gemm_tn_ref.restype = c.c_int
    lib.f16_gemm_tn_ref.argtypes = [P, P, P] + [c.c_int] * 4
    return lib


lib = _load()


def _p(a):
    return a.ctypes.data_as(ctypes.c_void_p)


def get_perms():
    perm = np.zeros(1024, np.int32)
    sp = np.zeros(64, np.int32)
    sps = np.zeros(32, np.int32)
    lib.marlin_get_perms(_p(perm), _p(sp), _p(sps))
    return perm, sp, sps


def pack_weights(q):
    q = np.ascontiguousarray(q, np.uint8)
    K, N = q.shape
    B = np.zeros((K // 16, 2 * N), np.int32)
    lib.marlin_pack_weights(_p(q), K, N, _p(B))
    return B


def unpack_weights(B, K, N):
    B = np.ascontiguousarray(B, np.int32)
    q = np.zeros((K, N), np.uint8)
    lib.marlin_unpack_weights(_p(B), K, N, _p(q))
    return q


def pack_scales(s, groupwise):
    s = np.ascontiguousarray(s).view(np.uint16)
    G, N = s.shape
    out = np.zeros((G, N), np.uint16)
    lib.marlin_pack_scales(_p(s), G, N, int(groupwise), _p(out))
    return out.view(np.float16)


def unpack_scales(sp, groupwise):
    sp = np.ascontiguousarray(sp).view(np.uint16)
    G, N = sp.shape
    out = np.zeros((G, N), np.uint16)
    lib.marlin_unpack_scales(_p(sp), G, N, int(groupwise), _p(out))
    return out.view(np.float16)


def dequant(B, sp, K, N, groupsize):
    B = np.ascontiguousarray(B, np.int32)
    sp = np.ascontiguousarray(sp).view(np.uint16)
    W = np.zeros((K, N), np.uint16)
    lib.w4a16_dequant_ref(_p(B), _p(sp), K, N, groupsize, _p(W))
    return W.view(np.float16)


def gemm(A, B, sp, N, groupsize, threads=0):
    A = np.ascontiguousarray(A).view(np.uint16)
    B = np.ascontiguousarray(B, np.int32)
    sp = np.ascontiguousarray(sp).view(np.uint16)
    M, K = A.shape
    C = np.zeros((M, N), np.uint16)
    rc = lib.w4a16_gemm_ref(_p(A), _p(B), _p(sp), _p(C), M, N, K, groupsize, threads)
    assert rc == 0
    return C.view(np.float16)


def dense_gemm_tn(A, B, threads=0):
    """A (M, K) and B (N, K) float16 -> C (M, N) float16, fp32 accumulation."""
    A = np.ascontiguousarray(A).view(np.uint16)
    B = np.ascontiguousarray(B).view(np.uint16)
    M, K = A.shape
    N = B.shape[0]
    assert B.shape[1] == K
    C = np.zeros((M, N), np.uint16)
    rc = lib.f16_gemm_tn_ref(_p(A), _p(B), _p(C), M, N, K, threads)
    assert rc == 0
    return C.view(np.float16)


def gemm_f64(A, B, sp, N, groupsize):
    A = np.ascontiguousarray(A).view(np.uint16)
    B = np.ascontiguousarray(B, np.int32)
    sp = np.ascontiguousarray(sp).view(np.uint16)
    M, K = A.shape
    C = np.zeros((M, N), np.float64)
    lib.w4a16_gemm_ref_f64(_p(A), _p(B), _p(sp), _p(C), M, N, K, groupsize)
    return C


def gen_quant4(w, groupsize):
    w = np.ascontiguousarray(w).view(np.uint16)
    K, N = w.shape
    G = 1 if groupsize <= 0 else K // groupsize
    q = np.zeros((K, N), np.uint8)
    s = np.zeros((G, N), np.uint16)
    ref = np.zeros((K, N), np.uint16)
    lib.gen_quant4_ref(_p(w), K, N, groupsize, _p(q), _p(s), _p(ref))
    return q, s.view(np.float16), ref.view(np.float16)


class Compare(ctypes.Structure):
    _fields_ = [("max_abs_err", ctypes.c_double), ("max_abs_ref", ctypes.c_double),
                ("rel_mean_abs_err", ctypes.c_double), ("cosine", ctypes.c_double),
                ("mismatched_bits", ctypes.c_longlong)]


def compare(C, Cref):
    C = np.ascontiguousarray(C).view(np.uint16)
    Cref = np.ascontiguousarray(Cref).view(np.uint16)
    assert C.shape == Cref.shape
    out = Compare()
    lib.w4a16_compare(_p(C), _p(Cref), C.size, ctypes.byref(out))
    return out


def make_problem(M, N, K, groupsize, seed=0):
    """Seeded synthetic inputs with the benchmark's distributions: A ~ N(0,1)
    in fp16, weights uniform on {0..15} (zero point 8), scales ~ U(0.001, 0.02)
    in fp16.  Returns logical q / s and the Marlin-packed B / sp."""
    rng = np.random.default_rng(seed)
    A = rng.standard_normal((M, K), dtype=np.float32).astype(np.float16)
    q = rng.integers(0, 16, size=(K, N), dtype=np.uint8)
    G = 1 if groupsize <= 0 else K // groupsize
    s = rng.uniform(0.001, 0.02, size=(G, N)).astype(np.float16)
    B = pack_weights(q)
    sp = pack_scales(s, groupwise=(G > 1))
    return A, q, s, B, sp
