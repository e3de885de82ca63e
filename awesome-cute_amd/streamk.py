"""Dense fp16 GEMM with a stream-K tail (the reference's gemm/streamk_gemm) over
the C ABI of libmarlin_amd.so: C = A @ B.T with A (m, k) and B (n, k) in fp16,
fp32 accumulation.  The GEMM always runs in the HIP library; a missing library
is an import-time error."""
import ctypes
import os

import torch

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "libmarlin_amd.so")
if not os.path.exists(_LIB_PATH):
    raise ImportError(
        f"{_LIB_PATH} is missing: build it first (python __graft_entry__.py build, or "
        "python awesome-cute_amd/build.py); the GEMM has no other implementation")
_lib = ctypes.CDLL(_LIB_PATH)
_P, _I = ctypes.c_void_p, ctypes.c_int
_lib.streamk_gemm_tn.restype = _I
_lib.streamk_gemm_tn.argtypes = [_P, _P, _P, _I, _I, _I, _I, _P]
_lib.streamk_amd_check.restype = _I
_lib.streamk_amd_check.argtypes = [_I, _I, _I]
_lib.streamk_amd_plan.restype = _I
_lib.streamk_amd_plan.argtypes = [_I, _I, _I, _I, _P]
_lib.streamk_amd_tile_coord.restype = None
_lib.streamk_amd_tile_coord.argtypes = [_I, _I, _I, _P]
_lib.streamk_amd_last_error.restype = ctypes.c_char_p


def check(m, n, k):
    """Return code streamk_gemm_tn would give for these sizes (no GPU touched)."""
    return _lib.streamk_amd_check(m, n, k)


def plan(m, n, k, cus=256):
    """The split of the output tiles (tile_rows x tile_cols) into data-parallel and stream-K tiles."""
    out = (ctypes.c_int * 8)()
    rc = _lib.streamk_amd_plan(m, n, k, cus, out)
    keys = ("tiles_m", "tiles_n", "dp_tiles", "sk_tiles", "k_slices", "grid", "tile_rows", "tile_cols")
    return rc, dict(zip(keys, out))


def tile_coord(tile, tiles_m, tiles_n):
    """(row tile, column tile) of a tile number."""
    out = (ctypes.c_int * 2)()
    _lib.streamk_amd_tile_coord(tile, tiles_m, tiles_n, out)
    return out[0], out[1]


def gemm(A, B, C=None):
    """C (m, n) = A (m, k) @ B (n, k).T on the current stream; returns C."""
    for name, t in (("A", A), ("B", B)):
        if t.dtype != torch.half or not t.is_cuda or not t.is_contiguous() or t.dim() != 2:
            raise ValueError(f"{name} must be a contiguous 2-d torch.half tensor on the GPU")
    m, k = A.shape
    n = B.shape[0]
    if B.shape[1] != k:
        raise ValueError("A and B must have the same k")
    if C is None:
        C = torch.empty((m, n), dtype=torch.half, device=A.device)
    elif C.shape != (m, n) or C.dtype != torch.half or not C.is_contiguous() or C.device != A.device:
        raise ValueError("C must be a contiguous (m, n) torch.half tensor on A's device")
    dev = A.get_device()
    stream = torch.cuda.current_stream(dev).cuda_stream
    rc = _lib.streamk_gemm_tn(A.data_ptr(), B.data_ptr(), C.data_ptr(), m, n, k, dev, stream)
    if rc == 1:
        raise ValueError(f"shape (m={m}, n={n}, k={k}) not supported: n must be a multiple of 256, "
                         "k of 64")
    if rc != 0:
        raise RuntimeError("streamk_gemm_tn: " + _lib.streamk_amd_last_error().decode())
    return C
