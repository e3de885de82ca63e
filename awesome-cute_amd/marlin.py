"""Host-side mirror of the reference's `marlin` module (gemm/marlin_gemm/marlin.py)
over the C ABI of libmarlin_amd.so: `mul`, `Layer`, `replace_linear`, and the
packing permutations.  The GEMM itself always runs in the HIP library; there is
no fallback path, and a missing library is an import-time error.
"""
import ctypes
import os
import threading

import numpy as np
import torch
import torch.nn as nn

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "libmarlin_amd.so")

if not os.path.exists(_LIB_PATH):
    raise ImportError(
        f"{_LIB_PATH} is missing: build it first (python __graft_entry__.py build, or "
        "python awesome-cute_amd/build.py); the W4A16 GEMM has no other implementation")
_lib = ctypes.CDLL(_LIB_PATH)

_P = ctypes.c_void_p
_I = ctypes.c_int
_lib.marlin_mul.restype = _I
_lib.marlin_mul.argtypes = [_P, _P, _P, _P, _I, _I, _I, _I, _P, ctypes.c_longlong, _I, _P,
                            _I, _I, _I, _I, _I, ctypes.c_char_p, _I]
for _name in ("marlin_gemm", "marlin_cute", "marlin_official", "marlin_gemm_static"):
    getattr(_lib, _name).restype = _I
    getattr(_lib, _name).argtypes = [_P, _P, _P, _P, _I, _I, _I, _P, _I, _I, _P, _I, _I, _I, _I]
_lib.marlin_gemm_static_capacity.restype = ctypes.c_longlong
_lib.marlin_amd_scratch_bytes.restype = ctypes.c_longlong
_lib.marlin_amd_scratch_bytes.argtypes = [_I, _P]
_lib.marlin_amd_release.restype = ctypes.c_longlong
_lib.marlin_amd_release.argtypes = [_I]
_lib.marlin_amd_device_info.restype = _I
_lib.marlin_amd_device_info.argtypes = [_I, _P]
_lib.marlin_amd_check.restype = _I
_lib.marlin_amd_check.argtypes = [_I] * 6
_lib.marlin_amd_plan.restype = _I
_lib.marlin_amd_plan.argtypes = [_I] * 8 + [_P]
_lib.marlin_amd_force_k_slices.restype = None
_lib.marlin_amd_force_k_slices.argtypes = [_I]
_lib.marlin_amd_force_tile_rows.restype = None
_lib.marlin_amd_force_tile_rows.argtypes = [_I]
_lib.marlin_amd_force_row_halves.restype = None
_lib.marlin_amd_force_row_halves.argtypes = [_I]
_lib.marlin_amd_force_kernel.restype = None
_lib.marlin_amd_force_kernel.argtypes = [_I]
_lib.marlin_amd_plan_costs.restype = _I
_lib.marlin_amd_plan_costs.argtypes = [_I, _I, _I, _I, _I, _P]
_lib.marlin_amd_force_strips.restype = None
_lib.marlin_amd_force_strips.argtypes = [_I]
_lib.marlin_amd_work_order.restype = None
_lib.marlin_amd_work_order.argtypes = [_I, _P]
_lib.marlin_amd_last_error.restype = ctypes.c_char_p
_lib.marlin_amd_version.restype = ctypes.c_char_p


def mul(A, B, C, s, workspace, thread_k=-1, thread_n=-1, sms=-1, max_par=16, cute_version=True):
    """FP16 x INT4 multiply, C = A @ dequant(B); interface of reference marlin.py:11-24.

    A: (m, k) half, row-major.  B: (k/16, 2n) int32 in Marlin format (`Layer.pack`).
    C: (m, n) half, overwritten.  s: (k/groupsize, n) half scales, or (1, n).
    workspace: at least n/128*max_par zero int32 entries; zero again afterwards.
    thread_k / thread_n / sms: tile and grid hints, -1 = automatic.
    cute_version: accepted for compatibility; both values run the same kernels.
    Asynchronous on the current stream of A's device.  Raises RuntimeError where
    the reference binding raises (marlin_gemm.cpp:27-31,48-55).
    """
    if torch.compiler.is_compiling():
        # under torch.compile the call is one opaque operator that mutates C and
        # workspace (the reference advertises use within torch.compile, marlin.py:12)
        return torch.ops.marlin_amd.mul(A, B, C, s, workspace, thread_k, thread_n, sms, max_par,
                                        cute_version)
    _mul_eager(A, B, C, s, workspace, thread_k, thread_n, sms, max_par, cute_version)


def _mul_eager(A, B, C, s, workspace, thread_k, thread_n, sms, max_par, cute_version):
    if not (A.is_cuda and B.is_cuda and C.is_cuda and s.is_cuda and workspace.is_cuda):
        _complain((("A", A), ("B", B), ("C", C), ("s", s), ("workspace", workspace)), "is_cuda",
                  "must be a GPU tensor")
    if not (A.is_contiguous() and B.is_contiguous() and C.is_contiguous() and s.is_contiguous()
            and workspace.is_contiguous()):
        _complain((("A", A), ("B", B), ("C", C), ("s", s), ("workspace", workspace)),
                  "is_contiguous", "must be contiguous")
    dev = A.get_device()
    err = _errbuf()
    rc = _lib.marlin_mul(A.data_ptr(), B.data_ptr(), C.data_ptr(), s.data_ptr(),
                         A.size(0), C.size(1), A.size(1), s.size(0),
                         workspace.data_ptr(), workspace.numel(), dev, _raw_stream(dev),
                         thread_k, thread_n, sms, max_par, 1 if cute_version else 0,
                         err, 512)
    if rc != 0:
        raise RuntimeError(err.value.decode() or f"marlin_mul failed with code {rc}")


# The same call as an operator of torch's dispatcher, for compilers that trace
# Python: `mul` routes through it while torch.compile is tracing and calls the
# library directly otherwise (the dispatcher costs more host time than the
# one-row kernel takes).  It returns nothing; C and workspace are mutated.
@torch.library.custom_op("marlin_amd::mul", mutates_args=("C", "workspace"))
def _mul_op(A: torch.Tensor, B: torch.Tensor, C: torch.Tensor, s: torch.Tensor,
            workspace: torch.Tensor, thread_k: int, thread_n: int, sms: int, max_par: int,
            cute_version: bool) -> None:
    _mul_eager(A, B, C, s, workspace, thread_k, thread_n, sms, max_par, cute_version)


@_mul_op.register_fake
def _mul_fake(A, B, C, s, workspace, thread_k, thread_n, sms, max_par, cute_version):
    return None


def _complain(named, attr, what):
    for name, t in named:
        v = getattr(t, attr)
        if not (v() if callable(v) else v):
            raise RuntimeError(f"{name} {what}")


# The host side of a call matters at one row (the kernel takes 6.5 us): the
# error buffer is kept per thread, and the current stream is read through
# torch's raw-handle accessor where this torch build has it.
_tls = threading.local()


def _errbuf():
    buf = getattr(_tls, "err", None)
    if buf is None:
        buf = _tls.err = ctypes.create_string_buffer(512)
    return buf


_get_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)


def _raw_stream(dev):
    if _get_raw_stream is not None:
        return _get_raw_stream(dev)
    return torch.cuda.current_stream(dev).cuda_stream


# ---------------------------------------------------------------------------
# Packed layout.  Word w (0..127) of a 16 x 64 block belongs to Marlin lane
# w // 4 = 4c + t and 16-column tile j = w % 4; its nibble e holds
# k = 2t + (e >> 2 & 1) + 8 (e & 1),  n = 16 j + c + 8 (e >> 1 & 1).

def _block_coords():
    w = np.arange(128)[:, None]
    e = np.arange(8)[None, :]
    lane, j = w // 4, w % 4
    t, c = lane % 4, lane // 4
    k = 2 * t + ((e >> 2) & 1) + 8 * (e & 1)
    n = 16 * j + c + 8 * ((e >> 1) & 1)
    return k, n


def _get_perms():
    """Same three permutations as reference marlin.py:29-55, from the closed form:
    `perm` gathers a run of four row-major 16x16 tiles into nibble order."""
    k, n = _block_coords()
    perm = (256 * (n // 16) + 16 * k + n % 16).reshape(-1)
    scale_perm = [i + 8 * j for i in range(8) for j in range(8)]
    scale_perm_single = [2 * i + o for i in range(4) for o in (0, 1, 8, 9, 16, 17, 24, 25)]
    return torch.from_numpy(perm.astype(np.int64)), scale_perm, scale_perm_single


_perm, _scale_perm, _scale_perm_single = _get_perms()
_k_in_block, _n_in_block = _block_coords()
_block_gather = torch.from_numpy((64 * _k_in_block + _n_in_block).reshape(-1).astype(np.int64))


def pack_weights(q):
    """(k, n) integer tensor with values in [0, 15] -> (k/16, 2n) int32 Marlin words."""
    k, n = q.shape
    if k % 16 or n % 64:
        raise ValueError("k must be divisible by 16 and n by 64")
    blocks = q.reshape(k // 16, 16, n // 64, 64).permute(0, 2, 1, 3).reshape(k // 16, n // 64, 1024)
    nib = blocks[:, :, _block_gather.to(q.device)].reshape(k // 16, n // 64, 128, 8).to(torch.int64)
    shifts = torch.arange(0, 32, 4, device=q.device, dtype=torch.int64)
    words = (nib << shifts).sum(-1)  # < 2^32
    words = torch.where(words >= 2 ** 31, words - 2 ** 32, words)
    return words.reshape(k // 16, 2 * n).to(torch.int32)


def pack_scales(s, groupwise):
    """(groups, n) scales -> the order the kernels read them in (marlin.py:111-118)."""
    n = s.shape[1]
    if groupwise:
        out = s.reshape(-1, 64)[:, _scale_perm]
    else:
        out = s.reshape(-1, 32)[:, _scale_perm_single]
    return out.reshape(-1, n).contiguous()


def quantize(w, groupsize=-1):
    """Symmetric 4-bit quantisation of a (k, n) half weight, as the reference
    test helper gen_quant4 (marlin_test.py:18-40): per group and column
    s = max|w| * 2/15, q = clamp(round(w/s) + 8, 0, 15).  Returns the
    fake-quantised weight (k, n), q (k, n) int32 and s (groups, n)."""
    k, n = w.shape
    gs = k if groupsize == -1 else groupsize
    wg = w.reshape(k // gs, gs, n)
    s = wg.abs().amax(dim=1, keepdim=True)
    s = s * (2 / 15)
    q = torch.clamp(torch.round(wg / s).int() + 8, 0, 15)
    ref = (q - 8).to(w.dtype) * s
    return ref.reshape(k, n), q.reshape(k, n), s.reshape(k // gs, n)


class Layer(nn.Module):
    """4-bit (symmetric, grouped) linear layer without bias; interface of reference
    marlin.py:60-131."""

    def __init__(self, infeatures, outfeatures, groupsize=-1, cute_version=True):
        super().__init__()
        if groupsize not in [-1, 128]:
            raise ValueError('Only groupsize -1 and 128 are supported.')
        if infeatures % 128 != 0 or outfeatures % 256 != 0:
            raise ValueError('`infeatures` must be divisible by 128 and `outfeatures` by 256.')
        if groupsize == -1:
            groupsize = infeatures
        if infeatures % groupsize != 0:
            raise ValueError('`infeatures` must be divisible by `groupsize`.')
        self.k = infeatures
        self.n = outfeatures
        self.groupsize = groupsize
        self.cute_version = cute_version
        self.register_buffer('B', torch.empty((self.k // 16, self.n * 16 // 8), dtype=torch.int))
        self.register_buffer('s', torch.empty((self.k // groupsize, self.n), dtype=torch.half))
        # sized for the narrowest column tile (128) and the default max_par (16)
        self.register_buffer('workspace', torch.zeros(self.n // 128 * 16, dtype=torch.int),
                             persistent=False)

    def forward(self, A):
        C = torch.empty(A.shape[:-1] + (self.s.shape[1],), dtype=A.dtype, device=A.device)
        mul(A.reshape((-1, A.shape[-1])), self.B, C.view((-1, C.shape[-1])), self.s,
            self.workspace, cute_version=self.cute_version)
        return C

    def pack(self, linear, scales):
        """Fill B and s from a fake-quantised `torch.nn.Linear` (half weights) and its
        scales of shape (outfeatures, groups)."""
        if linear.weight.dtype != torch.half:
            raise ValueError('Only `torch.half` weights are supported.')
        s = scales.t()                 # (groups, n)
        w = linear.weight.data.t()     # (k, n)
        groupwise = self.groupsize != self.k
        s_full = s.repeat_interleave(self.groupsize, dim=0) if groupwise else s
        q = torch.clamp(torch.round(w / s_full).int() + 8, 0, 15)
        self.B[:, :] = pack_weights(q).to(self.B.device)
        self.s[:, :] = pack_scales(s, groupwise).to(self.s.device)


def replace_linear(module, name_filter=lambda n: True, groupsize=-1, name=''):
    """Recursively swap every `torch.nn.Linear` selected by `name_filter` for an
    empty `Layer` (reference marlin.py:134-151)."""
    if isinstance(module, Layer):
        return
    for child_name, child in list(module.named_children()):
        full = f"{name}.{child_name}" if name else child_name
        if isinstance(child, nn.Linear) and name_filter(full):
            setattr(module, child_name,
                    Layer(child.in_features, child.out_features, groupsize=groupsize))
        else:
            replace_linear(child, name_filter, groupsize=groupsize, name=full)


def check(m, n, k, groupsize=-1, thread_k=-1, thread_n=-1):
    """Return code marlin_gemm would give for these sizes (no GPU touched)."""
    return _lib.marlin_amd_check(m, n, k, groupsize, thread_k, thread_n)


def force_kernel(which):
    """0 = choose by cost, 1 = streaming kernel, 2 = prefill kernel, 3 = column-strip kernel
    (at most 1024 rows; other problems are planned as with 0), 4 = by cost without the
    column-strip kernel -- calling thread only."""
    _lib.marlin_amd_force_kernel(int(which))


def force_strips(strips):
    """16-column strips per workgroup of the column-strip kernel (1 to 4); 0 = choose by
    cost (calling thread only)."""
    _lib.marlin_amd_force_strips(int(strips))


def force_k_slices(slices):
    """Slices of the k range per prefill tile; 0 = choose by cost (calling thread only)."""
    _lib.marlin_amd_force_k_slices(int(slices))


def force_tile_rows(rows):
    """Rows of C per prefill workgroup (64 or 128); 0 = choose by cost (calling thread only)."""
    _lib.marlin_amd_force_tile_rows(int(rows))


def force_row_halves(mode):
    """Whether the streaming kernel cuts the rows into parts computed by separate workgroups
    (17..64 rows in two halves, more in parts of 32 within one launch): 0 = choose by cost,
    1 = never, 2 = wherever possible (calling thread only)."""
    _lib.marlin_amd_force_row_halves(int(mode))


def work_order(grid):
    """Work index of every workgroup of a streaming launch of `grid` workgroups."""
    out = (ctypes.c_int * grid)()
    _lib.marlin_amd_work_order(grid, out)
    return list(out)


def plan(m, n, k, groupsize=-1, thread_k=-1, thread_n=-1, sms=-1, cus=256):
    """Kernel, grid and stream-K partition marlin_gemm would use."""
    out = (ctypes.c_int * 13)()
    rc = _lib.marlin_amd_plan(m, n, k, groupsize, thread_k, thread_n, sms, cus, out)
    keys = ("kernel", "grid", "granules_per_wg", "col_tiles", "granules_per_tile", "launches",
            "k_slices", "tile_rows", "wgs_per_tile", "partial_kib", "row_parts", "part_rows", "strips")
    return rc, dict(zip(keys, out))


def plan_costs(m, n, k, groupsize=-1, cus=256):
    """The fitted costs (us) the planner compares: streaming kernel as planned, prefill kernel,
    column strips and their width (-1 where a kernel cannot run the shape)."""
    out = (ctypes.c_double * 4)()
    rc = _lib.marlin_amd_plan_costs(m, n, k, groupsize, cus, out)
    return rc, dict(zip(("stream", "prefill", "strips", "strips_per_wg"), out))


def scratch_bytes(dev=-1):
    """(bytes, buffers) of partial-sum scratch the library holds (no GPU touched)."""
    n = ctypes.c_int(0)
    return _lib.marlin_amd_scratch_bytes(dev, ctypes.byref(n)), n.value


def release(dev=-1):
    """Free the library's partial-sum scratch (waits for the device); bytes freed."""
    return _lib.marlin_amd_release(dev)


def device_info(dev=0):
    """Compute units, shader clock (kHz), memory clock (kHz), bus width (bits), L2 bytes."""
    out = (ctypes.c_int * 5)()
    if _lib.marlin_amd_device_info(dev, out) != 0:
        raise RuntimeError(_lib.marlin_amd_last_error().decode())
    return dict(zip(("compute_units", "clock_khz", "memory_clock_khz", "bus_width_bits",
                     "l2_bytes"), out))


def gemm_raw(entry, A, B, C, s, workspace, groupsize, thread_k=-1, thread_n=-1, sms=-1,
             max_par=16, stream=None):
    """One of the 15-argument C entries (`marlin_gemm`, `marlin_cute`, `marlin_official`,
    `marlin_gemm_static`) on tensors: returns the entry's integer code."""
    dev = A.get_device()
    return getattr(_lib, entry)(A.data_ptr(), B.data_ptr(), C.data_ptr(), s.data_ptr(),
                                A.size(0), C.size(1), A.size(1), workspace.data_ptr(), groupsize,
                                dev, _raw_stream(dev) if stream is None else stream,
                                thread_k, thread_n, sms, max_par)


_probe_lib = None


def _probes():
    """The probe library beside this one (libmarlin_amd_probe.so), loaded on first use."""
    global _probe_lib
    if _probe_lib is None:
        path = os.path.join(_HERE, "libmarlin_amd_probe.so")
        if not os.path.exists(path):
            raise RuntimeError(f"{path} is missing: build it (python awesome-cute_amd/build.py)")
        lib = ctypes.CDLL(path)
        lib.marlin_amd_probe.restype = _I
        lib.marlin_amd_probe.argtypes = [_I, _P, _I, _I, _I, _I, _P]
        lib.marlin_amd_probe_issue.restype = _I
        lib.marlin_amd_probe_issue.argtypes = [_I, _I, _I, _I, _I, _P]
        lib.marlin_amd_probe_pull.restype = _I
        lib.marlin_amd_probe_pull.argtypes = [_P, ctypes.c_longlong, ctypes.c_longlong, _I, _I, _P]
        lib.marlin_amd_probe_last_error.restype = ctypes.c_char_p
        _probe_lib = lib
    return _probe_lib


def _probe_check(rc, what):
    if rc != 0:
        raise RuntimeError(f"{what} failed with code {rc}: "
                           f"{_probes().marlin_amd_probe_last_error().decode()}")


def probe(kind, B, n, k, m=1):
    """Measurement probe on the current stream: kind 0 = empty launch, 1 = plain read of the
    packed weights B with the work split of the kernel planned for m rows of this shape, 2 = a
    loop of nothing but MFMAs (n*k/8192 per wave, 8 waves per compute unit) (marlin_amd_probe)."""
    dev = B.get_device()
    _probe_check(_probes().marlin_amd_probe(kind, B.data_ptr(), m, n, k, dev, _raw_stream(dev)),
                 "marlin_amd_probe")


def probe_issue(n_valu, n_lds=0, n_global=0, iters=2000, workgroups=256):
    """Shader cycles per MFMA of a lone wave per SIMD that issues, behind every MFMA, n_valu
    packed-fp16 VALU operations and, behind the first n_lds / n_global of every eight, a 16-byte
    LDS read / global load: median over the workgroups (marlin_amd_probe_issue)."""
    out = (ctypes.c_float * workgroups)()
    _probe_check(_probes().marlin_amd_probe_issue(n_valu, n_lds, n_global, iters, workgroups, out),
                 "marlin_amd_probe_issue")
    return float(np.median(np.frombuffer(out, dtype=np.float32))) / 32.0


def probe_pull(src, bytes_per_workgroup, depth, workgroups):
    """Microseconds every one of `workgroups` workgroups needs to read its own
    bytes_per_workgroup of the tensor `src` with `depth` 16-byte loads in flight per thread
    (marlin_amd_probe_pull; the kernel's own 100 MHz clock)."""
    out = (ctypes.c_float * workgroups)()
    _probe_check(_probes().marlin_amd_probe_pull(src.data_ptr(), src.numel() * src.element_size(),
                                                 bytes_per_workgroup, depth, workgroups, out),
                 "marlin_amd_probe_pull")
    return np.frombuffer(out, dtype=np.float32) / 100.0


def last_error():
    return _lib.marlin_amd_last_error().decode()
