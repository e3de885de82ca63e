"""The binding module the reference's Python imports as `marlin_lib`
(gemm/marlin_gemm/marlin.py:5-8), over the C ABI of libmarlin_amd.so.

`mul` has the signature and defaults of the pybind function
(marlin_gemm.cpp:19-22, 58-60): positional tensors, then thread_k, thread_n,
sms, max_par = 8 and cute_version.  It raises RuntimeError with the binding's
messages (marlin_gemm.cpp:27-31, 48-55).
"""
from marlin import mul as _mul


def mul(A, B, C, s, workspace, thread_k=-1, thread_n=-1, sms=-1, max_par=8, cute_version=True):
    """Marlin FP16xINT4 multiply; C = A @ dequant(B) on the current stream of A's device."""
    _mul(A, B, C, s, workspace, thread_k, thread_n, sms, max_par, cute_version)
