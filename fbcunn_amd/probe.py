"""ctypes binding of libfbfftconv_probe.so, the measurement library (include/fbfftconv_probe.h).

It holds an instrumented copy of the contraction's tile kernel and is loaded by bench.py and one
test only; nothing in the product path imports this module, and the shipped library does not
contain its symbol.
"""
import ctypes
import os

import torch

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libfbfftconv_probe.so")
_lib = None


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise ImportError("%s is missing: build it with `python -m fbcunn_amd.build`" % LIB_PATH)
        handle = ctypes.CDLL(LIB_PATH)
        fn = handle.fbfc_probe_contraction_clock
        fn.restype = ctypes.c_int
        fn.argtypes = [ctypes.c_int] + [ctypes.c_void_p] * 3 + [ctypes.c_int] * 5 + \
                      [ctypes.c_void_p, ctypes.POINTER(ctypes.c_float), ctypes.c_void_p]
        _lib = handle
    return _lib


def contractionClock(mode, A, B, C, launches=20):
    """Shader clock (MHz) the 64x64 tile contraction kernel runs at over `launches` back-to-back launches
    of C = op(A, B) (mode 0: A conj(B)^T, 1: A B, 2: conj(A)^T B; operands (Q, rows, cols, 2) float32 on
    the GPU); C receives the unscaled product.  The MFMA peak is quoted at the chip's peak clock,
    sustained fp32 MFMA work runs below it."""
    for t in (A, B, C):
        if not (isinstance(t, torch.Tensor) and t.is_cuda and t.dtype == torch.float32 and t.dim() == 4
                and t.is_contiguous()):
            raise TypeError("operands must be contiguous 4-D float32 GPU tensors")
    Q, m, n = C.size(0), C.size(1), C.size(2)
    k = A.size(1) if mode == 2 else A.size(2)
    exp_a = (Q, k, m, 2) if mode == 2 else (Q, m, k, 2)
    exp_b = (Q, n, k, 2) if mode == 0 else (Q, k, n, 2)
    if mode not in (0, 1, 2) or tuple(A.shape) != exp_a or tuple(B.shape) != exp_b:
        raise ValueError("operand shapes do not match: A %s B %s C %s" % (tuple(A.shape), tuple(B.shape), tuple(C.shape)))
    ticks = torch.zeros(4, dtype=torch.int64, device=C.device)
    mhz = ctypes.c_float(0.0)
    rc = lib().fbfc_probe_contraction_clock(mode, A.data_ptr(), B.data_ptr(), C.data_ptr(), Q, m, n, k, int(launches),
                                            ticks.data_ptr(), ctypes.byref(mhz),
                                            torch.cuda.current_stream().cuda_stream)
    if rc == 1:
        raise ValueError("the clock probe takes m, n multiples of 64, k of 16 and 16-byte aligned operands")
    if rc != 0:
        raise RuntimeError("contraction clock probe failed (HIP error)")
    return float(mhz.value)
