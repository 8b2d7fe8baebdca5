"""ctypes front of oracle/liboracle.so (plain-C restatement of the reference's
CPU convolution, bias loops, naive DFT and per-frequency contraction).

TEST INFRASTRUCTURE ONLY: never imported by the product package.
"""
import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_SO = os.path.join(_HERE, "liboracle.so")
_lib = None

_f32p = ctypes.POINTER(ctypes.c_float)
_L = ctypes.c_long


def build(force=False):
    """Compile refconv.c with gcc (a few seconds)."""
    if force or not os.path.exists(_SO) or \
            os.path.getmtime(_SO) < os.path.getmtime(os.path.join(_HERE, "refconv.c")):
        subprocess.check_call(["make", "-C", _HERE, "-B", "liboracle.so"],
                              stdout=subprocess.DEVNULL)
    return _SO


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(_SO):
            build()
        _lib = ctypes.CDLL(_SO)
        _lib.orc_is_within.argtypes = [ctypes.c_float, ctypes.c_float, ctypes.c_float]
        _lib.orc_is_within.restype = ctypes.c_int
    return _lib


def set_threads(n):
    """OpenMP threads of the parallel loops from now on (n < 1: unchanged); returns the count in effect."""
    fn = lib().orc_set_threads
    fn.argtypes, fn.restype = [ctypes.c_int], ctypes.c_int
    return int(fn(int(n)))


def _p(a):
    return a.ctypes.data_as(_f32p)


def _c(a):
    a = np.ascontiguousarray(a, dtype=np.float32)
    return a


def _pad4(padding):
    if padding is None:
        return (0, 0, 0, 0)
    return tuple(int(x) for x in padding)  # (top, bottom, left, right)


def cross_correlation_valid(inp, filt, stride=(1, 1), padding=None):
    """fprop oracle.  inp (B,P,H,W), filt (F,P,kH,kW) -> (B,F,oR,oC)."""
    inp, filt = _c(inp), _c(filt)
    B, P, H, W = inp.shape
    F, P2, kH, kW = filt.shape
    if P != P2:
        raise ValueError("num planes mismatch")
    pt, pb, pl, pr = _pad4(padding)
    if stride[0] < 1 or stride[1] < 1:
        raise ValueError("filter stride should be >= 1")
    oR = (H + pt + pb - kH) // stride[0] + 1
    oC = (W + pl + pr - kW) // stride[1] + 1
    if oR < 1 or oC < 1:
        raise ValueError("filter must be <= input in size")
    out = np.empty((B, F, oR, oC), np.float32)
    rc = lib().orc_cross_correlation_valid(
        _p(inp), _L(B), _L(P), _L(H), _L(W), _p(filt), _L(F), _L(kH), _L(kW),
        _L(stride[0]), _L(stride[1]), _L(pt), _L(pb), _L(pl), _L(pr), _p(out))
    if rc != 0:
        raise ValueError("oracle rejected arguments (code %d)" % rc)
    return out


def convolution_full(gout, filt, stride=(1, 1), padding=None):
    """bprop oracle.  gout (B,F,oR,oC), filt (F,P,kH,kW) -> gradInput (B,P,H,W)."""
    gout, filt = _c(gout), _c(filt)
    B, F, oR, oC = gout.shape
    F2, P, kH, kW = filt.shape
    if F != F2:
        raise ValueError("num planes mismatch")
    pt, pb, pl, pr = _pad4(padding)
    H = (oR - 1) * stride[0] + kH - pt - pb
    W = (oC - 1) * stride[1] + kW - pl - pr
    gin = np.empty((B, P, H, W), np.float32)
    rc = lib().orc_convolution_full(
        _p(gout), _L(B), _L(F), _L(oR), _L(oC), _p(filt), _L(P), _L(kH), _L(kW),
        _L(stride[0]), _L(stride[1]), _L(pt), _L(pb), _L(pl), _L(pr), _p(gin))
    if rc != 0:
        raise ValueError("oracle rejected arguments (code %d)" % rc)
    return gin


def cross_correlation_reverse_valid(inp, gout, stride=(1, 1), scale=1.0, padding=None):
    """accGrad oracle.  inp (B,P,H,W), gout (B,F,oR,oC) -> gradWeight (F,P,kH,kW)."""
    inp, gout = _c(inp), _c(gout)
    B, P, H, W = inp.shape
    B2, F, oR, oC = gout.shape
    if B != B2:
        raise ValueError("batch size mismatch")
    pt, pb, pl, pr = _pad4(padding)
    kH = H + pt + pb - (oR - 1) * stride[0]
    kW = W + pl + pr - (oC - 1) * stride[1]
    gw = np.empty((F, P, kH, kW), np.float32)
    rc = lib().orc_cross_correlation_reverse_valid(
        _p(inp), _L(B), _L(P), _L(H), _L(W), _p(gout), _L(F), _L(oR), _L(oC),
        _L(stride[0]), _L(stride[1]), ctypes.c_float(scale),
        _L(pt), _L(pb), _L(pl), _L(pr), _p(gw))
    if rc != 0:
        raise ValueError("oracle rejected arguments (code %d)" % rc)
    return gw


def bias_update_output(out, bias):
    out = _c(out).copy()
    bias = _c(bias)
    B, F, R, C = out.shape
    lib().orc_bias_update_output(_p(out), _L(B), _L(F), _L(R), _L(C), _p(bias))
    return out


def bias_acc_grad_parameters(gout, scale=1.0):
    gout = _c(gout)
    B, F, R, C = gout.shape
    gb = np.empty((F,), np.float32)
    lib().orc_bias_acc_grad_parameters(_p(gout), _L(B), _L(F), _L(R), _L(C),
                                       ctypes.c_float(scale), _p(gb))
    return gb


def is_within(a, b, rel):
    return bool(lib().orc_is_within(float(a), float(b), float(rel)))


def dft2d_r2c(x, n_rows, n_cols, pad_u=0, pad_l=0):
    """x (planes,h,w) -> (planes, n_rows, n_cols//2+1, 2), naive DFT."""
    x = _c(x)
    planes, h, w = x.shape
    out = np.empty((planes, n_rows, n_cols // 2 + 1, 2), np.float32)
    lib().orc_dft2d_r2c(_p(x), _L(planes), _L(h), _L(w), _L(pad_u), _L(pad_l),
                        _L(n_rows), _L(n_cols), _p(out))
    return out


def idft2d_c2r(freq, h, w, n_cols, pad_u=0, pad_l=0):
    """freq (planes, n_rows, n_cols//2+1, 2) -> (planes,h,w), unnormalised, cropped."""
    freq = _c(freq)
    planes, n_rows, nch, two = freq.shape
    assert two == 2 and nch == n_cols // 2 + 1
    out = np.empty((planes, h, w), np.float32)
    lib().orc_idft2d_c2r(_p(freq), _L(planes), _L(h), _L(w), _L(pad_u), _L(pad_l),
                         _L(n_rows), _L(n_cols), _p(out))
    return out


def freq_contract(pass_, A, Bm, nB, nP, nF, alpha):
    """Plane-major spectra (d0,d1,Q,2); see refconv.c for the three passes."""
    A, Bm = _c(A), _c(Bm)
    Q = A.shape[2]
    shape = {0: (nB, nF, Q, 2), 1: (nB, nP, Q, 2), 2: (nF, nP, Q, 2)}[pass_]
    C = np.empty(shape, np.float32)
    lib().orc_freq_contract(ctypes.c_int(pass_), _p(A), _p(Bm), _p(C),
                            _L(nB), _L(nP), _L(nF), _L(Q), ctypes.c_float(alpha))
    return C
