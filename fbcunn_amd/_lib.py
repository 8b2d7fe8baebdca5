"""ctypes binding of libfbfftconv.so (the C ABI declared in include/fbfftconv.h).

There is no fallback: if the library is missing or a call fails, an exception
is raised.  torch is imported first so that the library binds to the HIP runtime
already loaded in the process (device pointers and streams must belong to one
runtime).
"""
import ctypes
import os

import torch  # noqa: F401  (loads the HIP runtime this library must share)

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libfbfftconv.so")

OK, ERR_INVALID_ARGUMENT, ERR_UNSUPPORTED_SIZE, ERR_UNSUPPORTED_DIMENSION, ERR_OUT_OF_MEMORY, ERR_HIP = range(6)
REUSE_NONE, REUSE_INPUT, REUSE_OUTPUT, REUSE_WEIGHT, REUSE_ALL = 0, 1, 2, 4, 7
STAGE_NAMES = ("fft_a", "fft_b", "mm", "ifft", "bias_grad")


class FbfcError(RuntimeError):
    def __init__(self, code, message):
        super().__init__("fbfftconv error %d: %s" % (code, message))
        self.code = code
        self.message = message


class ConvDesc(ctypes.Structure):
    _fields_ = [(n, ctypes.c_int) for n in
                ("batch", "in_planes", "out_planes", "in_h", "in_w", "k_h", "k_w",
                 "stride_h", "stride_w", "pad_h", "pad_w")]


class PlanInfo(ctypes.Structure):
    _fields_ = [("fft_size", ctypes.c_int), ("n_freq", ctypes.c_int),
                ("out_h", ctypes.c_int), ("out_w", ctypes.c_int),
                ("input_freq_bytes", ctypes.c_size_t), ("weight_freq_bytes", ctypes.c_size_t),
                ("output_freq_bytes", ctypes.c_size_t), ("scratch_bytes", ctypes.c_size_t),
                ("tiles_h", ctypes.c_int), ("tiles_w", ctypes.c_int),
                ("backward_freq_bytes", ctypes.c_size_t)]


_vp, _i, _f, _l = ctypes.c_void_p, ctypes.c_int, ctypes.c_float, ctypes.c_long

# name -> (restype, argtypes); must list every symbol include/fbfftconv.h declares
SIGNATURES = {
    "fbfc_version": (ctypes.c_char_p, []),
    "fbfc_last_error": (ctypes.c_char_p, []),
    "fbfc_last_launch": (ctypes.c_char_p, []),
    "fbfc_plan_query": (_i, [ctypes.POINTER(ConvDesc), ctypes.POINTER(PlanInfo)]),
    "fbfc_plan_create": (_i, [ctypes.POINTER(ConvDesc), ctypes.POINTER(_vp)]),
    "fbfc_plan_query_tiled": (_i, [ctypes.POINTER(ConvDesc), _i, _i, ctypes.POINTER(PlanInfo)]),
    "fbfc_plan_create_tiled": (_i, [ctypes.POINTER(ConvDesc), _i, _i, ctypes.POINTER(_vp)]),
    "fbfc_plan_create_tiled_iterated": (_i, [ctypes.POINTER(ConvDesc), _i, _i, ctypes.POINTER(_vp)]),
    "fbfc_plan_destroy": (_i, [_vp]),
    "fbfc_plan_get_info": (_i, [_vp, ctypes.POINTER(PlanInfo)]),
    "fbfc_update_output": (_i, [_vp, _vp, _vp, _vp, _vp, _vp]),
    "fbfc_update_grad_input": (_i, [_vp, _vp, _vp, _vp, _vp]),
    "fbfc_acc_grad_parameters": (_i, [_vp, _vp, _vp, _vp, _vp, _f, _vp]),
    "fbfc_backward": (_i, [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _f, _vp]),
    "fbfc_plan_prepare_backward": (_i, [_vp]),
    "fbfc_plan_set_reuse": (_i, [_vp, ctypes.c_uint]),
    "fbfc_plan_set_timed": (_i, [_vp, _i]),
    "fbfc_plan_stage_ms": (_i, [_vp, ctypes.POINTER(_f), _i]),
    "fbfc_plan_stage_kernel": (_i, [_vp, _i, ctypes.c_char_p, ctypes.c_size_t]),
    "fbfc_debug_force_contraction_kernel": (_i, [_i]),
    "fbfc_debug_force_spectrum_streaming": (_i, [_i]),
    "fbfc_fft2d": (_i, [_vp, _l, _i, _i, _i, _i, _i, _vp, _vp]),
    "fbfc_ifft2d": (_i, [_vp, _l, _i, _i, _i, _i, _i, _vp, _vp, _i, _vp]),
    "fbfc_planes_layout_workspace_bytes": (ctypes.c_size_t, [_l, _i]),
    "fbfc_fft2d_planes": (_i, [_vp, _l, _i, _i, _i, _i, _i, _vp, _vp, _vp]),
    "fbfc_ifft2d_planes": (_i, [_vp, _l, _i, _i, _i, _i, _i, _vp, _vp, _vp]),
    "fbfc_transpose_mm_planes_workspace_bytes": (ctypes.c_size_t, [_i, _i, _i, _i]),
    "fbfc_transpose_mm_planes": (_i, [_vp, _vp, _vp, _i, _i, _i, _i, _f, _i, _i, _i, _vp, _vp]),
    "fbfc_fft1d": (_i, [_vp, _l, _i, _i, _i, _vp, _vp]),
    "fbfc_ifft1d": (_i, [_vp, _l, _i, _i, _i, _vp, _vp]),
    "fbfc_transpose_mm": (_i, [_vp, _vp, _vp, _i, _i, _i, _i, _f, _i, _i, _i, _vp]),
    "fbfc_direct_update_output": (_i, [ctypes.POINTER(ConvDesc), _vp, _vp, _vp, _vp, _vp]),
    "fbfc_direct_update_grad_input": (_i, [ctypes.POINTER(ConvDesc), _vp, _vp, _vp, _vp]),
    "fbfc_direct_acc_grad_parameters": (_i, [ctypes.POINTER(ConvDesc), _vp, _vp, _vp, _vp, _f, _vp, _vp]),
    "fbfc_update_output_bias": (_i, [_vp, _vp, _i, _i, _i, _i, _vp]),
    "fbfc_update_output_bias_strided": (_i, [_vp, _vp, _i, _i, _i, _i, _l, _l, _l, _l, _l, _vp]),
    "fbfc_acc_grad_parameters_bias_strided": (_i, [_vp, _vp, _f, _i, _i, _i, _i, _l, _l, _l, _l, _l, _vp, _vp]),
    "fbfc_bias_grad_scratch_bytes": (ctypes.c_size_t, [_i, _i]),
    "fbfc_acc_grad_parameters_bias": (_i, [_vp, _vp, _f, _i, _i, _i, _i, _vp, _vp]),
    "fbfc_acc_grad_parameters_bias_noalloc": (_i, [_vp, _vp, _f, _i, _i, _i, _i, _vp]),
}

_lib = None


def lib():
    """The loaded library; raises if it has not been built (python -m fbcunn_amd.build)."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise ImportError(
                "%s is missing: build it with `python -m fbcunn_amd.build` "
                "(there is no CPU or PyTorch fallback for this path)" % LIB_PATH)
        handle = ctypes.CDLL(LIB_PATH)
        for name, (res, args) in SIGNATURES.items():
            fn = getattr(handle, name)  # AttributeError if a declared symbol is not exported
            fn.restype = res
            fn.argtypes = args
        _lib = handle
    return _lib


def check(rc):
    if rc != OK:
        raise FbfcError(rc, lib().fbfc_last_error().decode())
    return rc


def plan_query(tile_h=0, tile_w=0, **kw):
    """Host-only planning: returns a PlanInfo or raises FbfcError (no GPU needed).
    With tile sizes given, plans the tiled variant."""
    d = ConvDesc(**kw)
    info = PlanInfo()
    if tile_h or tile_w:
        check(lib().fbfc_plan_query_tiled(ctypes.byref(d), tile_h, tile_w, ctypes.byref(info)))
    else:
        check(lib().fbfc_plan_query(ctypes.byref(d), ctypes.byref(info)))
    return info
