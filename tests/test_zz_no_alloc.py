"""The entry point that allocates nothing (fbfc_acc_grad_parameters_bias_noalloc) against the entry
point it is a variant of (fbfc_acc_grad_parameters_bias), called through the C ABI: bit-equal
results on two calls in a row, the second on a smaller input, plus the CPU oracle and the size
limit.  Bit equality is the bar: both run the same two kernels in the same order."""
import ctypes

import numpy as np
import pytest
import torch

from fbcunn_amd import _lib, synth
from gpu_util import dev, host

pytestmark = pytest.mark.gpu


def _both(g, scale):
    lib = _lib.lib()
    B, F, h, w = g.shape
    gd = dev(g)
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    want = torch.full((F,), float("nan"), device="cuda")
    nbytes = lib.fbfc_bias_grad_scratch_bytes(B, F)
    work = torch.empty((nbytes + 3) // 4, device="cuda")
    _lib.check(lib.fbfc_acc_grad_parameters_bias(gd.data_ptr(), want.data_ptr(), ctypes.c_float(scale), B, F, h, w,
                                                 work.data_ptr(), stream))
    got = torch.full((F,), float("nan"), device="cuda")
    _lib.check(lib.fbfc_acc_grad_parameters_bias_noalloc(gd.data_ptr(), got.data_ptr(), ctypes.c_float(scale),
                                                         B, F, h, w, stream))
    torch.cuda.synchronize()
    return host(got), host(want)


def test_no_alloc_bias_gradient_twice_in_a_row(oracle):
    # first a large call (all 16 batch slices, many planes), then a smaller one that must not see
    # what the first left in the shared array
    for seed, shape, scale in ((91, (32, 300, 13, 13), 0.5), (92, (3, 7, 5, 9), 1.25), (93, (128, 128, 13, 13), 1.0)):
        g = synth.uniform(seed, shape)
        got, want = _both(g, scale)
        assert np.isfinite(got).all()
        assert np.array_equal(got, want), np.abs(got - want).max()
        np.testing.assert_allclose(got, oracle.bias_acc_grad_parameters(g, scale), rtol=5e-4, atol=1e-5)


def test_no_alloc_rejects_sizes_beyond_its_array():
    lib = _lib.lib()
    x = torch.zeros(8, device="cuda")
    rc = lib.fbfc_acc_grad_parameters_bias_noalloc(x.data_ptr(), x.data_ptr(), ctypes.c_float(1.0), 1, 4097, 1, 1,
                                                   ctypes.c_void_p(0))
    assert rc == _lib.ERR_UNSUPPORTED_SIZE
    assert b"4096" in lib.fbfc_last_error()


def test_no_alloc_bias_gradient_replays_from_a_graph():
    """After one eager call on the device (which looks the fixed array up) the entry point can be captured
    into a graph; every replay, with eager work and a synchronisation in between, gives the eager bits."""
    lib = _lib.lib()
    g = dev(synth.uniform(94, (16, 40, 7, 9)))
    B, F, h, w = g.shape
    out = torch.full((F,), float("nan"), device="cuda")

    def call():
        _lib.check(lib.fbfc_acc_grad_parameters_bias_noalloc(g.data_ptr(), out.data_ptr(), ctypes.c_float(0.75), B, F, h, w,
                                                             ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)))
    call()
    torch.cuda.synchronize()
    want = host(out).copy()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        call()
    torch.cuda.current_stream().wait_stream(side)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        call()
    for rep in range(3):
        out.fill_(float("nan"))
        (g * 2).sum().item()
        graph.replay()
        torch.cuda.synchronize()
        assert np.array_equal(host(out), want), "replay %d differs from the eager result" % rep
