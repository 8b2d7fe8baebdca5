"""Two host threads, each with its own layers and its own stream, call the library at the same time.  The
library keeps its state per plan (buffers, reuse flags) and per thread (last error), and prepares its kernels
once per device under a mutex, so what each thread computes must equal, bit for bit, what the same calls gave
before on one thread.  The reference runs one Lua thread (fbcunn/SpatialConvolutionFFT.lua has no locking);
a C-ABI library has no such guarantee from its callers."""
import threading

import pytest
import torch

pytestmark = pytest.mark.gpu

# B, P, F, k, H, pad, tile, reuse: untiled at three FFT sizes and one tiled layer
LAYERS = [
    (16, 32, 48, 3, 13, 1, None, None),
    (8, 16, 24, 5, 27, 2, None, "all"),
    (4, 8, 16, 7, 50, 3, None, "weight"),
    (4, 16, 16, 3, 40, 1, 16, None),
]


def _make(spec, seed):
    from fbcunn_amd import nn
    B, P, F, k, H, pad, tile, reuse = spec
    kw = {} if reuse is None else {"memoryReusePolicy": reuse}
    if tile is None:
        net = nn.SpatialConvolutionFBFFT(P, F, k, k, 1, 1, pad, pad, **kw)
    else:
        net = nn.SpatialConvolutionFFTTiled(P, F, k, k, 1, 1, pad, pad, tile, tile, **kw)
    gen = torch.Generator(device="cuda").manual_seed(seed)
    net.weight.copy_(torch.randn(F, P, k, k, device="cuda", generator=gen) * 0.05)
    net.bias.copy_(torch.rand(F, device="cuda", generator=gen) - 0.5)
    o = H + 2 * pad - k + 1
    x = torch.rand(B, P, H, H, device="cuda", generator=gen) * 2 - 1
    g = torch.rand(B, F, o, o, device="cuda", generator=gen) * 2 - 1
    return net, x, g


def _step(net, x, g):
    out = net.updateOutput(x).clone()
    gi = net.backward(x, g, 0.25).clone()
    return out, gi, net.gradWeight.clone(), net.gradBias.clone()


def test_two_host_threads_with_their_own_plans_and_streams():
    from fbcunn_amd import _lib
    jobs = [[_make(spec, 100 * t + i) for i, spec in enumerate(LAYERS)] for t in range(2)]
    want = [[_step(*job) for job in jobs[t]] for t in range(2)]
    torch.cuda.synchronize()
    errors = []
    start = threading.Barrier(2)

    def work(t):
        try:
            stream = torch.cuda.Stream()
            start.wait()
            with torch.cuda.stream(stream):
                for rep in range(25):
                    for i, job in enumerate(jobs[t]):
                        got = _step(*job)
                        for name, a, b in zip(("output", "gradInput", "gradWeight", "gradBias"), got, want[t][i]):
                            if not torch.equal(a, b):
                                errors.append("thread %d layer %d rep %d: %s differs" % (t, i, rep, name))
                                start.abort()
                                return
                # a failing call leaves its message with the thread that made it: both threads fail in
                # different ways, meet, and only then read what the library kept for them
                buf = torch.zeros(64, device="cuda")
                if t == 0:
                    bad = _lib.lib().fbfc_fft2d(None, 1, 4, 4, 0, 0, 8, None, None)
                    expect = "null argument"
                else:
                    bad = _lib.lib().fbfc_fft2d(buf.data_ptr(), 1, 4, 4, 0, 0, 12, buf.data_ptr(), None)
                    expect = "unsupported size"
                start.wait(timeout=120)
                msg = _lib.lib().fbfc_last_error().decode()
                if bad == 0 or expect not in msg:
                    errors.append("thread %d: last error %r after code %d" % (t, msg, bad))
            stream.synchronize()
        except Exception as e:  # noqa: BLE001 - reported through the list, the thread must not die silently
            errors.append("thread %d: %r" % (t, e))
            start.abort()

    threads = [threading.Thread(target=work, args=(t,)) for t in range(2)]
    for th in threads:
        th.start()
    for th in threads:
        th.join()
    torch.cuda.synchronize()
    assert not errors, errors
