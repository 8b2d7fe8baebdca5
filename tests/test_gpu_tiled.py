"""GPU parity of the tiled FFT convolution (nn.SpatialConvolutionFFTTiled and its
Sync / Async / Iterated instantiations) against the CPU oracle: a tiled module
must give the results of the plain convolution (the reference checks it against
cuDNN with the same procedure, test/test_FFT.lua:160-256, tiled VGG shapes
:463-505).  Bars as for the untiled modules.
"""
import numpy as np
import pytest
import torch

from fbcunn_amd import synth
from gpu_util import dev, host, max_rel, rel_l2

pytestmark = pytest.mark.gpu
MAX_REL, REL_L2 = 1e-3, 1e-4


@pytest.fixture(scope="module")
def nn():
    from fbcunn_amd import nn as mod
    return mod


def _close(got, want, what):
    assert np.isfinite(got).all(), what
    mr, l2 = max_rel(got, want), rel_l2(got, want)
    assert mr <= MAX_REL and l2 <= REL_L2, "%s: max_rel %.3g rel_l2 %.3g" % (what, mr, l2)


def _tensors(B, P, F, kH, kW, iH, iW, padH, padW, seed):
    x = synth.uniform(seed, (B, P, iH, iW), stream=0)
    w = synth.normal(seed, (F, P, kH, kW), 0.0, 0.05, stream=1)
    bias = synth.uniform(seed, (F,), -0.1, 0.1, stream=2)
    oH, oW = iH + 2 * padH - kH + 1, iW + 2 * padW - kW + 1
    g = synth.uniform(seed, (B, F, oH, oW), stream=3)
    return x, w, bias, g


def _three_passes(net, x, w, bias, g, scale):
    net.weight.copy_(dev(w))
    net.bias.copy_(dev(bias))
    net.gradWeight.fill_(float("nan"))
    net.gradBias.fill_(float("nan"))
    xd, gd = dev(x), dev(g)
    out = host(net.updateOutput(xd))
    gin = host(net.updateGradInput(xd, gd))
    net.accGradParameters(xd, gd, scale)
    res = out, gin, host(net.gradWeight), host(net.gradBias)
    net.cleanupBuffers()
    return res


# batch, inputPlanes, outputPlanes, kH, kW, iH, iW, padH, padW, tileH, tileW
TILED = [
    (2, 3, 4, 3, 3, 20, 20, 1, 1, 8, 8),        # whole tiles and a ragged last tile
    (2, 3, 4, 3, 3, 24, 24, 0, 0, 8, 8),
    (1, 4, 3, 3, 3, 40, 37, 1, 1, 16, 16),      # rectangular image
    (2, 2, 5, 5, 5, 50, 50, 2, 2, 16, 16),
    (1, 3, 2, 3, 3, 70, 66, 1, 1, 32, 32),
    (1, 2, 3, 7, 7, 64, 64, 3, 3, 32, 32),
    (2, 3, 2, 3, 5, 30, 41, 2, 0, 16, 16),      # rectangular kernel: steps differ per axis
    (1, 2, 2, 5, 5, 33, 33, 4, 4, 16, 16),      # pad = k - 1
    (1, 2, 2, 3, 3, 45, 45, 1, 1, 12, 12),      # tile below its FFT size
    (1, 2, 2, 3, 3, 45, 52, 1, 1, 10, 14),      # rectangular tile
    (3, 20, 18, 3, 3, 19, 19, 1, 1, 16, 16),    # more planes than a workgroup's share
]


@pytest.mark.parametrize("problem", TILED)
def test_tiled_three_passes_vs_oracle(nn, oracle, problem):
    B, P, F, kH, kW, iH, iW, padH, padW, tH, tW = problem
    seed = 900 + sum(problem)
    x, w, bias, g = _tensors(B, P, F, kH, kW, iH, iW, padH, padW, seed)
    net = nn.SpatialConvolutionFFTTiled(P, F, kW, kH, 1, 1, padW, padH, tW, tH)
    out, gin, gw, gb = _three_passes(net, x, w, bias, g, 0.41)
    pad = (padH, padH, padW, padW)
    _close(out, oracle.bias_update_output(oracle.cross_correlation_valid(x, w, (1, 1), pad), bias), "output")
    _close(gin, oracle.convolution_full(g, w, (1, 1), pad), "gradInput")
    _close(gw, oracle.cross_correlation_reverse_valid(x, g, (1, 1), 0.41, pad), "gradWeight")
    _close(gb, oracle.bias_acc_grad_parameters(g, 0.41), "gradBias")


@pytest.mark.parametrize("cls", ["SpatialConvolutionFFTTiledSync", "SpatialConvolutionFFTTiledAsync",
                                 "SpatialConvolutionFFTTiledIterated"])
def test_tiled_variants_share_results(nn, oracle, cls):
    B, P, F, k, H, pad = 2, 3, 4, 3, 26, 1
    x, w, bias, g = _tensors(B, P, F, k, k, H, H, pad, pad, 77)
    net = getattr(nn, cls)(P, F, k, k, 1, 1, pad, pad)          # default tile 16
    assert (net.tileSizeH, net.tileSizeW) == (16, 16)
    out, gin, gw, gb = _three_passes(net, x, w, bias, g, 1.0)
    p4 = (pad,) * 4
    _close(out, oracle.bias_update_output(oracle.cross_correlation_valid(x, w, (1, 1), p4), bias), "output")
    _close(gin, oracle.convolution_full(g, w, (1, 1), p4), "gradInput")
    _close(gw, oracle.cross_correlation_reverse_valid(x, g, (1, 1), 1.0, p4), "gradWeight")


@pytest.mark.parametrize("reuse", [None, "all", ["input", "weight"], "output"])
def test_tiled_reuse_policies(nn, oracle, reuse):
    B, P, F, k, H, pad = 2, 4, 3, 3, 30, 1
    x, w, bias, g = _tensors(B, P, F, k, k, H, H, pad, pad, 78)
    net = nn.SpatialConvolutionFFTTiled(P, F, k, k, 1, 1, pad, pad, 16, 16, reuse)
    p4 = (pad,) * 4
    want = (oracle.bias_update_output(oracle.cross_correlation_valid(x, w, (1, 1), p4), bias),
            oracle.convolution_full(g, w, (1, 1), p4),
            oracle.cross_correlation_reverse_valid(x, g, (1, 1), 0.5, p4))
    net.weight.copy_(dev(w))
    net.bias.copy_(dev(bias))
    xd, gd = dev(x), dev(g)
    for _ in range(2):   # the second round starts from the spectra the first one left behind
        _close(host(net.updateOutput(xd)), want[0], "output")
        _close(host(net.updateGradInput(xd, gd)), want[1], "gradInput")
        net.accGradParameters(xd, gd, 0.5)
        _close(host(net.gradWeight), want[2], "gradWeight")
        _close(host(net.gradBias), oracle.bias_acc_grad_parameters(g, 0.5), "gradBias")
    net.cleanupBuffers()


def test_tiled_equals_untiled_on_vgg_like_shape(nn):
    """112 x 112, 3 x 3, pad 1 (test/test_FFT.lua:466-467 at a reduced plane count): too large for
    the oracle in a test, so the tiled result is held against the untiled FFT-128 path, which the
    oracle tests cover, and against the adjoint identity <fprop(x), g> = <x, bprop(g)>."""
    B, P, F, k, H, pad = 4, 16, 32, 3, 112, 1
    x, w, bias, g = _tensors(B, P, F, k, k, H, H, pad, pad, 79)
    tiled = nn.SpatialConvolutionFFTTiled(P, F, k, k, 1, 1, pad, pad, 32, 32)
    plain = nn.SpatialConvolutionFBFFT(P, F, k, k, 1, 1, pad, pad)
    a = _three_passes(tiled, x, w, bias, g, 0.25)
    b = _three_passes(plain, x, w, bias, g, 0.25)
    for got, want, what in zip(a, b, ("output", "gradInput", "gradWeight", "gradBias")):
        _close(got, want, what)
    out_nobias = a[0].astype(np.float64) - bias.reshape(1, -1, 1, 1)
    lhs = float((out_nobias * g).sum())
    rhs = float((x.astype(np.float64) * a[1]).sum())
    assert abs(lhs - rhs) <= 1e-4 * max(abs(lhs), abs(rhs), 1.0)


def test_tiled_errors(nn):
    from fbcunn_amd._lib import FbfcError, ERR_INVALID_ARGUMENT, ERR_UNSUPPORTED_SIZE
    x = torch.zeros(1, 2, 20, 20, device="cuda")
    with pytest.raises(FbfcError) as e:      # SpatialConvolutionFFTTiled.lua:757-760
        nn.SpatialConvolutionFFTTiled(2, 2, 5, 5, 1, 1, 0, 0, 4, 4).updateOutput(x)
    assert e.value.code == ERR_INVALID_ARGUMENT and "smaller than kernel" in e.value.message
    with pytest.raises(FbfcError) as e:      # :508-512
        nn.SpatialConvolutionFFTTiled(2, 2, 3, 3, 1, 1, 0, 0, 32, 32).updateOutput(x)
    assert e.value.code == ERR_INVALID_ARGUMENT and "Tile size too large" in e.value.message
    big = torch.zeros(1, 1, 100, 100, device="cuda")
    with pytest.raises(FbfcError) as e:
        nn.SpatialConvolutionFFTTiled(1, 1, 3, 3, 1, 1, 0, 0, 64, 64).updateOutput(big)
    assert e.value.code == ERR_UNSUPPORTED_SIZE


# ---- nn.SpatialConvolutionFFTTiledIterated: the fused kernels ------------------------------------------
# batch, inputPlanes, outputPlanes, kH, kW, iH, iW, padH, padW, tileH, tileW
ITERATED = TILED + [
    (2, 3, 64, 3, 3, 28, 28, 1, 1, 16, 16),     # first-layer shape: weights in registers, two blocks of output planes
    (2, 64, 3, 3, 3, 28, 28, 1, 1, 16, 16),     # last-layer shape: the contracted side in chunks
    (1, 40, 70, 3, 3, 20, 20, 1, 1, 16, 16),    # both sides beyond one batch of planes, ragged last block
    (2, 1, 5, 5, 5, 40, 40, 2, 2, 32, 32),      # one input plane
    (2, 3, 70, 3, 3, 18, 18, 1, 1, 8, 8),       # tiles of 8
    (1, 7, 33, 3, 3, 12, 12, 1, 1, 8, 8),
]


@pytest.mark.parametrize("problem", ITERATED)
def test_iterated_three_passes_vs_oracle(nn, oracle, problem):
    """Every pass as one fused kernel (plus the transform of the weights): same bars as the other modules."""
    B, P, F, kH, kW, iH, iW, padH, padW, tH, tW = problem
    seed = 1900 + sum(problem)
    x, w, bias, g = _tensors(B, P, F, kH, kW, iH, iW, padH, padW, seed)
    net = nn.SpatialConvolutionFFTTiledIterated(P, F, kW, kH, 1, 1, padW, padH, tW, tH)
    assert net.memoryReusePolicy == ["none"]
    net.weight.copy_(dev(w))
    net.bias.copy_(dev(bias))
    net.gradWeight.fill_(float("nan"))
    net.gradBias.fill_(float("nan"))
    xd, gd = dev(x), dev(g)
    out = host(net.updateOutput(xd))
    kernels = net.stageKernels(xd)
    assert "fused_conv_kernel" in kernels["mm"] and "ifft" not in kernels, kernels
    gin = host(net.updateGradInput(xd, gd))
    assert "fused_conv_kernel" in net.stageKernels(xd)["mm"]
    net.accGradParameters(xd, gd, 0.41)
    assert "fused_accgrad_kernel" in net.stageKernels(xd)["mm"]
    gw, gb = host(net.gradWeight), host(net.gradBias)
    net.cleanupBuffers()
    pad = (padH, padH, padW, padW)
    _close(out, oracle.bias_update_output(oracle.cross_correlation_valid(x, w, (1, 1), pad), bias), "output")
    _close(gin, oracle.convolution_full(g, w, (1, 1), pad), "gradInput")
    _close(gw, oracle.cross_correlation_reverse_valid(x, g, (1, 1), 0.41, pad), "gradWeight")
    _close(gb, oracle.bias_acc_grad_parameters(g, 0.41), "gradBias")


def test_iterated_first_layer_112(nn, oracle):
    """3 -> 64 planes, 112 x 112, 3 x 3, pad 1, tiles of 16 (the shape the fused kernels are for): output and
    gradWeight against the oracle on a slice of the planes, everything against the three-kernel tiled module,
    and twice in a row (the second call finds the plan's buffers as the first left them)."""
    B, P, F, k, H, pad = 4, 3, 64, 3, 112, 1
    x, w, bias, g = _tensors(B, P, F, k, k, H, H, pad, pad, 1979)
    fused = nn.SpatialConvolutionFFTTiledIterated(P, F, k, k, 1, 1, pad, pad, 16, 16)
    plain = nn.SpatialConvolutionFFTTiled(P, F, k, k, 1, 1, pad, pad, 16, 16)
    b = _three_passes(plain, x, w, bias, g, 0.25)
    fused.weight.copy_(dev(w))
    fused.bias.copy_(dev(bias))
    xd, gd = dev(x), dev(g)
    for _ in range(2):
        fused.gradWeight.fill_(float("nan"))
        out = host(fused.updateOutput(xd))
        gin = host(fused.updateGradInput(xd, gd))
        fused.accGradParameters(xd, gd, 0.25)
        a = (out, gin, host(fused.gradWeight), host(fused.gradBias))
        for got, want, what in zip(a, b, ("output", "gradInput", "gradWeight", "gradBias")):
            _close(got, want, what)
    fused.cleanupBuffers()
    p4 = (pad,) * 4
    fs = [0, 31, 32, 63]
    _close(a[0][:, fs], oracle.bias_update_output(oracle.cross_correlation_valid(x, w[fs], (1, 1), p4), bias[fs]), "output")
    _close(a[2][fs], oracle.cross_correlation_reverse_valid(x, g[:, fs], (1, 1), 0.25, p4), "gradWeight")
    _close(a[1], oracle.convolution_full(g, w, (1, 1), p4), "gradInput")


def test_iterated_backward_and_graph_replay(nn):
    """backward() on the fused module runs its two passes one after the other (same bits as the separate calls),
    and the three fused passes can be captured into a graph: they allocate nothing and use no memset."""
    B, P, F, k, H, pad = 3, 3, 40, 3, 30, 1
    x, w, bias, g = _tensors(B, P, F, k, k, H, H, pad, pad, 2024)
    net = nn.SpatialConvolutionFFTTiledIterated(P, F, k, k, 1, 1, pad, pad, 16, 16)
    net.weight.copy_(dev(w))
    net.bias.copy_(dev(bias))
    xd, gd = dev(x), dev(g)

    def step():
        net.updateOutput(xd)
        net.updateGradInput(xd, gd)
        net.accGradParameters(xd, gd, 0.5)

    results = lambda: [net.output, net.gradInput, net.gradWeight, net.gradBias]
    step()
    torch.cuda.synchronize()
    want = [host(t).copy() for t in results()]
    for t in results()[1:]:
        t.fill_(float("nan"))
    net.backward(xd, gd, 0.5)
    for got, ref, name in zip(results()[1:], want[1:], ("gradInput", "gradWeight", "gradBias")):
        assert np.array_equal(host(got), ref), name
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        step()
    torch.cuda.current_stream().wait_stream(side)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        step()
    for rep in range(3):
        for t in results():
            t.fill_(float("nan"))
        (xd * 2).sum().item()
        graph.replay()
        torch.cuda.synchronize()
        for got, ref, name in zip(results(), want, ("output", "gradInput", "gradWeight", "gradBias")):
            assert np.array_equal(host(got), ref), "replay %d: %s differs from the eager result" % (rep, name)
    net.cleanupBuffers()
