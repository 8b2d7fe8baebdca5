"""GPU checks of the tuning front fbnn.SpatialConvolution (fbcunn/SpatialConvolution.lua):
whatever strategy wins, the three passes must match the CPU oracle; strategies that cannot
run the layer or exceed the memory limit are left out."""
import numpy as np
import pytest
import torch

from fbcunn_amd import synth
from gpu_util import dev, host, max_rel, rel_l2

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def fbnn():
    from fbcunn_amd import fbnn as mod
    return mod


def _close(got, want, what):
    mr, l2 = max_rel(got, want), rel_l2(got, want)
    assert mr <= 1e-3 and l2 <= 1e-4, "%s: max_rel %.3g rel_l2 %.3g" % (what, mr, l2)


@pytest.mark.parametrize("shape", [(2, 3, 4, 3, 13, 1), (2, 4, 3, 3, 40, 1), (1, 2, 3, 5, 70, 2)])
def test_tuned_module_matches_oracle(fbnn, oracle, shape):
    B, P, F, k, H, pad = shape
    x = synth.uniform(31, (B, P, H, H), stream=0)
    w = synth.normal(31, (F, P, k, k), 0.0, 0.05, stream=1)
    bias = synth.uniform(31, (F,), -0.1, 0.1, stream=2)
    o = H + 2 * pad - k + 1
    g = synth.uniform(31, (B, F, o, o), stream=3)
    net = fbnn.SpatialConvolution(P, F, k, k, 1, 1, pad, pad)
    net.weight.copy_(dev(w))
    net.bias.copy_(dev(bias))
    net.gradWeight.fill_(7.0)
    xd, gd = dev(x), dev(g)
    out = host(net.updateOutput(xd))
    assert net.bestModuleInst is not None and net.bestKey in net.timings
    assert float(net.gradWeight.min()) == 7.0            # tuning leaves the caller's gradients alone
    gin = host(net.updateGradInput(xd, gd))
    net.accGradParameters(xd, gd, 0.3)
    p4 = (pad,) * 4
    _close(out, oracle.bias_update_output(oracle.cross_correlation_valid(x, w, (1, 1), p4), bias), "output")
    _close(gin, oracle.convolution_full(g, w, (1, 1), p4), "gradInput")
    _close(host(net.gradWeight), oracle.cross_correlation_reverse_valid(x, g, (1, 1), 0.3, p4), "gradWeight")
    _close(host(net.gradBias), oracle.bias_acc_grad_parameters(g, 0.3), "gradBias")
    # a 13 x 13 image has no room for 16 x 16 tiles: those strategies are marked as not runnable
    if H == 13:
        assert all(v is None for (cls, tile, _), v in net.timings.items() if tile is not None)
    # a 70 x 70 image needs FFT 128 untiled; tiled candidates must have been timed as well
    if H == 70:
        assert any(v is not None for (cls, tile, _), v in net.timings.items() if tile is not None)
    net.cleanupBuffers()


def test_tuned_module_memory_limit_and_inference_only(fbnn):
    P, F, k, H, pad = 4, 4, 3, 40, 1
    x = torch.zeros(2, P, H, H, device="cuda")
    net = fbnn.SpatialConvolution(P, F, k, k, 1, 1, pad, pad, maximalMemoryOverhead=1, inferenceOnly=True)
    net.updateOutput(x)                           # no FFT buffer fits in one byte: the direct path is left
    assert net.bestKey[0] == "SpatialConvolutionDirect"
    assert all(v is None or "skipped" in v or key[0] == "SpatialConvolutionDirect" for key, v in net.timings.items())
    net = fbnn.SpatialConvolution(P, F, k, k, 1, 1, pad, pad, None, True)
    net.updateOutput(x)
    assert all(v is None or v["ms"][1] == 0.0 for v in net.timings.values())
    with pytest.raises(AssertionError):
        net.updateGradInput(x, x)
    with pytest.raises(ValueError):
        net.updateOutput(torch.zeros(3, P, H, H, device="cuda"))      # tuned for another batch
    net.cleanupBuffers()


# (the oracle keeps the reference's precondition (H - kH) % stride == 0, test/ReferenceConvolutions.cpp:112-114)
@pytest.mark.parametrize("shape", [(2, 3, 4, 3, 3, 13, 15, 2, 2, 1, 1), (3, 2, 5, 5, 4, 23, 18, 3, 2, 2, 1),
                                   (1, 4, 2, 2, 2, 9, 9, 1, 1, 0, 0), (2, 3, 3, 7, 7, 23, 22, 4, 3, 6, 5)])
def test_direct_convolution_matches_oracle_with_strides(oracle, shape):
    """The non-FFT path (the reference's cuDNN fallback, fbcunn/SpatialConvolutionFFT.lua:323-393)
    against the oracle, which takes strides (test/ReferenceConvolutions.cpp:86-200)."""
    from fbcunn_amd import nn
    B, P, F, kH, kW, H, W, sH, sW, padH, padW = shape
    x = synth.uniform(61, (B, P, H, W), stream=0)
    w = synth.normal(61, (F, P, kH, kW), 0.0, 0.05, stream=1)
    bias = synth.uniform(61, (F,), -0.1, 0.1, stream=2)
    oH, oW = (H + 2 * padH - kH) // sH + 1, (W + 2 * padW - kW) // sW + 1
    g = synth.uniform(61, (B, F, oH, oW), stream=3)
    net = nn.SpatialConvolutionDirect(P, F, kW, kH, sW, sH, padW, padH)
    net.weight.copy_(dev(w))
    net.bias.copy_(dev(bias))
    net.gradWeight.fill_(float("nan"))
    net.gradBias.fill_(float("nan"))
    xd, gd = dev(x), dev(g)
    p4 = (padH, padH, padW, padW)
    want = oracle.bias_update_output(oracle.cross_correlation_valid(x, w, (sH, sW), p4), bias)
    assert want.shape == (B, F, oH, oW)
    _close(host(net.updateOutput(xd)), want, "output")
    # the oracle's full convolution is (oH - 1) sH + kH - 2 padH rows high, which can be short of the
    # input when (H + 2 padH - kH) % sH != 0; the rows it has are compared, the whole tensor through
    # the adjoint identity <out - bias, g> = <x, gradInput>
    gi = oracle.convolution_full(g, w, (sH, sW), p4)
    got = host(net.updateGradInput(xd, gd))
    _close(got[:, :, :gi.shape[2], :gi.shape[3]], gi, "gradInput")
    lhs = float(np.sum((want - bias.reshape(1, -1, 1, 1)).astype(np.float64) * g))
    assert abs(lhs - float(np.sum(x.astype(np.float64) * got))) <= 1e-4 * max(abs(lhs), 1.0)
    net.accGradParameters(xd, gd, 0.7)
    # the oracle sizes gradWeight as H + 2 padH - (oH - 1) sH rows, which exceeds kH by the rows the
    # strided windows never reach; the kH x kW corner is the layer's gradWeight
    gw = oracle.cross_correlation_reverse_valid(x, g, (sH, sW), 0.7, p4)
    _close(host(net.gradWeight), np.ascontiguousarray(gw[:, :, :kH, :kW]), "gradWeight")
    _close(host(net.gradBias), oracle.bias_acc_grad_parameters(g, 0.7), "gradBias")


def test_tuned_module_runs_strided_layers_on_the_direct_path(fbnn, oracle):
    B, P, F, k, H, s, pad = 2, 3, 4, 5, 21, 2, 2
    x = synth.uniform(71, (B, P, H, H), stream=0)
    w = synth.normal(71, (F, P, k, k), 0.0, 0.05, stream=1)
    net = fbnn.SpatialConvolution(P, F, k, k, s, s, pad, pad)
    net.weight.copy_(dev(w))
    net.bias.zero_()
    out = host(net.updateOutput(dev(x)))
    assert net.bestKey[0] == "SpatialConvolutionDirect" and len(net.timings) == 1
    _close(out, oracle.cross_correlation_valid(x, w, (s, s), (pad,) * 4), "output")
    net.cleanupBuffers()


def test_self_check_hook(fbnn):
    """fbcunn/SpatialConvolutionFFT.lua:91-133, 160-161 and fbcunn/SpatialConvolution.lua:387-399: with
    cudnnDebug set every pass is compared with the non-FFT path; the tuning front does so for its
    winner and fails loudly."""
    from fbcunn_amd import nn
    from fbcunn_amd._lib import FbfcError
    B, P, F, k, H, pad = 4, 5, 6, 3, 40, 1
    x = torch.randn(B, P, H, H, device="cuda")
    g = torch.randn(B, F, H, H, device="cuda")
    for cls, extra in (("SpatialConvolutionFBFFT", ()), ("SpatialConvolutionFFTTiled", (16, 16))):
        net = getattr(nn, cls)(P, F, k, k, 1, 1, pad, pad, *extra)
        net.cudnnDebug = True
        state = torch.cuda.get_rng_state()
        net.updateOutput(x)
        net.updateGradInput(x, g)
        net.accGradParameters(x, g, 0.5)
        assert net.cudnnChecks, cls
        assert torch.equal(state, torch.cuda.get_rng_state())   # the hook draws nothing from the caller's random stream
        net.prec = 1e-12                      # no float32 result is that close: the hook must notice
        net.updateOutput(x)
        assert not net.cudnnChecks
        net.cleanupBuffers()
    tuned = fbnn.SpatialConvolution(P, F, k, k, 1, 1, pad, pad)
    fft_only = [c for c in tuned._candidates(H, H) if c[0] != "SpatialConvolutionDirect"]
    tuned._candidates = lambda iH, iW: fft_only       # a layer this small is fastest on the direct path
    tuned.updateOutput(x)                     # tunes, then checks the winner: passes
    assert tuned.bestModuleInst.cudnnChecks
    tuned.cleanupBuffers()
    old = nn.SpatialConvolutionFFT.prec
    try:
        nn.SpatialConvolutionFFT.prec = 1e-12
        bad = fbnn.SpatialConvolution(P, F, k, k, 1, 1, pad, pad)
        bad.selfCheck = True
        # make sure an FFT strategy wins, so that there is something to check
        bad._candidates = lambda iH, iW: [("SpatialConvolutionFBFFT", None, "none")]
        bad.gradWeight.fill_(3.0)
        bad.gradBias.fill_(-2.0)
        with pytest.raises(FbfcError):
            bad.updateOutput(x)
        # a tuning run that ends in an error still leaves the caller's gradients as they were
        assert float(bad.gradWeight.min()) == 3.0 == float(bad.gradWeight.max())
        assert float(bad.gradBias.min()) == -2.0 == float(bad.gradBias.max())
    finally:
        nn.SpatialConvolutionFFT.prec = old


@pytest.mark.parametrize("shape", [(2, 3, 4, 3, 3, 13, 15, 1, 1, 1, 1), (3, 2, 5, 5, 4, 23, 18, 3, 2, 2, 1)])
def test_vendor_convolution_matches_oracle(oracle, shape):
    """The platform library's convolution behind the module protocol (the place cudnn.SpatialConvolution has
    in fbcunn/SpatialConvolution.lua:259-269) against the oracle; accGradParameters assigns."""
    from fbcunn_amd.vendor import SpatialConvolutionMIOpen
    B, P, F, kh, kw, H, W, sh, sw, ph, pw = shape
    x = synth.uniform(41, (B, P, H, W), stream=0)
    w = synth.normal(41, (F, P, kh, kw), 0.0, 0.1, stream=1)
    bias = synth.uniform(41, (F,), -0.1, 0.1, stream=2)
    oh, ow = (H + 2 * ph - kh) // sh + 1, (W + 2 * pw - kw) // sw + 1
    g = synth.uniform(41, (B, F, oh, ow), stream=3)
    net = SpatialConvolutionMIOpen(P, F, kw, kh, sw, sh, pw, ph, init=False)
    net.weight.copy_(dev(w))
    net.bias.copy_(dev(bias))
    net.gradWeight.fill_(float("nan"))
    net.gradBias.fill_(float("nan"))
    xd, gd = dev(x), dev(g)
    p4 = (ph, ph, pw, pw)
    _close(host(net.updateOutput(xd)), oracle.bias_update_output(oracle.cross_correlation_valid(x, w, (sh, sw), p4), bias), "output")
    # (what the oracle leaves out for strides that do not divide the padded extent: see the direct test above)
    gi = oracle.convolution_full(g, w, (sh, sw), p4)
    got = host(net.updateGradInput(xd, gd))
    _close(got[:, :, :gi.shape[2], :gi.shape[3]], gi, "gradInput")
    net.accGradParameters(xd, gd, 0.5)
    want_gw = np.ascontiguousarray(oracle.cross_correlation_reverse_valid(x, g, (sh, sw), 0.5, p4)[:, :, :kh, :kw])
    _close(host(net.gradWeight), want_gw, "gradWeight")
    _close(host(net.gradBias), oracle.bias_acc_grad_parameters(g, 0.5), "gradBias")
    net.gradWeight.fill_(float("nan"))
    got2 = host(net.backward(xd, gd, 0.5))
    assert np.array_equal(got2, got)
    _close(host(net.gradWeight), want_gw, "gradWeight of backward()")


def test_tuned_module_with_the_vendor_candidate(fbnn, oracle):
    """vendor=True adds the library's convolution to the candidates; whichever wins matches the oracle and,
    when it is the library, has passed the check against the direct convolution."""
    B, P, F, k, H, pad = 2, 4, 3, 3, 40, 1
    x = synth.uniform(43, (B, P, H, H), stream=0)
    w = synth.normal(43, (F, P, k, k), 0.0, 0.05, stream=1)
    bias = synth.uniform(43, (F,), -0.1, 0.1, stream=2)
    g = synth.uniform(43, (B, F, H, H), stream=3)
    net = fbnn.SpatialConvolution(P, F, k, k, 1, 1, pad, pad, vendor=True)
    net.weight.copy_(dev(w))
    net.bias.copy_(dev(bias))
    xd, gd = dev(x), dev(g)
    out = host(net.updateOutput(xd))
    key = ("SpatialConvolutionMIOpen", None, "none")
    assert key in net.timings and net.timings[key] is not None and len(net.timings[key]["ms"]) == 3
    gin = host(net.updateGradInput(xd, gd))
    net.accGradParameters(xd, gd, 1.0)
    p4 = (pad,) * 4
    _close(out, oracle.bias_update_output(oracle.cross_correlation_valid(x, w, (1, 1), p4), bias), "output")
    _close(gin, oracle.convolution_full(g, w, (1, 1), p4), "gradInput")
    _close(host(net.gradWeight), oracle.cross_correlation_reverse_valid(x, g, (1, 1), 1.0, p4), "gradWeight")
    # without the flag the library is not among the candidates
    plain = fbnn.SpatialConvolution(P, F, k, k, 1, 1, pad, pad)
    assert all(c[0] != "SpatialConvolutionMIOpen" for c in plain._candidates(H, H))
    net.cleanupBuffers()
