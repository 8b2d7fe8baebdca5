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
    from fbcunn_amd._lib import FbfcError
    with pytest.raises(FbfcError):
        net.updateOutput(x)                       # nothing fits in one byte
    assert all(v is None or "skipped" in v for v in net.timings.values())
    net = fbnn.SpatialConvolution(P, F, k, k, 1, 1, pad, pad, None, True)
    net.updateOutput(x)
    assert all(v is None or v["ms"][1] == 0.0 for v in net.timings.values())
    with pytest.raises(AssertionError):
        net.updateGradInput(x, x)
    with pytest.raises(ValueError):
        net.updateOutput(torch.zeros(3, P, H, H, device="cuda"))      # tuned for another batch
    net.cleanupBuffers()


def test_tuned_module_rejects_strides(fbnn):
    with pytest.raises(ValueError):
        fbnn.SpatialConvolution(3, 3, 3, 3, 2, 2)
