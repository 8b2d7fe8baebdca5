"""GPU parity of the three passes of nn.SpatialConvolutionFBFFT / ...FBFFTGemm
against the CPU oracle, following the procedure of the reference's integration
test (test/test_FFT.lua:100-256): same weights and bias on both sides, zeroed
gradients, updateOutput / updateGradInput / accGradParameters with a random
scale, compared per tensor.

Bars (both asserted):
  max |gpu - cpu| / max |cpu| <= 1e-3   the stated bound for this path
  ||gpu - cpu|| / ||cpu||     <= 1e-4   the reference's own (test/test_FFT.lua:15)
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


def _run_layer(nn, oracle, cls, B, P, F, kH, kW, iH, iW, padH, padW, seed, scale=0.37, reuse=None):
    x = synth.uniform(seed, (B, P, iH, iW), stream=0)
    w = synth.normal(seed, (F, P, kH, kW), 0.0, 0.05, stream=1)
    bias = synth.uniform(seed, (F,), -0.1, 0.1, stream=2)
    oH, oW = iH + 2 * padH - kH + 1, iW + 2 * padW - kW + 1
    g = synth.uniform(seed, (B, F, oH, oW), stream=3)
    pad = (padH, padH, padW, padW)

    net = getattr(nn, cls)(P, F, kW, kH, 1, 1, padW, padH, reuse)
    net.weight.copy_(dev(w))
    net.bias.copy_(dev(bias))
    net.gradWeight.fill_(float("nan"))       # the FBFFT path assigns: stale values must vanish
    net.gradBias.fill_(float("nan"))
    xd, gd = dev(x), dev(g)
    out = host(net.updateOutput(xd))
    gin = host(net.updateGradInput(xd, gd))
    net.accGradParameters(xd, gd, scale)
    gw, gb = host(net.gradWeight), host(net.gradBias)
    net.cleanupBuffers()

    want_out = oracle.bias_update_output(oracle.cross_correlation_valid(x, w, (1, 1), pad), bias)
    assert out.shape == want_out.shape == (B, F, oH, oW)
    _close(out, want_out, "output")
    _close(gin, oracle.convolution_full(g, w, (1, 1), pad), "gradInput")
    _close(gw, oracle.cross_correlation_reverse_valid(x, g, (1, 1), scale, pad), "gradWeight")
    _close(gb, oracle.bias_acc_grad_parameters(g, scale), "gradBias")


# batch, inputPlanes, outputPlanes, kH, kW, iH, iW, padH, padW  (the reference's column order)
PROBLEMS = [
    (1, 1, 1, 1, 1, 1, 1, 0, 0), (1, 1, 1, 1, 1, 1, 2, 0, 0), (1, 1, 1, 1, 1, 1, 3, 0, 0),   # test_FFT.lua:498-500
    (1, 16, 16, 3, 3, 8, 8, 0, 0), (8, 3, 24, 3, 3, 8, 8, 0, 0),                          # FFT size 8
    (1, 16, 16, 3, 3, 16, 16, 0, 0), (6, 3, 20, 3, 3, 16, 16, 0, 0),                      # FFT size 16
    (1, 16, 16, 3, 3, 32, 32, 0, 0), (4, 3, 12, 3, 3, 32, 32, 0, 0),                      # FFT size 32
    (2, 5, 7, 5, 5, 27, 27, 2, 2), (3, 4, 6, 3, 3, 13, 13, 1, 1), (2, 6, 5, 9, 9, 55, 55, 4, 4),
    (2, 3, 4, 3, 5, 10, 17, 2, 0), (2, 3, 4, 6, 2, 20, 9, 0, 1), (1, 2, 3, 4, 4, 40, 23, 3, 3),  # rectangular
    (3, 70, 66, 3, 3, 12, 12, 1, 1),                                                     # ragged GEMM tiles
    (5, 2, 3, 7, 7, 7, 7, 6, 6),                                                          # pad = k-1 (full conv)
    (2, 3, 4, 5, 5, 100, 90, 2, 2), (1, 2, 2, 11, 11, 118, 118, 5, 5),                    # FFT size 128
]


@pytest.mark.parametrize("cls", ["SpatialConvolutionFBFFT", "SpatialConvolutionFBFFTGemm"])
@pytest.mark.parametrize("problem", PROBLEMS)
def test_three_passes_vs_oracle(nn, oracle, cls, problem):
    _run_layer(nn, oracle, cls, *problem, seed=500 + sum(problem))


def test_random_configurations(nn, oracle):
    """test_FFT.lua:588-609 draws 25 random shapes per size regime with pad 0..4."""
    rng = np.random.RandomState(7)
    for i in range(12):
        k = int(rng.randint(1, 8))
        pad = int(rng.randint(0, min(k, 5)))
        iH = int(rng.randint(k, (30 if i % 2 else 56) - 2 * pad))
        iW = int(rng.randint(k, (30 if i % 2 else 56) - 2 * pad))
        B, P, F = (int(rng.randint(1, 6)) for _ in range(3))
        _run_layer(nn, oracle, "SpatialConvolutionFBFFT", B, P, F, k, k, iH, iW, pad, pad, seed=900 + i,
                   scale=float(rng.randint(1, 101)) / 100.0)


def test_config1_fixture_fprop(nn):
    """batch 4, 16 -> 16 planes, 32x32, 5x5, no padding, seed 1001: the committed
    CPU-oracle vector (tests/golden/config1_fprop.npy)."""
    import os
    want = np.load(os.path.join(os.path.dirname(__file__), "golden", "config1_fprop.npy"))
    x = synth.uniform(1001, (4, 16, 32, 32), stream=0)
    w = synth.uniform(1001, (16, 16, 5, 5), stream=1)
    net = nn.SpatialConvolutionFBFFT(16, 16, 5, 5)
    net.weight.copy_(dev(w))
    net.bias.zero_()
    _close(host(net.updateOutput(dev(x))), want, "config 1 output")


def test_config3_fprop_full_size(nn, oracle):
    """batch 128, 64 -> 64, 27x27, 5x5, pad 2 (FFT 32), seed 1003."""
    B, P, F, k, n, pad = 128, 64, 64, 5, 27, 2
    x = synth.uniform(1003, (B, P, n, n), stream=0)
    w = synth.normal(1003, (F, P, k, k), 0.0, 0.05, stream=1)
    bias = synth.uniform(1003, (F,), -0.1, 0.1, stream=2)
    net = nn.SpatialConvolutionFBFFT(P, F, k, k, 1, 1, pad, pad)
    net.weight.copy_(dev(w))
    net.bias.copy_(dev(bias))
    out = host(net.updateOutput(dev(x)))
    want = oracle.bias_update_output(oracle.cross_correlation_valid(x, w, (1, 1), (pad,) * 4), bias)
    _close(out, want, "config 3 output")


def test_config4_training_step_full_size(nn, oracle):
    """batch 128, 128 -> 128, 13x13, 3x3, pad 1 (FFT 16), all three passes, seed 1004."""
    _run_layer(nn, oracle, "SpatialConvolutionFBFFT", 128, 128, 128, 3, 3, 13, 13, 1, 1, seed=1004, scale=1.0)


def test_config5_large_kernel_sampled(nn, oracle):
    """batch 64, 96 -> 256, 55x55, 9x9, pad 4 (FFT 64), seed 1005.  One pass costs
    771 GFLOP on the CPU, so the oracle is evaluated on slices: output and
    gradInput for 2 images x 8 planes, gradWeight for 8 x 8 filter planes (every
    one of those values still sums over all 96 / 256 / 64 contracted planes)."""
    B, P, F, k, n, pad = 64, 96, 256, 9, 55, 4
    x = synth.uniform(1005, (B, P, n, n), stream=0)
    w = synth.normal(1005, (F, P, k, k), 0.0, 0.02, stream=1)
    g = synth.uniform(1005, (B, F, n, n), stream=3)
    net = nn.SpatialConvolutionFBFFT(P, F, k, k, 1, 1, pad, pad)
    net.weight.copy_(dev(w))
    net.bias.zero_()
    xd, gd = dev(x), dev(g)
    out = host(net.updateOutput(xd))
    gin = host(net.updateGradInput(xd, gd))
    net.accGradParameters(xd, gd, 1.0)
    gw, gb = host(net.gradWeight), host(net.gradBias)
    bs, fs, ps = [0, 63], list(range(100, 108)), list(range(40, 48))
    p4 = (pad,) * 4
    _close(out[bs][:, fs], oracle.cross_correlation_valid(x[bs], w[fs], (1, 1), p4), "config 5 output")
    _close(gin[bs][:, ps], oracle.convolution_full(g[bs], w[:, ps], (1, 1), p4), "config 5 gradInput")
    _close(gw[fs][:, ps], oracle.cross_correlation_reverse_valid(x[:, ps], g[:, fs], (1, 1), 1.0, p4),
           "config 5 gradWeight")
    _close(gb, oracle.bias_acc_grad_parameters(g, 1.0), "config 5 gradBias")
    # a second slice that straddles the contraction's tile borders (64 images, filter planes 64 and 192,
    # input planes in the last 32-wide block) and the transforms' plane groups (test/test_FFT.lua:160-256
    # compares whole tensors; here every sampled value still sums over all contracted planes)
    bs, fs, ps = [1, 31, 62], list(range(60, 69)) + list(range(250, 256)), list(range(90, 96))
    _close(out[bs][:, fs], oracle.cross_correlation_valid(x[bs], w[fs], (1, 1), p4), "config 5 output, slice 2")
    _close(gin[bs][:, ps], oracle.convolution_full(g[bs], w[:, ps], (1, 1), p4), "config 5 gradInput, slice 2")
    _close(gw[fs][:, ps], oracle.cross_correlation_reverse_valid(x[:, ps], g[:, fs], (1, 1), 1.0, p4),
           "config 5 gradWeight, slice 2")
    # size-independent property on the whole tensors: <out, g> = <x, gradInput> = <w, gradWeight>
    lhs = float(torch.dot(net.output.double().flatten(), gd.double().flatten()))
    assert abs(lhs - float(torch.dot(xd.double().flatten(), net.gradInput.double().flatten()))) <= 1e-4 * abs(lhs)
    assert abs(lhs - float(torch.dot(net.weight.double().flatten(), net.gradWeight.double().flatten()))) <= 1e-4 * abs(lhs)


def test_closed_form_ones(nn):
    """test/ConvolutionTest.cpp:1316-1374: ones(7x7) fully convolved with ones(3x3)."""
    net = nn.SpatialConvolutionFBFFT(1, 1, 3, 3)
    net.weight.fill_(1.0)
    edge = np.array([1, 2, 3, 3, 3, 3, 3, 2, 1], np.float64)
    gin = host(net.updateGradInput(torch.zeros(1, 1, 9, 9, device="cuda"), torch.ones(1, 1, 7, 7, device="cuda")))
    np.testing.assert_allclose(gin[0, 0], np.outer(edge, edge), atol=5e-5)


def test_delta_kernel_is_a_shift(nn):
    net = nn.SpatialConvolutionFBFFT(1, 1, 3, 3, 1, 1, 1, 1)
    net.weight.zero_()
    net.weight[0, 0, 2, 0] = 1.0
    net.bias.zero_()
    x = synth.uniform(77, (2, 1, 12, 12))
    out = host(net.updateOutput(dev(x)))
    want = np.zeros_like(x)
    want[:, :, :-1, 1:] = x[:, :, 1:, :-1]          # out[r][c] = x[r+1][c-1]
    np.testing.assert_allclose(out, want, atol=1e-5)


def test_reuse_policy_gives_same_results(nn, oracle):
    """memoryReuseAll (bprop reuses FFT(weight), accGrad reuses FFT(gradOutput) and
    FFT(input)) must not change any result (SpatialConvolutionFBFFT.lua:226-230,305-322)."""
    _run_layer(nn, oracle, "SpatialConvolutionFBFFT", 4, 6, 5, 3, 3, 13, 13, 1, 1, seed=321, reuse="all")
    _run_layer(nn, oracle, "SpatialConvolutionFBFFT", 4, 6, 5, 5, 5, 20, 20, 2, 2, seed=322, reuse=["weight"])


def test_acc_grad_overwrites_and_bias_functions(nn, oracle):
    B, F, h = 5, 7, 11
    g = synth.uniform(55, (B, F, h, h))
    gb = torch.full((F,), 123.0, device="cuda")
    nn.accGradParametersBias(dev(g), gb, 0.5)
    np.testing.assert_allclose(host(gb), oracle.bias_acc_grad_parameters(g, 0.5), rtol=5e-4, atol=1e-5)
    bias = np.arange(F, dtype=np.float32)
    out = dev(g)
    nn.updateOutputBias(out, dev(bias))
    np.testing.assert_allclose(host(out), oracle.bias_update_output(g, bias), rtol=1e-6, atol=1e-6)


@pytest.mark.parametrize("t1,t2", [(0, 1), (1, 3), (2, 3), (0, 2), (1, 1)])
def test_bias_functions_take_non_contiguous_tensors(nn, oracle, t1, t2):
    """test/BiasTest.cpp:38-63: the feature-map tensor is made with two dimensions swapped and
    transposed back, so that it has the logical shape but an out-of-order memory layout."""
    B, F, h, w = 5, 7, 6, 11
    g = synth.uniform(56 + t1 + 4 * t2, (B, F, h, w))
    sizes = [B, F, h, w]
    sizes[t1], sizes[t2] = sizes[t2], sizes[t1]
    store = torch.empty(sizes, device="cuda")
    view = store.transpose(t1, t2)              # logical (B, F, h, w), non-contiguous unless t1 == t2
    view.copy_(dev(g))
    assert tuple(view.shape) == (B, F, h, w) and view.is_contiguous() == (t1 == t2)
    gb_store = torch.full((F, 3), 123.0, device="cuda")
    gb = gb_store[:, 1]                          # stride 3
    nn.accGradParametersBias(view, gb, 0.25)
    np.testing.assert_allclose(host(gb), oracle.bias_acc_grad_parameters(g, 0.25), rtol=5e-4, atol=1e-5)
    assert (host(gb_store[:, 0]) == 123.0).all() and (host(gb_store[:, 2]) == 123.0).all()
    bias = synth.uniform(77, (F,))
    nn.updateOutputBias(view, dev(bias))
    np.testing.assert_allclose(host(view.contiguous()), oracle.bias_update_output(g, bias), rtol=1e-6, atol=1e-6)


@pytest.mark.parametrize("reuse", ["all", "output"])
def test_second_acc_grad_under_reuse_transforms_its_own_grad_output(nn, oracle, reuse):
    """updateOutput, accGradParameters, updateOutput, accGradParameters with another gradOutput and no
    updateGradInput in between: the second accGradParameters must not take the spectrum of the first
    gradOutput (memoryReuseOutput only covers the updateGradInput -> accGradParameters pair of one step,
    fbcunn/SpatialConvolutionFBFFT.lua:305-322)."""
    B, P, F, k, H, pad = 4, 6, 5, 3, 13, 1
    x = synth.uniform(41, (B, P, H, H), stream=0)
    w = synth.normal(41, (F, P, k, k), 0.0, 0.05, stream=1)
    g1 = synth.uniform(41, (B, F, H, H), stream=3)
    g2 = synth.uniform(42, (B, F, H, H), stream=3)
    net = nn.SpatialConvolutionFBFFT(P, F, k, k, 1, 1, pad, pad, reuse)
    net.weight.copy_(dev(w))
    xd = dev(x)
    p4 = (pad,) * 4
    for g in (g1, g2, g1):
        net.updateOutput(xd)
        net.accGradParameters(xd, dev(g), 1.0)
        _close(host(net.gradWeight), oracle.cross_correlation_reverse_valid(x, g, (1, 1), 1.0, p4), "gradWeight")
        _close(host(net.gradBias), oracle.bias_acc_grad_parameters(g, 1.0), "gradBias")
    # the pair the policy is for still shares the spectrum and gives the same numbers
    net.updateOutput(xd)
    net.updateGradInput(xd, dev(g2))
    net.accGradParameters(xd, dev(g2), 1.0)
    _close(host(net.gradWeight), oracle.cross_correlation_reverse_valid(x, g2, (1, 1), 1.0, p4), "gradWeight")
    # two accGradParameters in a row with different gradOutput
    net.accGradParameters(xd, dev(g1), 1.0)
    _close(host(net.gradWeight), oracle.cross_correlation_reverse_valid(x, g1, (1, 1), 1.0, p4), "gradWeight")
    net.cleanupBuffers()


def test_module_argument_errors(nn):
    with pytest.raises(ValueError):
        nn.SpatialConvolutionFBFFT(3, 4, 3, 3, 2, 1)            # stride
    with pytest.raises(ValueError):
        nn.SpatialConvolutionFBFFT(3, 4, 3, 3, 1, 1, 3, 0)      # pad >= kernel
    net = nn.SpatialConvolutionFBFFT(3, 4, 3, 3)
    with pytest.raises(TypeError):
        net.updateOutput(torch.zeros(1, 3, 8, 8))               # not on the GPU
    with pytest.raises(nn.FbfcError) as e:
        net.updateOutput(torch.zeros(1, 3, 200, 200, device="cuda"))   # FFT size 256: beyond fbfft's 128
    assert e.value.code == 2


@pytest.mark.parametrize("cls,extra", [("SpatialConvolutionFBFFT", ()), ("SpatialConvolutionFFTTiled", (16, 16))])
def test_backward_equals_the_two_passes(nn, oracle, cls, extra):
    """backward() shares FFT(gradOutput) between its two passes (SpatialConvolutionFFT.lua:405-416):
    same results as updateGradInput + accGradParameters, and as the oracle."""
    B, P, F, k, H, pad = 3, 5, 4, 3, 29, 1
    x = synth.uniform(41, (B, P, H, H), stream=0)
    w = synth.normal(41, (F, P, k, k), 0.0, 0.05, stream=1)
    g = synth.uniform(41, (B, F, H, H), stream=3)
    xd, gd = dev(x), dev(g)
    a = getattr(nn, cls)(P, F, k, k, 1, 1, pad, pad, *extra)
    b = getattr(nn, cls)(P, F, k, k, 1, 1, pad, pad, *extra)
    for net in (a, b):
        net.weight.copy_(dev(w))
        net.gradWeight.fill_(float("nan"))
        net.gradBias.fill_(float("nan"))
    gin = host(a.backward(xd, gd, 0.7))
    b.updateGradInput(xd, gd)
    b.accGradParameters(xd, gd, 0.7)
    assert np.array_equal(gin, host(b.gradInput))
    assert np.array_equal(host(a.gradWeight), host(b.gradWeight))
    assert np.array_equal(host(a.gradBias), host(b.gradBias))
    p4 = (pad,) * 4
    _close(gin, oracle.convolution_full(g, w, (1, 1), p4), "gradInput")
    _close(host(a.gradWeight), oracle.cross_correlation_reverse_valid(x, g, (1, 1), 0.7, p4), "gradWeight")
    _close(host(a.gradBias), oracle.bias_acc_grad_parameters(g, 0.7), "gradBias")
    a.cleanupBuffers()
    b.cleanupBuffers()


# (B, P, F, k, H, pad, reuse, what the contraction stage must have launched)
_GROUPED = [
    (128, 128, 128, 3, 13, 1, None, "cgemm_backward_kernel"),    # N = 16: tiles + split blocks of both problems
    (128, 128, 128, 3, 13, 1, "all", "cgemm_backward_kernel"),
    (64, 64, 64, 5, 27, 2, None, "cgemm_backward_kernel"),       # N = 32
    (64, 64, 128, 3, 13, 0, None, "cgemm_backward_kernel"),      # split blocks only + tiles and blocks
    (16, 96, 64, 3, 14, 1, None, "cgemm_"),                      # 96 planes, even sizes: whatever kernels fit
    (8, 32, 32, 9, 57, 0, None, "cgemm_"),                       # N = 64: stages of several launches
    # partial reuse: backward() transforms fewer tensors and must still launch them the way its two passes do
    # (at N = 64 the size of a launch picks the kernel)
    (64, 128, 64, 3, 58, 1, "weight", "cgemm_"),
    (32, 16, 256, 2, 32, 1, "weight", "cgemm_"),
    (64, 128, 64, 3, 58, 1, "input", "cgemm_"),
    (16, 32, 32, 3, 14, 1, "weight", "cgemm_"),                  # N = 16, even sizes
    (16, 32, 32, 3, 13, 0, "output", "cgemm_"),
    # input even-sized, gradOutput odd-sized: the two staging variants of the forward transform meet
    (16, 32, 32, 2, 14, 0, "weight", "cgemm_"),
    (16, 32, 32, 2, 14, 0, None, "cgemm_"),
    (8, 16, 16, 4, 30, 0, "input", "cgemm_"),
    # N = 32: the forward kernel is picked per operand by its plane count (12288 planes of gradOutput take the
    # two-rows-per-lane kernel, 8192 of input and 6144 of weight the one-row-per-lane one); with partial reuse
    # backward() transforms another subset of them than its two passes do
    (128, 64, 96, 5, 27, 2, None, "cgemm_"),
    (128, 64, 96, 5, 27, 2, "weight", "cgemm_"),
    (128, 64, 96, 5, 27, 2, "input", "cgemm_"),
    (128, 96, 64, 5, 26, 2, "output", "cgemm_"),
]


@pytest.mark.parametrize("B,P,F,k,H,pad,reuse,mm", _GROUPED)
def test_backward_one_grid_per_stage(nn, B, P, F, k, H, pad, reuse, mm):
    """An untiled backward() issues each stage of its two passes as one grid where one kernel can
    take them all (SpatialConvolutionFFT.lua:405-416 only orders the passes): bit-equal to the two
    passes run one after the other, with and without buffer reuse, and again on a second call."""
    x = synth.uniform(91, (B, P, H, H), stream=0)
    w = synth.normal(91, (F, P, k, k), 0.0, 0.05, stream=1)
    oh = H + 2 * pad - k + 1
    xd = dev(x)
    kw = {} if reuse is None else {"memoryReusePolicy": reuse}
    a = nn.SpatialConvolutionFBFFT(P, F, k, k, 1, 1, pad, pad, **kw)
    b = nn.SpatialConvolutionFBFFT(P, F, k, k, 1, 1, pad, pad, **kw)
    for net in (a, b):
        net.weight.copy_(dev(w))
    for it in range(2):
        g = synth.uniform(92 + it, (B, F, oh, oh), stream=3)
        gd = dev(g)
        for net in (a, b):
            net.gradWeight.fill_(float("nan"))
            net.gradBias.fill_(float("nan"))
            net.updateOutput(xd)     # with reuse: leaves the spectra of input and weight in the plan
        gin = host(a.backward(xd, gd, 0.7))
        stages = a.stageKernels(xd)
        b.updateGradInput(xd, gd)
        b.accGradParameters(xd, gd, 0.7)
        assert np.isfinite(gin).all()
        assert np.array_equal(gin, host(b.gradInput)), "gradInput, call %d" % it
        assert np.array_equal(host(a.gradWeight), host(b.gradWeight)), "gradWeight, call %d" % it
        assert np.array_equal(host(a.gradBias), host(b.gradBias)), "gradBias, call %d" % it
        assert mm in stages["mm"], stages
        if mm == "cgemm_backward_kernel":
            # one launch per stage
            assert all(v.count("grid=") == 1 for v in stages.values()), stages
    a.cleanupBuffers()
    b.cleanupBuffers()


def test_backward_between_other_passes(nn, oracle):
    """backward() reuses the spectrum updateGradInput leaves in the plan: with other passes and
    changing inputs around it, every result must still be the one of the current inputs."""
    B, P, F, k, H, pad = 4, 6, 5, 3, 13, 1
    net = nn.SpatialConvolutionFBFFT(P, F, k, k, 1, 1, pad, pad)
    w = synth.normal(51, (F, P, k, k), 0.0, 0.05, stream=1)
    net.weight.copy_(dev(w))
    net.bias.zero_()
    p4 = (pad,) * 4
    for it in range(4):
        x = synth.uniform(60 + it, (B, P, H, H), stream=0)
        g = synth.uniform(60 + it, (B, F, H, H), stream=3)
        xd, gd = dev(x), dev(g)
        out = net.updateOutput(xd)
        gin = net.backward(xd, gd, 1.0)
        out2 = net.updateOutput(xd)
        _close(host(gin), oracle.convolution_full(g, w, (1, 1), p4), "gradInput %d" % it)
        _close(host(net.gradWeight), oracle.cross_correlation_reverse_valid(x, g, (1, 1), 1.0, p4), "gradWeight %d" % it)
        _close(host(net.gradBias), oracle.bias_acc_grad_parameters(g, 1.0), "gradBias %d" % it)
        _close(host(out2), oracle.cross_correlation_valid(x, w, (1, 1), p4), "output %d" % it)
    net.cleanupBuffers()


def test_spectrum_store_policy_does_not_change_results(nn):
    """How the forward transforms store their spectra (written through for the contraction to find in the
    memory-side cache, or non-temporal) is a matter of speed only: all three passes are bit-identical either way."""
    from fbcunn_amd import _lib
    B, P, F, k, H, pad = 16, 32, 64, 3, 13, 1
    x = dev(synth.uniform(71, (B, P, H, H), stream=0))
    g = dev(synth.uniform(71, (B, F, H, H), stream=3))
    w = dev(synth.normal(71, (F, P, k, k), 0.0, 0.05, stream=1))
    results = []
    try:
        for mode in (1, -1):
            _lib.check(_lib.lib().fbfc_debug_force_spectrum_streaming(mode))
            net = nn.SpatialConvolutionFBFFT(P, F, k, k, 1, 1, pad, pad)
            net.weight.copy_(w)
            net.bias.zero_()
            out = host(net.updateOutput(x)).copy()
            gin = host(net.updateGradInput(x, g)).copy()
            net.accGradParameters(x, g, 1.0)
            results.append((out, gin, host(net.gradWeight).copy(), host(net.gradBias).copy()))
            net.cleanupBuffers()
    finally:
        _lib.check(_lib.lib().fbfc_debug_force_spectrum_streaming(-1))
    for other in results[1:]:
        for a, b in zip(results[0], other):
            assert np.isfinite(a).all() and np.array_equal(a, b)


@pytest.mark.parametrize("shape", [(16, 32, 32, 3, 13, 1), (2, 8, 24, 9, 55, 4)])
def test_timed_passes_give_the_untimed_results(nn, shape):
    """fbfc_plan_set_timed: with repetitions (reps > 0) and with per-launch dispatch timing (reps < 0) a pass
    makes the launches of an untimed one, so every result keeps its bits; every stage that ran reports a
    positive time, and the per-launch figure of a stage is no longer than the same stage between two events."""
    B, P, F, k, H, pad = shape
    o = H + 2 * pad - k + 1
    net = nn.SpatialConvolutionFBFFT(P, F, k, k, 1, 1, pad, pad)
    net.weight.copy_(dev(synth.normal(8, (F, P, k, k), 0.0, 0.05, stream=1)))
    net.bias.copy_(dev(synth.uniform(8, (F,), -0.1, 0.1, stream=2)))
    x, g = dev(synth.uniform(8, (B, P, H, H), stream=0)), dev(synth.uniform(8, (B, F, o, o), stream=3))

    def step():
        net.updateOutput(x)
        net.updateGradInput(x, g)
        net.accGradParameters(x, g, 0.5)
        return [host(t).copy() for t in (net.output, net.gradInput, net.gradWeight, net.gradBias)]

    want = step()
    times = {}
    for reps in (1, 3, -1):
        net.timed = reps
        got = step()
        for a, b in zip(got, want):
            assert np.array_equal(a, b), "timed = %d changes a result" % reps
        times[reps] = net.stageTimes(x)               # of the last pass, accGradParameters
        assert times[reps]["mm"] > 0 and times[reps]["ifft"] > 0 and times[reps]["fft_a"] > 0
    net.timed = False
    for s in ("fft_a", "mm", "ifft"):
        assert times[-1][s] <= times[1][s] * 1.05 + 0.002, (s, times)
    net.cleanupBuffers()
