"""Random layers, drawn the way the reference draws its random problems (test/test_FFT.lua:588-609) but over
more of the parameter space (ragged sizes, plane counts that miss every tile size, every reuse policy, tiled and
untiled): the FFT path against the direct convolution (both on the GPU, rel-L2 <= 2e-5, the reference's own bound
for such a comparison, fbcunn/SpatialConvolutionFFT.lua:15), and backward() bit for bit against updateGradInput +
accGradParameters called one after the other.  The direct path is checked against the CPU oracle elsewhere."""
import random

import pytest
import torch

pytestmark = pytest.mark.gpu

PREC = 2e-5


def _rel(a, b):
    return (a - b).norm().item() / max(b.norm().item(), 1e-20)


def _draw(rng, tiled):
    while True:
        k = rng.choice([1, 2, 3, 3, 5, 7, 9])
        pad = rng.randint(0, k - 1)
        H = rng.randint(max(k, 2), rng.choice([12, 14, 30, 30, 60, 100]))
        W = H if rng.random() < 0.6 else rng.randint(max(k, 2), H)
        B = rng.choice([1, 2, 3, 8, 16, 32, 64, 128])
        P = rng.choice([1, 3, 16, 32, 48, 64, 96, 128])
        F = rng.choice([1, 5, 16, 32, 64, 96, 128, 256])
        if B * P * H * W > 2e7 or B * F * H * W > 2e7 or H + 2 * pad > 128 or W + 2 * pad > 128:
            continue
        oh, ow = H + 2 * pad - k + 1, W + 2 * pad - k + 1
        tile = None
        if tiled:
            tiles = [t for t in (8, 16, 32) if k <= t <= min(oh, ow)]
            if not tiles:
                continue
            tile = rng.choice(tiles)
            step = tile - k + 1
            n = max(tile, 8)
            if B * -(-oh // step) * -(-ow // step) * max(P, F) * n * n > 4e7:
                continue
        reuse = rng.choice([None, "all", "input", "weight", "output"])
        return B, P, F, k, H, W, pad, tile, reuse


@pytest.mark.parametrize("seed,count,tiled", [(11, 120, False), (12, 120, False), (13, 80, True)])
def test_random_layers_against_the_direct_path(seed, count, tiled):
    from fbcunn_amd import nn
    rng = random.Random(seed)
    torch.manual_seed(seed)
    for it in range(count):
        B, P, F, k, H, W, pad, tile, reuse = _draw(rng, tiled)
        tag = "seed %d #%d: B%d P%d F%d k%d %dx%d pad%d tile %s reuse %s" % (seed, it, B, P, F, k, H, W, pad, tile, reuse)
        kw = {} if reuse is None else {"memoryReusePolicy": reuse}
        if tiled:
            a = nn.SpatialConvolutionFFTTiled(P, F, k, k, 1, 1, pad, pad, tile, tile, **kw)
            b = nn.SpatialConvolutionFFTTiled(P, F, k, k, 1, 1, pad, pad, tile, tile, **kw)
        else:
            a = nn.SpatialConvolutionFBFFT(P, F, k, k, 1, 1, pad, pad, **kw)
            b = nn.SpatialConvolutionFBFFT(P, F, k, k, 1, 1, pad, pad, **kw)
        d = nn.SpatialConvolutionDirect(P, F, k, k, 1, 1, pad, pad)
        w = torch.randn(F, P, k, k, device="cuda") * 0.05
        bias = torch.rand(F, device="cuda") - 0.5
        for net in (a, b, d):
            net.weight.copy_(w)
            net.bias.copy_(bias)
        oh, ow = H + 2 * pad - k + 1, W + 2 * pad - k + 1
        x = torch.rand(B, P, H, W, device="cuda") * 2 - 1
        g = torch.rand(B, F, oh, ow, device="cuda") * 2 - 1
        for rep in range(2):   # the second round runs on whatever the reuse policy kept
            oa, ob, od = a.updateOutput(x), b.updateOutput(x), d.updateOutput(x)
            ga = a.backward(x, g, 0.5)
            b.updateGradInput(x, g)
            b.accGradParameters(x, g, 0.5)
            d.updateGradInput(x, g)
            d.accGradParameters(x, g, 0.5)
            for name, got, ref in (("output", oa, od), ("gradInput", ga, d.gradInput),
                                   ("gradWeight", a.gradWeight, d.gradWeight), ("gradBias", a.gradBias, d.gradBias)):
                assert torch.isfinite(got).all(), "%s: %s, round %d" % (tag, name, rep)
                assert _rel(got, ref) <= PREC, "%s: %s off the direct path by %.2e, round %d" % (tag, name, _rel(got, ref), rep)
            for name, got, ref in (("output", oa, ob), ("gradInput", ga, b.gradInput),
                                   ("gradWeight", a.gradWeight, b.gradWeight), ("gradBias", a.gradBias, b.gradBias)):
                assert torch.equal(got, ref), "%s: backward() and the two passes differ in %s, round %d" % (tag, name, rep)
        a.cleanupBuffers()
        b.cleanupBuffers()
