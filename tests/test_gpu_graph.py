"""The three passes can be captured into a HIP graph: they allocate nothing, do not synchronise
and issue no memset.  Every replay is checked against the eager result, with eager work and
synchronisation between the replays."""
import numpy as np
import pytest
import torch

from fbcunn_amd import synth
from gpu_util import dev, host

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("B,P,F,k,H,pad", [(8, 32, 32, 3, 13, 1), (4, 16, 48, 5, 27, 2), (2, 16, 16, 9, 55, 4)])
def test_passes_replay_from_a_graph(B, P, F, k, H, pad):
    from fbcunn_amd import nn
    o = H + 2 * pad - k + 1
    net = nn.SpatialConvolutionFBFFT(P, F, k, k, 1, 1, pad, pad)
    net.weight.copy_(dev(synth.normal(5, (F, P, k, k), 0.0, 0.05, stream=1)))
    net.bias.copy_(dev(synth.uniform(5, (F,), -0.1, 0.1, stream=2)))
    x, g = dev(synth.uniform(5, (B, P, H, H), stream=0)), dev(synth.uniform(5, (B, F, o, o), stream=3))

    def step():
        net.updateOutput(x)
        net.updateGradInput(x, g)
        net.accGradParameters(x, g, 0.25)

    results = lambda: [net.output, net.gradInput, net.gradWeight, net.gradBias]
    step()                                   # creates the plan and the result tensors
    torch.cuda.synchronize()
    want = [host(t).copy() for t in results()]

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
        (x * 2).sum().item()                 # eager work and a synchronisation between replays
        graph.replay()
        torch.cuda.synchronize()
        for got, ref, name in zip(results(), want, ("output", "gradInput", "gradWeight", "gradBias")):
            assert np.array_equal(host(got), ref), "replay %d: %s differs from the eager result" % (rep, name)
    net.cleanupBuffers()


@pytest.mark.parametrize("B,P,F,k,H,pad", [(64, 64, 128, 3, 13, 1), (4, 16, 48, 5, 27, 2)])
def test_backward_replays_from_a_graph(B, P, F, k, H, pad):
    """backward() with one grid per stage: prepareBackward() makes the two extra spectrum buffers, the pass
    itself allocates nothing and can be captured."""
    from fbcunn_amd import nn
    o = H + 2 * pad - k + 1
    net = nn.SpatialConvolutionFBFFT(P, F, k, k, 1, 1, pad, pad)
    net.weight.copy_(dev(synth.normal(6, (F, P, k, k), 0.0, 0.05, stream=1)))
    x, g = dev(synth.uniform(6, (B, P, H, H), stream=0)), dev(synth.uniform(6, (B, F, o, o), stream=3))

    def step():
        net.updateOutput(x)
        net.backward(x, g, 0.5)

    results = lambda: [net.output, net.gradInput, net.gradWeight, net.gradBias]
    assert net.prepareBackward(x) is True
    step()
    torch.cuda.synchronize()
    if B == 64:   # shapes the tile kernels take run both contractions as one grid
        assert "cgemm_backward_kernel" in net.stageKernels(x)["mm"]
    assert ";" not in net.stageKernels(x)["ifft"]   # both inverse transforms in one launch: the one-grid-per-stage form ran
    want = [host(t).copy() for t in results()]
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
        (x * 2).sum().item()
        graph.replay()
        torch.cuda.synchronize()
        for got, ref, name in zip(results(), want, ("output", "gradInput", "gradWeight", "gradBias")):
            assert np.array_equal(host(got), ref), "replay %d: %s differs from the eager result" % (rep, name)
    net.cleanupBuffers()
