"""Host-side mirror of fbnn.SpatialConvolution (fbcunn/SpatialConvolution.lua): the front
that, on the first updateOutput, times the strategies that fit the layer and keeps the
fastest (:188-422).  Candidates: the FFT modules (untiled, tiles of 16 and 32, with and
without memory reuse) and the direct convolution, which stands where the reference has
cuDNN: it runs every layer (strides above 1, sizes no transform covers) and it is what
the winner is checked against after tuning (:387-399), to the reference's 2e-5.  With
vendor=True the platform library's convolution (MIOpen) is timed as one more candidate.
"""
import time

import torch

from . import _lib
from . import modules as nn
from . import vendor as vendor_mod

__all__ = ["SpatialConvolution"]


def _time_function(fn, *args):
    """3 trials, the first dropped, mean of the rest in ms (SpatialConvolution.lua:98-112)."""
    num_trials, total = 3, 0.0
    torch.cuda.synchronize()
    for i in range(num_trials):
        t0 = time.perf_counter()
        fn(*args)
        torch.cuda.synchronize()
        if i > 0:
            total += time.perf_counter() - t0
    return total / (num_trials - 1) * 1e3


class SpatialConvolution:
    """fbnn.SpatialConvolution(nInputPlane, nOutputPlane, kW, kH, dW, dH, padLeft, padUp,
    maximalMemoryOverhead, inferenceOnly)."""

    reportErrors = False
    # the direct candidate is plain, untuned code: above this many FLOPs per pass it is timed on a slice of
    # the batch and the time scaled up, so that tuning a large layer does not spend seconds on it
    directTimingFlops = 20e9

    def __init__(self, nInputPlane, nOutputPlane, kW, kH, dW=1, dH=1, padLeft=0, padUp=0,
                 maximalMemoryOverhead=None, inferenceOnly=False, device="cuda", vendor=False):
        self.inputPlanes, self.outputPlanes = nInputPlane, nOutputPlane
        self.kW, self.kH, self.dW, self.dH = kW, kH, dW, dH
        self.padLeft, self.padUp = padLeft, padUp
        self.maximalMemoryOverhead = maximalMemoryOverhead
        self.inferenceOnly = bool(inferenceOnly)
        self.vendor = bool(vendor)
        self.reportLevel = 0
        self.device = torch.device(device)
        # after tuning, run the winning FFT strategy against the direct convolution (the reference
        # always does, fbcunn/SpatialConvolution.lua:387-399) and fail if they differ
        self.selfCheck = True
        # parameters live here and are handed to the strategy that wins
        holder = nn.SpatialConvolutionDirect(nInputPlane, nOutputPlane, kW, kH, dW, dH, padLeft, padUp, device=device)
        self.weight, self.bias = holder.weight, holder.bias
        self.gradWeight, self.gradBias = holder.gradWeight, holder.gradBias
        self.output = None
        self.gradInput = None
        self.bestModuleInst = None
        self.timings = {}

    def setInferenceOnly(self, val):
        assert isinstance(val, bool)
        self.inferenceOnly = val

    # -- candidates (SpatialConvolution.lua:237-300) -----------------------------------
    def _candidates(self, iH, iW):
        reuse_all, reuse_none = nn.SpatialConvolutionFFT.memoryReuseAll, nn.SpatialConvolutionFFT.memoryReuseNone
        direct = [("SpatialConvolutionDirect", None, reuse_none)]
        if self.vendor:
            direct.append(("SpatialConvolutionMIOpen", None, reuse_none))
        if self.dW != 1 or self.dH != 1:
            return direct           # "fft only supports stride-1 convolutions atm"
        cands = direct + [("SpatialConvolutionFBFFT", None, reuse_all), ("SpatialConvolutionFBFFT", None, reuse_none)]
        if self.kH <= 9 and self.kW <= 9:
            tiles = (16, 32)
        else:
            tiles = (32,)
        for t in tiles:
            for reuse in (reuse_none, reuse_all):
                cands.append(("SpatialConvolutionFFTTiled", t, reuse))
        # the fused kernels keep the spectra on chip and sum over the contracted planes on the vector ALUs:
        # a candidate where one side has few planes (first and last layers)
        if min(self.inputPlanes, self.outputPlanes) <= 8:
            for t in tiles:
                cands.append(("SpatialConvolutionFFTTiledIterated", t, reuse_none))
        return cands

    def _plan_bytes(self, batch, iH, iW, tile, reuse, cls=""):
        """Frequency-buffer bytes the strategy would allocate, or None if it cannot run."""
        kw = dict(batch=batch, in_planes=self.inputPlanes, out_planes=self.outputPlanes, in_h=iH, in_w=iW,
                  k_h=self.kH, k_w=self.kW, stride_h=self.dH, stride_w=self.dW, pad_h=self.padUp,
                  pad_w=self.padLeft)
        try:
            info = _lib.plan_query(tile_h=tile or 0, tile_w=tile or 0, **kw)
        except _lib.FbfcError:
            return None
        if cls.endswith("Iterated"):
            return info.weight_freq_bytes       # the fused passes own the weight spectrum only
        sizes = (info.input_freq_bytes, info.weight_freq_bytes, info.output_freq_bytes)
        # + the result buffer of a reuse policy, + what backward() adds (training only)
        return (sum(sizes) + (max(sizes) if reuse != nn.SpatialConvolutionFFT.memoryReuseNone else 0)
                + (0 if self.inferenceOnly else info.backward_freq_bytes))

    def _make(self, cls, tile, reuse):
        args = (self.inputPlanes, self.outputPlanes, self.kW, self.kH, self.dW, self.dH, self.padLeft, self.padUp)
        if cls == "SpatialConvolutionDirect":
            inst = nn.SpatialConvolutionDirect(*args, device=self.device, init=False)
        elif cls == "SpatialConvolutionMIOpen":
            inst = vendor_mod.SpatialConvolutionMIOpen(*args, device=self.device, init=False)
        elif tile is None:
            inst = getattr(nn, cls)(*args, reuse, device=self.device)
        elif cls.endswith("Iterated"):
            inst = getattr(nn, cls)(*args, tile, tile, device=self.device)
        else:
            inst = getattr(nn, cls)(*args, tile, tile, reuse, device=self.device)
        inst.weight, inst.bias = self.weight, self.bias
        inst.gradWeight, inst.gradBias = self.gradWeight, self.gradBias
        return inst

    def _pick(self, input, grad_output):
        """Times every candidate and returns (winner, its ms); raises if none runs or the self-check fails."""
        B, _, iH, iW = input.shape
        best, best_ms = None, float("inf")
        self.timings = {}
        for cls, tile, reuse in self._candidates(iH, iW):
            spatial = cls in ("SpatialConvolutionDirect", "SpatialConvolutionMIOpen")
            nbytes = 0 if spatial else self._plan_bytes(B, iH, iW, tile, reuse, cls)
            key = (cls, tile, reuse)
            if nbytes is None:
                self.timings[key] = None          # the strategy cannot run this layer
                continue
            if self.maximalMemoryOverhead is not None and nbytes > self.maximalMemoryOverhead:
                self.timings[key] = {"memoryConsumption": nbytes, "skipped": "exceeds maximalMemoryOverhead"}
                continue
            inst = self._make(cls, tile, reuse)
            x_t, g_t, factor = input, grad_output, 1.0
            if cls == "SpatialConvolutionDirect":
                flops = 2.0 * B * self.outputPlanes * self.inputPlanes * grad_output.size(2) * grad_output.size(3) * self.kH * self.kW
                if flops > self.directTimingFlops and B > 1:
                    nb = max(1, int(B * self.directTimingFlops / flops))
                    x_t, g_t, factor = input[:nb], grad_output[:nb], B / float(nb)
            try:
                t1 = factor * _time_function(inst.updateOutput, x_t)
                t2 = t3 = 0.0
                if not self.inferenceOnly:
                    t2 = factor * _time_function(inst.updateGradInput, x_t, g_t)
                    t3 = factor * _time_function(inst.accGradParameters, x_t, g_t, 1.0)
            except (_lib.FbfcError, RuntimeError) as err:
                if cls != "SpatialConvolutionMIOpen" and not isinstance(err, _lib.FbfcError):
                    raise
                if self.reportErrors:
                    print("%s tile %s: %s" % (cls, tile, err))
                inst.cleanupBuffers()
                self.timings[key] = None
                continue
            self.timings[key] = {"memoryConsumption": nbytes, "ms": (t1, t2, t3)}
            if t1 + t2 + t3 < best_ms:
                if best is not None:
                    best.cleanupBuffers()
                best, best_ms = inst, t1 + t2 + t3
                self.bestKey = key
            else:
                inst.cleanupBuffers()
        if best is None:
            raise _lib.FbfcError(_lib.ERR_UNSUPPORTED_SIZE, "no strategy can run this layer")
        # correctness check of an FFT winner against the direct convolution, on random data
        if self.selfCheck and isinstance(best, vendor_mod.SpatialConvolutionMIOpen):
            self._check_vendor(best, input, grad_output)
        elif self.selfCheck and not isinstance(best, nn.SpatialConvolutionDirect):
            best.cudnnDebug, best.cudnnChecks = True, True
            x = torch.randn_like(input)
            g = torch.randn_like(grad_output)
            best.updateOutput(x)
            if not self.inferenceOnly:
                best.updateGradInput(x, g)
                best.accGradParameters(x, g, 1.0)
            best.cudnnDebug = False
            if not best.cudnnChecks:
                best.cleanupBuffers()
                raise _lib.FbfcError(_lib.ERR_HIP, "self-check of %s against the direct convolution failed" % (self.bestKey,))
        return best, best_ms

    def _check_vendor(self, best, input, grad_output):
        """The library's results against the direct convolution on random data, to the tolerance the FFT
        modules' own check uses."""
        ref = self._make("SpatialConvolutionDirect", None, None)
        ref.gradWeight, ref.gradBias = torch.empty_like(self.gradWeight), torch.empty_like(self.gradBias)
        x = torch.randn_like(input)
        g = torch.randn_like(grad_output)
        pairs = [(best.updateOutput(x), ref.updateOutput(x))]
        if not self.inferenceOnly:
            pairs.append((best.updateGradInput(x, g), ref.updateGradInput(x, g)))
            best.accGradParameters(x, g, 1.0)
            ref.accGradParameters(x, g, 1.0)
            pairs.append((best.gradWeight, ref.gradWeight))
            pairs.append((best.gradBias, ref.gradBias))
        for got, want in pairs:
            want = want.double()
            err = float((want - got.double()).norm()) / (float(want.norm()) + 1e-8)
            if not (bool(torch.isfinite(got).all()) and err <= nn.SpatialConvolutionFFT.prec):
                raise _lib.FbfcError(_lib.ERR_HIP, "self-check of the vendor convolution against the direct one failed")

    def _tune(self, input):
        B, _, iH, iW = input.shape
        oH, oW = (iH + 2 * self.padUp - self.kH) // self.dH + 1, (iW + 2 * self.padLeft - self.kW) // self.dW + 1
        grad_output = torch.zeros(B, self.outputPlanes, max(oH, 1), max(oW, 1), device=input.device)
        # tuning must not disturb the caller's gradients, whichever way it ends
        keep_gw, keep_gb = self.gradWeight.clone(), self.gradBias.clone()
        try:
            best, best_ms = self._pick(input, grad_output)
        finally:
            self.gradWeight.copy_(keep_gw)
            self.gradBias.copy_(keep_gb)
        if self.reportLevel >= 1:
            print("Best FFT: ", best_ms, " ", self.bestKey)
        self.bestModuleInst = best
        self.batchSize, self.iH, self.iW = B, iH, iW

    # -- nn.Module protocol --------------------------------------------------------------
    def updateOutput(self, input):
        if input.dim() != 4:
            raise ValueError("Only supports 4-D tensors atm")
        if self.bestModuleInst is None:
            self._tune(input)
        if (self.batchSize, self.iH, self.iW) != (input.size(0), input.size(2), input.size(3)):
            raise ValueError("tuned for %s, got %s" % ((self.batchSize, self.iH, self.iW), tuple(input.shape)))
        self.bestModuleInst.weight, self.bestModuleInst.bias = self.weight, self.bias
        self.output = self.bestModuleInst.updateOutput(input)
        return self.output

    forward = updateOutput

    def updateGradInput(self, input, gradOutput):
        assert self.bestModuleInst is not None, "Must have been tuned in updateOutput already!"
        assert not self.inferenceOnly, "Inference only specified => no gradInput "
        self.gradInput = self.bestModuleInst.updateGradInput(input, gradOutput)
        return self.gradInput

    def accGradParameters(self, input, gradOutput, scale=1.0):
        assert self.bestModuleInst is not None, "Must have been tuned in updateOutput already!"
        assert not self.inferenceOnly, "Inference only specified => no accGrads "
        self.bestModuleInst.gradWeight, self.bestModuleInst.gradBias = self.gradWeight, self.gradBias
        self.bestModuleInst.accGradParameters(input, gradOutput, scale)

    def cleanupBuffers(self):
        if self.bestModuleInst is not None:
            self.bestModuleInst.cleanupBuffers()
        self.bestModuleInst = None
