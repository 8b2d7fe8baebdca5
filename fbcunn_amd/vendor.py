"""The platform library's convolution (MIOpen, reached through torch's aten::convolution) behind the
module protocol of this package.

It stands where cudnn.SpatialConvolution stands in the reference: an optional candidate of the tuning
front (fbcunn/SpatialConvolution.lua:259-269) and the figure the FFT path is measured against in
bench.py.  Nothing in libfbfftconv.so or in the FFT modules calls it; it is off unless asked for.
accGradParameters assigns gradWeight and gradBias (scaled), like the other modules here.
"""
import math

import torch

__all__ = ["SpatialConvolutionMIOpen"]


class SpatialConvolutionMIOpen:
    def __init__(self, nInputPlane, nOutputPlane, kW, kH, dW=1, dH=1, padW=0, padH=0, device="cuda", init=True):
        self.nInputPlane, self.nOutputPlane = nInputPlane, nOutputPlane
        self.kW, self.kH, self.dW, self.dH, self.padW, self.padH = kW, kH, dW, dH, padW, padH
        self.device = torch.device(device)
        self.weight = torch.empty(nOutputPlane, nInputPlane, kH, kW, device=self.device)
        self.bias = torch.empty(nOutputPlane, device=self.device)
        self.gradWeight = torch.zeros(nOutputPlane, nInputPlane, kH, kW, device=self.device)
        self.gradBias = torch.zeros(nOutputPlane, device=self.device)
        self.output = None
        self.gradInput = None
        if init:
            stdv = 1.0 / math.sqrt(kW * kH * nInputPlane)
            self.weight.uniform_(-stdv, stdv)
            self.bias.uniform_(-stdv, stdv)

    def _check(self, input, gradOutput=None):
        if not isinstance(input, torch.Tensor) or not input.is_cuda:
            raise TypeError("input: CUDA support only!")
        if input.dtype != torch.float32 or input.dim() != 4 or input.size(1) != self.nInputPlane:
            raise ValueError("input must be float32 (batch, %d, h, w)" % self.nInputPlane)
        if gradOutput is not None:
            shape = (input.size(0), self.nOutputPlane, (input.size(2) + 2 * self.padH - self.kH) // self.dH + 1,
                     (input.size(3) + 2 * self.padW - self.kW) // self.dW + 1)
            if tuple(gradOutput.shape) != shape:
                raise ValueError("gradOutput has the wrong shape")

    def _backward(self, input, gradOutput, mask):
        return torch.ops.aten.convolution_backward(gradOutput, input, self.weight, [self.nOutputPlane],
                                                   [self.dH, self.dW], [self.padH, self.padW], [1, 1], False, [0, 0], 1,
                                                   mask)

    def updateOutput(self, input):
        self._check(input)
        self.output = torch.ops.aten.convolution(input, self.weight, self.bias, [self.dH, self.dW],
                                                 [self.padH, self.padW], [1, 1], False, [0, 0], 1)
        return self.output

    forward = updateOutput

    def updateGradInput(self, input, gradOutput):
        self._check(input, gradOutput)
        self.gradInput = self._backward(input, gradOutput, [True, False, False])[0]
        return self.gradInput

    def accGradParameters(self, input, gradOutput, scale=1.0):
        self._check(input, gradOutput)
        _, gw, gb = self._backward(input, gradOutput, [False, True, True])
        torch.mul(gw, scale, out=self.gradWeight)
        torch.mul(gb, scale, out=self.gradBias)

    def backward(self, input, gradOutput, scale=1.0):
        self._check(input, gradOutput)
        gi, gw, gb = self._backward(input, gradOutput, [True, True, True])
        self.gradInput = gi
        torch.mul(gw, scale, out=self.gradWeight)
        torch.mul(gb, scale, out=self.gradBias)
        return self.gradInput

    def cleanupBuffers(self):
        self.output = None
        self.gradInput = None
