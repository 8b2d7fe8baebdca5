-- nn.SpatialConvolutionDirect on libfbfftconv.so: the spatial-domain convolution that stands where
-- the reference's tuning front and fallback use cudnn.SpatialConvolution
-- (fbcunn/SpatialConvolution.lua:259-269, fbcunn/SpatialConvolutionFFT.lua:323-393); fbnn.SpatialConvolution
-- keeps its Lua tuning loop and times this class next to the FFT ones.  Any stride.  Marshalling only.
require 'cunn'
local ffi = require 'ffi'
local fbfc = require 'fbfftconv_ffi'
local C, check = fbfc.C, fbfc.check

local SpatialConvolutionDirect, parent = torch.class('nn.SpatialConvolutionDirect', 'nn.Module')

function SpatialConvolutionDirect:__init(nInputPlane, nOutputPlane, kW, kH, dW, dH, padW, padH)
   parent.__init(self)
   self.nInputPlane, self.nOutputPlane = nInputPlane, nOutputPlane
   self.kW, self.kH, self.dW, self.dH = kW, kH, dW or 1, dH or 1
   self.padW, self.padH = padW or 0, padH or 0
   self.weight = torch.CudaTensor(nOutputPlane, nInputPlane, kH, kW)
   self.bias = torch.CudaTensor(nOutputPlane)
   self.gradWeight = torch.CudaTensor(nOutputPlane, nInputPlane, kH, kW):zero()
   self.gradBias = torch.CudaTensor(nOutputPlane):zero()
   local stdv = 1 / math.sqrt(kW * kH * nInputPlane)
   self.weight:uniform(-stdv, stdv)
   self.bias:uniform(-stdv, stdv)
end

local function desc(self, input)
   return ffi.new('fbfc_conv_desc', {input:size(1), self.nInputPlane, self.nOutputPlane, input:size(3),
                                     input:size(4), self.kH, self.kW, self.dH, self.dW, self.padH, self.padW})
end

function SpatialConvolutionDirect:updateOutput(input)
   local oH = math.floor((input:size(3) + 2 * self.padH - self.kH) / self.dH) + 1
   local oW = math.floor((input:size(4) + 2 * self.padW - self.kW) / self.dW) + 1
   self.output = self.output or torch.CudaTensor()
   self.output:resize(input:size(1), self.nOutputPlane, oH, oW)
   check(C.fbfc_direct_update_output(desc(self, input), input:data(), self.weight:data(), self.bias:data(),
                                     self.output:data(), fbfc.stream()))
   return self.output
end

function SpatialConvolutionDirect:updateGradInput(input, gradOutput)
   self.gradInput = self.gradInput or torch.CudaTensor()
   self.gradInput:resizeAs(input)
   check(C.fbfc_direct_update_grad_input(desc(self, input), gradOutput:data(), self.weight:data(),
                                         self.gradInput:data(), fbfc.stream()))
   return self.gradInput
end

-- gradWeight and gradBias are assigned
function SpatialConvolutionDirect:accGradParameters(input, gradOutput, scale)
   local bytes = tonumber(C.fbfc_bias_grad_scratch_bytes(input:size(1), self.nOutputPlane))
   self.scratch = self.scratch or torch.CudaTensor()
   self.scratch:resize(math.ceil(bytes / 4))
   check(C.fbfc_direct_acc_grad_parameters(desc(self, input), input:data(), gradOutput:data(),
                                           self.gradWeight:data(), self.gradBias:data(), scale or 1,
                                           self.scratch:data(), fbfc.stream()))
end
