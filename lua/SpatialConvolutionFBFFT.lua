-- nn.SpatialConvolutionFBFFT on libfbfftconv.so: the three ...FFTImpl methods of
-- fbcunn/SpatialConvolutionFBFFT.lua:102-354 and backward() of
-- fbcunn/SpatialConvolutionFFT.lua:405-416, each one call into the C ABI.  The base class
-- nn.SpatialConvolutionFFT (constructor, reset, memoryReusePolicy, updateOutput /
-- updateGradInput / accGradParameters wrappers that allocate self.output and self.gradInput,
-- fbcunn/SpatialConvolutionFFT.lua:150-316, 430-629) is kept as it is.
-- Marshalling only.
require 'cunn'
local fbfc = require 'fbfftconv_ffi'
local C, check = fbfc.C, fbfc.check

local SpatialConvolutionFBFFT, parent =
   torch.class('nn.SpatialConvolutionFBFFT', 'nn.SpatialConvolutionFFT')

function SpatialConvolutionFBFFT:__init(nInputPlane, nOutputPlane, kW, kH, dW, dH,
                                        padLeft, padUp, memoryReusePolicy, numCudaStreams)
   assert(torch.type(nInputPlane) == 'number')
   assert(torch.type(nOutputPlane) == 'number')
   assert(torch.type(kW) == 'number')
   assert(torch.type(kH) == 'number')
   assert(torch.type(dW) == 'number')
   assert(torch.type(dH) == 'number')
   assert(memoryReusePolicy == nil or torch.type(memoryReusePolicy) == 'string' or
          torch.type(memoryReusePolicy) == 'table')
   parent.__init(self, nInputPlane, nOutputPlane, kW, kH, dW, dH, padLeft, padUp,
                 memoryReusePolicy, numCudaStreams)
   self.fftImplementation = 'fbfft'
   assert(self.dH == 1 and self.dW == 1, "fft only supports stride-1 convolutions atm")
   assert(self.padUp < self.kH and self.padLeft < self.kW, "Padding must be smaller than kernel")
end

-- tile sizes of the plan: none here, nn.SpatialConvolutionFFTTiled overrides
function SpatialConvolutionFBFFT:fbfcTile()
   return nil, nil
end

-- the frequency buffers belong to the plan: nothing to prepare on the Lua side
function SpatialConvolutionFBFFT:prepareSizeAndBuffers(input)
   return fbfc.plan(self, input, self:fbfcTile())
end

-- self.output was allocated by updateOutputFFT (fbcunn/SpatialConvolutionFFT.lua:435-441)
function SpatialConvolutionFBFFT:updateOutputFFTImpl(input, reuseList, metaData)
   assert(torch.type(input) == 'torch.CudaTensor', "CUDA support only!")
   assert(input:isContiguous() and self.output:isContiguous())
   local bias = self.bias:data()
   if metaData and metaData.skipBias then bias = nil end
   check(C.fbfc_update_output(self:prepareSizeAndBuffers(input), input:data(), self.weight:data(),
                              bias, self.output:data(), fbfc.stream()))
   return self.output
end

-- self.gradInput was allocated by updateGradInputFFT (fbcunn/SpatialConvolutionFFT.lua:501-507)
function SpatialConvolutionFBFFT:updateGradInputFFTImpl(input, gradOutput, reuseList, metaData)
   assert(torch.type(input) == 'torch.CudaTensor', "CUDA support only!")
   assert(gradOutput:isContiguous() and self.gradInput:isContiguous())
   check(C.fbfc_update_grad_input(self:prepareSizeAndBuffers(input), gradOutput:data(),
                                  self.weight:data(), self.gradInput:data(), fbfc.stream()))
   return self.gradInput
end

-- gradWeight and gradBias are assigned, as in the reference (accumulate = false,
-- fbcunn/SpatialConvolutionFBFFT.lua:337-349)
function SpatialConvolutionFBFFT:accGradParametersFFTImpl(input, gradOutput, scale, reuseList, metaData)
   assert(torch.type(input) == 'torch.CudaTensor', "CUDA support only!")
   assert(input:isContiguous() and gradOutput:isContiguous())
   local gradBias = self.gradBias:data()
   if metaData and metaData.skipBias then gradBias = nil end
   check(C.fbfc_acc_grad_parameters(self:prepareSizeAndBuffers(input), input:data(), gradOutput:data(),
                                    self.gradWeight:data(), gradBias, scale or 1, fbfc.stream()))
end

-- updateGradInput + accGradParameters sharing FFT(gradOutput)
function SpatialConvolutionFBFFT:backward(input, gradOutput, scale)
   assert(torch.type(input) == 'torch.CudaTensor', "CUDA support only!")
   if not self.gradInput or self.gradInput:nElement() == 0 then
      self.gradInput = torch.CudaTensor(input:size())
   end
   check(C.fbfc_backward(self:prepareSizeAndBuffers(input), input:data(), gradOutput:data(),
                         self.weight:data(), self.gradInput:data(), self.gradWeight:data(),
                         self.gradBias:data(), scale or 1, fbfc.stream()))
   return self.gradInput
end

function SpatialConvolutionFBFFT:cleanupBuffers()
   fbfc.cleanup(self)
   parent.cleanupBuffers(self)
end
