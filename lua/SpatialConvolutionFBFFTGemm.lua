-- nn.SpatialConvolutionFBFFTGemm on libfbfftconv.so.  The reference's class differs from
-- nn.SpatialConvolutionFBFFT only in how the per-frequency contraction is done: explicit
-- transposes to frequency-major plus cublasCgemmBatched (fbcunn/SpatialConvolutionFBFFTGemm.lua:92-454,
-- src/CuBLASWrapper.cpp:113-125, 437-452).  The library's spectra are frequency-major to begin
-- with and its contraction is one MFMA kernel, so both classes run the same three entry points;
-- this file keeps the class name, constructor and fields.
require 'cunn'

local SpatialConvolutionFBFFTGemm, parent =
   torch.class('nn.SpatialConvolutionFBFFTGemm', 'nn.SpatialConvolutionFBFFT')

function SpatialConvolutionFBFFTGemm:__init(nInputPlane, nOutputPlane, kW, kH, dW, dH,
                                            padLeft, padUp, memoryReusePolicy, numCudaStreams)
   parent.__init(self, nInputPlane, nOutputPlane, kW, kH, dW, dH, padLeft, padUp,
                 memoryReusePolicy, numCudaStreams)
end
