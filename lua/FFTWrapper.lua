-- nn.FFTWrapper with the fbfft implementation on libfbfftconv.so (fbcunn/FFTWrapper.lua:53-132;
-- the luaT functions FFTWrapper_fft / FFTWrapper_ffti of src/fft/FFTWrapperLua.cpp:209-299).
-- time: (batch dims..., n) or (batch dims..., h, w) real; frequency: the reference's layout,
-- (rows, N/2+1, 2) for one transform dimension and (planes..., N/2+1, N, 2) for two (the first
-- transform dimension halved; for N < 8 or N > 32 the two frequency axes are swapped, exactly as
-- fbfft leaves them, test/test_FFTModule.lua:238-241, 267-269).  The 2-D calls go through
-- fbfc_fft2d_planes / fbfc_ifft2d_planes with a workspace tensor, the counterpart of the buffer
-- argument the reference passes for sizes above 32 (fbcunn/FFTWrapper.lua:73-79, 114-122).
-- ffti is unnormalised.  Marshalling only.
require 'cunn'
local ffi = require 'ffi'
local fbfc = require 'fbfftconv_ffi'
local C, check = fbfc.C, fbfc.check

local FFTWrapper = torch.class('nn.FFTWrapper')

function FFTWrapper:__init(cufft, padLeft, padUp, timed)
   assert(cufft == 'fbfft' or cufft == false, 'only the fbfft implementation exists in this build')
   self.cufft = false
   self.timed = (timed == 'timed')
   self.padLeft = padLeft or 0
   self.padUp = padUp or 0
   self.batchDims = 0
end

local function geometry(time, frequency, batchDims)
   assert(torch.type(time) == 'torch.CudaTensor', 'FBFFT only with CudaTensors')
   assert(batchDims >= 1 and batchDims <= 2)
   assert(time:isContiguous() and frequency:isContiguous())
   local fftDims = time:nDimension() - batchDims
   assert(fftDims == 1 or fftDims == 2)
   local planes = 1
   for i = 1, batchDims do planes = planes * time:size(i) end
   return fftDims, planes
end

local function workspace(self, planes, n)
   local floats = math.ceil(tonumber(C.fbfc_planes_layout_workspace_bytes(planes, n)) / 4)
   if not self.buffer or self.buffer:nElement() < floats then
      self.buffer = torch.CudaTensor(floats)
   end
   return self.buffer
end

function FFTWrapper:fft(time, frequency, batchDims)
   local fftDims, planes = geometry(time, frequency, batchDims)
   self.batchDims = batchDims
   if fftDims == 1 then
      local n = (frequency:size(batchDims + 1) - 1) * 2
      check(C.fbfc_fft1d(time:data(), planes, time:size(batchDims + 1), self.padLeft, n,
                         frequency:data(), fbfc.stream()))
   else
      local n = frequency:size(batchDims + 2)
      check(C.fbfc_fft2d_planes(time:data(), planes, time:size(batchDims + 1), time:size(batchDims + 2),
                                self.padUp, self.padLeft, n, frequency:data(),
                                workspace(self, planes, n):data(), fbfc.stream()))
   end
   return frequency
end

function FFTWrapper:ffti(time, frequency, batchDims)
   local fftDims, planes = geometry(time, frequency, batchDims)
   self.batchDims = batchDims
   if fftDims == 1 then
      local n = (frequency:size(batchDims + 1) - 1) * 2
      check(C.fbfc_ifft1d(frequency:data(), planes, time:size(batchDims + 1), self.padLeft, n,
                          time:data(), fbfc.stream()))
   else
      local n = frequency:size(batchDims + 2)
      check(C.fbfc_ifft2d_planes(frequency:data(), planes, time:size(batchDims + 1), time:size(batchDims + 2),
                                 self.padUp, self.padLeft, n, time:data(),
                                 workspace(self, planes, n):data(), fbfc.stream()))
   end
   return time
end
