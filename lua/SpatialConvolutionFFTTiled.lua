-- nn.SpatialConvolutionFFTTiled and its Sync / Async / Iterated instantiations on libfbfftconv.so
-- (fbcunn/SpatialConvolutionFFTTiled.lua:260-330 constructor; the per-tile loops of :445-777 and of
-- SpatialConvolutionFFTTiledSync/Async/Iterated.lua happen inside the library: one launch per
-- stage covers all tiles).  Only the plan differs from the untiled module; the Iterated class asks for
-- the plan whose passes are fused kernels (fbfc_plan_create_tiled_iterated) and, like the reference's
-- (fbcunn/SpatialConvolutionFFTTiledIterated.lua:47-48), takes no memory reuse policy.
require 'cunn'

local SpatialConvolutionFFTTiled, parent =
   torch.class('nn.SpatialConvolutionFFTTiled', 'nn.SpatialConvolutionFBFFT')

function SpatialConvolutionFFTTiled:__init(nInputPlane, nOutputPlane, kW, kH, dW, dH,
                                           padLeft, padUp, tileSizeW, tileSizeH,
                                           memoryReusePolicy, numCudaStreams)
   assert(tileSizeW == nil or torch.type(tileSizeW) == 'number')
   assert(tileSizeH == nil or torch.type(tileSizeH) == 'number')
   parent.__init(self, nInputPlane, nOutputPlane, kW, kH, dW, dH, padLeft, padUp,
                 memoryReusePolicy, numCudaStreams)
   self.tileSizeH = tileSizeH or 16
   self.tileSizeW = tileSizeW or 16
end

function SpatialConvolutionFFTTiled:fbfcTile()
   return self.tileSizeH, self.tileSizeW
end

for _, name in ipairs({'Sync', 'Async', 'Iterated'}) do
   local cls, tiledParent = torch.class('nn.SpatialConvolutionFFTTiled' .. name,
                                        'nn.SpatialConvolutionFFTTiled')
   cls.__init = function(self, ...)
      tiledParent.__init(self, ...)
      if name == 'Iterated' then
         self.fbfcIterated = true
         self.memoryReusePolicy = {'none'}
      end
   end
end
