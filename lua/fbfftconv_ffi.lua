-- LuaJIT FFI declaration of libfbfftconv.so (include/fbfftconv.h, every symbol) and the three
-- helpers the module files share: error check, the stream of the current Torch state, plan cache.
-- Replaces the ffi.load of torch_fb_fbcunn_mm / torch_fb_fbcunn_convolution_bias
-- (fbcunn/SpatialConvolutionFBFFT.lua:7-13) and the cdefs of fbcunn/FFTCDefs.lua:3-34.
-- Marshalling only: no arithmetic and no policy lives on the Lua side.
local ffi = require 'ffi'

ffi.cdef[[
enum { FBFC_OK = 0, FBFC_ERR_INVALID_ARGUMENT = 1, FBFC_ERR_UNSUPPORTED_SIZE = 2,
       FBFC_ERR_UNSUPPORTED_DIMENSION = 3, FBFC_ERR_OUT_OF_MEMORY = 4, FBFC_ERR_HIP = 5 };
typedef struct { int batch, in_planes, out_planes, in_h, in_w, k_h, k_w,
                 stride_h, stride_w, pad_h, pad_w; } fbfc_conv_desc;
typedef struct { int fft_size, n_freq, out_h, out_w;
                 size_t input_freq_bytes, weight_freq_bytes, output_freq_bytes, scratch_bytes;
                 int tiles_h, tiles_w; size_t backward_freq_bytes; } fbfc_plan_info;
typedef struct fbfc_plan fbfc_plan;

const char *fbfc_version(void);
const char *fbfc_last_error(void);
const char *fbfc_last_launch(void);
int fbfc_plan_query(const fbfc_conv_desc *desc, fbfc_plan_info *info);
int fbfc_plan_create(const fbfc_conv_desc *desc, fbfc_plan **plan);
int fbfc_plan_destroy(fbfc_plan *plan);
int fbfc_plan_get_info(const fbfc_plan *plan, fbfc_plan_info *info);
int fbfc_plan_query_tiled(const fbfc_conv_desc *desc, int tile_h, int tile_w, fbfc_plan_info *info);
int fbfc_plan_create_tiled(const fbfc_conv_desc *desc, int tile_h, int tile_w, fbfc_plan **plan);
int fbfc_plan_create_tiled_iterated(const fbfc_conv_desc *desc, int tile_h, int tile_w, fbfc_plan **plan);
int fbfc_update_output(fbfc_plan *plan, const float *input, const float *weight, const float *bias,
                       float *output, void *stream);
int fbfc_update_grad_input(fbfc_plan *plan, const float *grad_output, const float *weight,
                           float *grad_input, void *stream);
int fbfc_acc_grad_parameters(fbfc_plan *plan, const float *input, const float *grad_output,
                             float *grad_weight, float *grad_bias, float scale, void *stream);
int fbfc_backward(fbfc_plan *plan, const float *input, const float *grad_output, const float *weight,
                  float *grad_input, float *grad_weight, float *grad_bias, float scale, void *stream);
int fbfc_plan_prepare_backward(fbfc_plan *plan);
enum { FBFC_REUSE_NONE = 0, FBFC_REUSE_INPUT = 1, FBFC_REUSE_OUTPUT = 2, FBFC_REUSE_WEIGHT = 4,
       FBFC_REUSE_ALL = 7 };
int fbfc_plan_set_reuse(fbfc_plan *plan, unsigned flags);
enum { FBFC_STAGE_FFT_A = 0, FBFC_STAGE_FFT_B = 1, FBFC_STAGE_MM = 2, FBFC_STAGE_IFFT = 3,
       FBFC_STAGE_BIAS_GRAD = 4, FBFC_NUM_STAGES = 5 };
int fbfc_plan_set_timed(fbfc_plan *plan, int reps);
int fbfc_plan_stage_ms(const fbfc_plan *plan, float *ms, int n);
int fbfc_plan_stage_kernel(const fbfc_plan *plan, int stage, char *name, size_t n);
int fbfc_debug_force_contraction_kernel(int variant);
int fbfc_debug_force_spectrum_streaming(int mode);
int fbfc_fft2d(const float *real, long planes, int h, int w, int pad_u, int pad_l, int fft_size,
               float *freq, void *stream);
int fbfc_ifft2d(const float *freq, long planes, int h, int w, int pad_u, int pad_l, int fft_size,
                float *real, const float *bias, int bias_period, void *stream);
size_t fbfc_planes_layout_workspace_bytes(long planes, int fft_size);
int fbfc_fft2d_planes(const float *real, long planes, int h, int w, int pad_u, int pad_l, int fft_size,
                      float *freq_planes, float *workspace, void *stream);
int fbfc_ifft2d_planes(const float *freq_planes, long planes, int h, int w, int pad_u, int pad_l,
                       int fft_size, float *real, float *workspace, void *stream);
int fbfc_fft1d(const float *real, long rows, int n, int pad_l, int fft_size, float *freq, void *stream);
int fbfc_ifft1d(const float *freq, long rows, int n, int pad_l, int fft_size, float *real, void *stream);
int fbfc_transpose_mm(const float *A, const float *B, float *C, int n_freq, int m, int n, int k,
                      float inv_norm, int conj_trans_a, int conj_trans_b, int accumulate, void *stream);
size_t fbfc_transpose_mm_planes_workspace_bytes(int n_freq, int m, int n, int k);
int fbfc_transpose_mm_planes(const float *A, const float *B, float *C, int n_freq, int m, int n, int k,
                             float inv_norm, int conj_trans_a, int conj_trans_b, int accumulate,
                             float *workspace, void *stream);
int fbfc_direct_update_output(const fbfc_conv_desc *desc, const float *input, const float *weight,
                              const float *bias, float *output, void *stream);
int fbfc_direct_update_grad_input(const fbfc_conv_desc *desc, const float *grad_output,
                                  const float *weight, float *grad_input, void *stream);
int fbfc_direct_acc_grad_parameters(const fbfc_conv_desc *desc, const float *input,
                                    const float *grad_output, float *grad_weight, float *grad_bias,
                                    float scale, float *scratch, void *stream);
int fbfc_update_output_bias(float *output, const float *bias, int batch, int planes, int h, int w,
                            void *stream);
int fbfc_update_output_bias_strided(float *output, const float *bias, int batch, int planes, int h, int w,
                                    long stride_b, long stride_f, long stride_h, long stride_w,
                                    long bias_stride, void *stream);
size_t fbfc_bias_grad_scratch_bytes(int batch, int planes);
int fbfc_acc_grad_parameters_bias(const float *grad_output, float *grad_bias, float scale, int batch,
                                  int planes, int h, int w, float *scratch, void *stream);
int fbfc_acc_grad_parameters_bias_strided(const float *grad_output, float *grad_bias, float scale,
                                          int batch, int planes, int h, int w, long stride_b,
                                          long stride_f, long stride_h, long stride_w,
                                          long bias_stride, float *scratch, void *stream);
int fbfc_acc_grad_parameters_bias_noalloc(const float *grad_output, float *grad_bias, float scale,
                                          int batch, int planes, int h, int w, void *stream);

/* from the HIP build of cutorch (libTHC): the stream the current Torch state launches on */
typedef struct THCState THCState;
void *THCState_getCurrentStream(THCState *state);
]]

local M = {}
M.C = ffi.load(package.searchpath('libfbfftconv', package.cpath) or 'fbfftconv')
local THC = ffi.load(package.searchpath('libTHC', package.cpath) or 'THC')

-- every entry point returns FBFC_OK or a code; the text is fbfc_last_error()
function M.check(rc)
   if rc ~= 0 then
      error('fbfftconv error ' .. tonumber(rc) .. ': ' .. ffi.string(M.C.fbfc_last_error()))
   end
end

-- The stream every launch of a pass goes to: the current stream of cutorch's THCState, i.e. what
-- cutorch.setStream() selected (the reference's native code asks the same question,
-- THCState_getCurrentStream(state): src/MM.cu:50, src/fft/FBFFTHost.cpp:162-166,
-- src/ConvolutionBias.cu:161-162).  cutorch._state is the THCState* the reference passes too
-- (fbcunn/SpatialConvolutionFBFFT.lua:157).
function M.stream()
   return THC.THCState_getCurrentStream(ffi.cast('THCState*', cutorch._state))
end

local reuseBits = {none = 0, input = 1, output = 2, weight = 4, all = 7}

-- One plan per (batch, iH, iW) of a module; replaces prepareSizeAndBuffers / getBuffer
-- (fbcunn/SpatialConvolutionFFT.lua:652-803).  tileH / tileW are nil for an untiled module.
function M.plan(module, input, tileH, tileW)
   module.fbfcPlans = module.fbfcPlans or {}
   local key = input:size(1) .. 'x' .. input:size(3) .. 'x' .. input:size(4)
   local plan = module.fbfcPlans[key]
   if not plan then
      local d = ffi.new('fbfc_conv_desc', {input:size(1), module.nInputPlane, module.nOutputPlane,
                                          input:size(3), input:size(4), module.kH, module.kW,
                                          module.dH, module.dW, module.padUp, module.padLeft})
      local p = ffi.new('fbfc_plan*[1]')
      if tileH and tileW and module.fbfcIterated then
         M.check(M.C.fbfc_plan_create_tiled_iterated(d, tileH, tileW, p))
      elseif tileH and tileW then
         M.check(M.C.fbfc_plan_create_tiled(d, tileH, tileW, p))
      else
         M.check(M.C.fbfc_plan_create(d, p))
      end
      plan = ffi.gc(p[0], M.C.fbfc_plan_destroy)
      local flags = 0
      for i = 1, #module.memoryReusePolicy do
         flags = bit.bor(flags, reuseBits[module.memoryReusePolicy[i]])
      end
      if flags ~= 0 then M.check(M.C.fbfc_plan_set_reuse(plan, flags)) end
      module.fbfcPlans[key] = plan
   end
   return plan
end

function M.cleanup(module)
   for _, plan in pairs(module.fbfcPlans or {}) do
      M.C.fbfc_plan_destroy(ffi.gc(plan, nil))
   end
   module.fbfcPlans = {}
end

return M
