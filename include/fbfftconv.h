/*
 * fbfftconv — C ABI of the MI355X (gfx950) FFT-convolution library.
 *
 * This is the boundary a host binding loads (LuaJIT ffi.load, ctypes, dlopen).
 * Every entry point takes plain device pointers, sizes and an opaque
 * hipStream_t (passed as void*); there are no torch/THC types.  Every entry
 * point returns FBFC_OK or an error code and never throws; the message for the
 * last error on the calling thread is fbfc_last_error().
 *
 * A plan is used by one host thread at a time; different plans and the
 * stand-alone entry points may be called from different host threads at once,
 * each with its own stream.
 *
 * Tensors are contiguous fp32, NCHW.  "planes" of a 4-D tensor (d0,d1,h,w) means
 * the d0*d1 flattened leading dimensions.
 *
 * Frequency-domain buffers are FREQUENCY-MAJOR, complex interleaved:
 *     freq[(ky * (N/2+1) + kx) * planes + plane] = (re, im)
 * with ky in [0,N) the row frequency, kx in [0,N/2] the (Hermitian-halved)
 * column frequency.  For a fixed frequency the planes form a dense row-major
 * (d0 x d1) complex matrix, which is what the per-frequency contraction reads.
 */
#ifndef FBFFTCONV_H
#define FBFFTCONV_H

#include <stddef.h>

#ifdef __cplusplus
extern "C" {
#endif

/* Error codes.  UNSUPPORTED_SIZE / UNSUPPORTED_DIMENSION mirror
 * FBFFTParameters::ErrorCode as used in src/fft/FBFFTHost.cpp:96-98,115,168. */
enum {
    FBFC_OK = 0,
    FBFC_ERR_INVALID_ARGUMENT = 1,
    FBFC_ERR_UNSUPPORTED_SIZE = 2,
    FBFC_ERR_UNSUPPORTED_DIMENSION = 3,
    FBFC_ERR_OUT_OF_MEMORY = 4,
    FBFC_ERR_HIP = 5
};

/* Constructor arguments of nn.SpatialConvolutionFBFFT
 * (fbcunn/SpatialConvolutionFBFFT.lua:26-96, fbcunn/SpatialConvolutionFFT.lua:150-177)
 * plus the batch and input size the reference only learns at the first call. */
typedef struct {
    int batch;      /* B */
    int in_planes;  /* nInputPlane  P */
    int out_planes; /* nOutputPlane F */
    int in_h, in_w; /* H, W */
    int k_h, k_w;   /* kH, kW */
    int stride_h, stride_w; /* dH, dW: must be 1 */
    int pad_h, pad_w;       /* padUp (= padDown), padLeft (= padRight): must be < kernel */
} fbfc_conv_desc;

/* What the reference derives in prepareFBFFTSizeAndBuffers
 * (fbcunn/SpatialConvolutionFFT.lua:947-964) and getBuffer (:692-803). */
typedef struct {
    int fft_size;        /* N: smallest 2^i >= max(H+2padH, W+2padW, kH, kW, oH, oW), i >= 1 */
    int n_freq;          /* Q = N * (N/2+1) */
    int out_h, out_w;    /* H + 2 padH - kH + 1, W + 2 padW - kW + 1 */
    size_t input_freq_bytes;   /* Q * B * P * 8 */
    size_t weight_freq_bytes;  /* Q * F * P * 8 */
    size_t output_freq_bytes;  /* Q * B * F * 8 */
    size_t scratch_bytes;      /* what fbfc_acc_grad_parameters_bias needs for this shape */
    int tiles_h, tiles_w;      /* output tiles per image (1 x 1 for an untiled plan) */
    size_t backward_freq_bytes; /* what fbfc_plan_prepare_backward adds: input_freq_bytes +
                                   weight_freq_bytes for an untiled plan, 0 for a tiled one */
} fbfc_plan_info;

typedef struct fbfc_plan fbfc_plan;

/* Library ------------------------------------------------------------------ */
const char *fbfc_version(void);
/* Message of the last failure on this thread ("" if none). */
const char *fbfc_last_error(void);

/* What the last stand-alone transform or contraction called from this thread launched:
 * "<kernel name> grid=<work-items>", several launches joined by "; ".  (For the passes of a plan see
 * fbfc_plan_stage_kernel.)  Counterpart of the log line of the reference's timed wrappers
 * (src/fft/FFTWrapperLua.cpp:137-152). */
const char *fbfc_last_launch(void);

/* Planning (host only; no GPU needed) ----------------------------------------
 * Validates the descriptor the way the module constructor and the FFT-size
 * choice do (stride 1: SpatialConvolutionFFT.lua:176, SpatialConvolutionFBFFT.lua:60-61;
 * pad < kernel: SpatialConvolutionFBFFT.lua:93-95; nextPowerOf2: SpatialConvolutionFFT.lua:875-882)
 * and fills *info.  FFT sizes above 128 are FBFC_ERR_UNSUPPORTED_SIZE (the reference's
 * fbfft stops at 128 as well); sizes below 8 run on an 8 x 8 canvas.  A tensor of more than
 * floor((2^31 - 1) / ((N/2 + 1) * 8)) planes (batch x planes, or output x input planes; 8.1 million
 * at N = 64) is FBFC_ERR_UNSUPPORTED_SIZE too, with the count in the message: one launch addresses
 * a frequency row of the spectrum with 32-bit offsets. */
int fbfc_plan_query(const fbfc_conv_desc *desc, fbfc_plan_info *info);

/* Plans -----------------------------------------------------------------------
 * A plan owns the three frequency-domain buffers of one layer shape (the
 * reference's inputBuffer / weightBuffer / outputBuffer,
 * SpatialConvolutionFFT.lua:652-688) on the current device.  Caller tensors are
 * never kept or freed.  Passes on one plan must not overlap in time. */
int fbfc_plan_create(const fbfc_conv_desc *desc, fbfc_plan **plan);
int fbfc_plan_destroy(fbfc_plan *plan);
int fbfc_plan_get_info(const fbfc_plan *plan, fbfc_plan_info *info);

/* Tiled plans: nn.SpatialConvolutionFFTTiled and its Sync / Async / Iterated instantiations
 * (fbcunn/SpatialConvolutionFFTTiled.lua:260-330 constructor, :445-560, :618-672, :745-777 tilings).
 * The image is cut into windows of tile_h x tile_w (the reference's tileSizeH / tileSizeW, default
 * 16) that are tile - kernel + 1 apart; each window is transformed with an FFT of the next power
 * of two (8, 16 or 32), so images far larger than one FFT are convolved with small transforms.
 * Results equal those of an untiled plan.  The passes are the same three entry points below; a
 * tiled plan's buffers hold batch * tiles planes.  Errors follow the reference: tile smaller than
 * the kernel ("Tiling cannot be smaller than kernel !"), tile larger than the output ("Tile size
 * too large ..."); tiles above 32 are FBFC_ERR_UNSUPPORTED_SIZE.  With a reuse policy set, the
 * spectrum of gradOutput is never reused (updateGradInput and accGradParameters window it
 * differently). */
int fbfc_plan_query_tiled(const fbfc_conv_desc *desc, int tile_h, int tile_w, fbfc_plan_info *info);
int fbfc_plan_create_tiled(const fbfc_conv_desc *desc, int tile_h, int tile_w, fbfc_plan **plan);

/* nn.SpatialConvolutionFFTTiledIterated (fbcunn/SpatialConvolutionFFTTiledIterated.lua:79-123,
 * 129-175, 180-229 -> convolveIteratedFFI, src/fft/FFTIteratedConvolution.cu:71-95): a tiled plan whose
 * passes each run as ONE fused kernel (window transforms, product over the contracted planes, inverse
 * transform) after the small transform of the weights, so that no spectrum of a feature map is written
 * to memory.  Same tiling rules, errors and results as fbfc_plan_create_tiled (rounding differs in the
 * last bits: the sums over planes run in another order); the same three pass entry points.  The plan
 * owns the weight spectrum only: fbfc_plan_get_info reports input_freq_bytes = output_freq_bytes = 0
 * and, in scratch_bytes, the partial-result buffer of accGradParameters.  The sum over the contracted
 * planes is vector arithmetic, not a matrix-core contraction: the kernel is meant for layers in which
 * one side has few planes (first and last layers), where the spectra dominate the traffic of the
 * three-kernel pass.  Like the reference's module it takes no reuse policy (fbfc_plan_set_reuse is
 * accepted and has no effect).  fbfc_backward runs its two passes one after the other. */
int fbfc_plan_create_tiled_iterated(const fbfc_conv_desc *desc, int tile_h, int tile_w, fbfc_plan **plan);

/* Replaces SpatialConvolutionFBFFT:updateOutputFFTImpl
 * (fbcunn/SpatialConvolutionFBFFT.lua:102-183):
 * output(B,F,oH,oW) = valid cross-correlation of zero-padded input(B,P,H,W) with
 * weight(F,P,kH,kW), plus bias(F) (bias may be NULL = the reference's skipBias). */
int fbfc_update_output(fbfc_plan *plan, const float *input, const float *weight,
                       const float *bias, float *output, void *stream);

/* Replaces SpatialConvolutionFBFFT:updateGradInputFFTImpl (:189-263):
 * grad_input(B,P,H,W) = full convolution of grad_output(B,F,oH,oW) with weight,
 * cropped to the un-padded input window. */
int fbfc_update_grad_input(fbfc_plan *plan, const float *grad_output, const float *weight,
                           float *grad_input, void *stream);

/* Replaces SpatialConvolutionFBFFT:accGradParametersFFTImpl (:269-354):
 * grad_weight(F,P,kH,kW) = scale * sum_b input(b,p) cross-correlated with
 * grad_output(b,f); grad_bias(F) = scale * sum grad_output.  Both are ASSIGNED
 * (the reference passes accumulate=false and its bias kernel assigns,
 * src/ConvolutionBias.cu:95).  grad_bias may be NULL (skipBias). */
int fbfc_acc_grad_parameters(fbfc_plan *plan, const float *input, const float *grad_output,
                             float *grad_weight, float *grad_bias, float scale, void *stream);

/* Replaces SpatialConvolutionFFT:backward (fbcunn/SpatialConvolutionFFT.lua:405-416):
 * updateGradInput followed by accGradParameters, the second reusing the spectrum of
 * gradOutput the first one computed (the reference passes its outputTransposeBuffer in the
 * reuse list) whatever the plan's reuse policy.  Tiled plans recompute it (their two passes
 * window gradOutput differently).  Results equal those of the two separate calls, bit for bit.
 * For an untiled plan on which fbfc_plan_prepare_backward has succeeded each stage of the two
 * passes is issued as one grid (the forward transforms of gradOutput, weight and input; both
 * contractions; both inverse transforms with the bias gradient); otherwise the pass runs as its
 * two halves.  Like every pass it allocates nothing. */
int fbfc_backward(fbfc_plan *plan, const float *input, const float *grad_output, const float *weight,
                  float *grad_input, float *grad_weight, float *grad_bias, float scale, void *stream);

/* Gives an untiled plan the two buffers the one-grid-per-stage form of fbfc_backward writes its
 * product spectra to (it reads all three operand spectra in one launch, so neither result may
 * overwrite one of them): backward_freq_bytes more device memory on the plan's device, kept until the
 * plan is destroyed.  Call it once, outside any stream capture.  FBFC_ERR_OUT_OF_MEMORY if there is
 * no room (fbfc_backward then keeps running as its two halves); a no-op for tiled plans and for a
 * plan that is prepared already.  No counterpart in the reference, whose modules allocate inside
 * their passes (fbcunn/SpatialConvolutionFFT.lua:652-688). */
int fbfc_plan_prepare_backward(fbfc_plan *plan);

/* Memory-reuse policy of the module (SpatialConvolutionFFT.lua:59-63,216-240;
 * used at SpatialConvolutionFBFFT.lua:226-230,305-322): with a flag set, the
 * pass that would recompute that spectrum reuses the one the previous pass left
 * in the plan's buffer.  Default 0 = memoryReuseNone (every pass recomputes). */
enum { FBFC_REUSE_NONE = 0, FBFC_REUSE_INPUT = 1, FBFC_REUSE_OUTPUT = 2, FBFC_REUSE_WEIGHT = 4,
       FBFC_REUSE_ALL = 7 };
int fbfc_plan_set_reuse(fbfc_plan *plan, unsigned flags);

/* Per-stage timing, the counterpart of the `timed` flag of nn.FFTWrapper /
 * nn.CuBLASWrapper (src/fft/FFTWrapperLua.cpp:82-177): with reps > 0 each pass issues
 * every launch of its schedule reps times back to back between two HIP events recorded
 * on the pass's stream (stages are pure functions of their inputs, so results are
 * unchanged) and synchronises at the end; fbfc_plan_stage_ms then reports the mean time
 * of one launch.  The launches are those of an untimed pass.  reps = 0 switches timing
 * off.  reps < 0: the pass runs exactly as an untimed one, every launch once, and each launch is
 * timed by the start and end of its own dispatch on the device (what a profiler's kernel trace
 * reports as the kernel's duration: no launch gap, no event overhead); a stage reports the sum
 * over its launches.  This is the duration of the kernel inside an ordinary pass, with its
 * operands wherever the previous kernel left them.  Stage slots: */
enum { FBFC_STAGE_FFT_A = 0,   /* the forward-FFT launch: both operands of the pass, or the
                                  first one alone when the second is reused */
       FBFC_STAGE_FFT_B = 1,   /* the second operand alone (when the first is reused) */
       FBFC_STAGE_MM = 2,      /* per-frequency contraction      */
       FBFC_STAGE_IFFT = 3,    /* inverse FFT (+ bias, + bias gradient in accGradParameters) */
       FBFC_STAGE_BIAS_GRAD = 4,  /* kept for layout; the bias gradient rides on the IFFT launch */
       FBFC_NUM_STAGES = 5 };
int fbfc_plan_set_timed(fbfc_plan *plan, int reps);
/* Milliseconds of each stage of the last timed pass (0 for a stage not run). */
int fbfc_plan_stage_ms(const fbfc_plan *plan, float *ms, int n);
/* What a stage of the plan's last pass launched, as a profiler trace shows it:
 * "<kernel name> grid=<work-items>", several launches joined by "; " ("" for a stage not run).  The
 * library picks its kernels by shape; this is the counterpart of the names the reference's timed
 * wrappers log (src/CuBLASWrapperLua.cpp:39-137, src/fft/FFTWrapperLua.cpp:137-152). */
int fbfc_plan_stage_kernel(const fbfc_plan *plan, int stage, char *name, size_t n);
/* Measurement knob (no counterpart in the reference): forces the contraction kernel variant for the
 * whole process.  -1 = choose by shape (default); 0 = register-staged LDS tiles with bounds checks,
 * 8 = LDS-direct tiles, 9 = LDS-direct tiles plus split blocks, 1 / 2 / 4 = register-fed kernel
 * with that many waves per block.  A variant that cannot run a shape falls back to the shape rule. */
int fbfc_debug_force_contraction_kernel(int variant);
/* Measurement knob (no counterpart in the reference): how the forward transforms store their spectra,
 * for the whole process.  -1 = by size (default): a spectrum of up to 144 MB is written through to the
 * memory side, whose cache keeps it for the contraction, a larger one is streamed past the caches with
 * non-temporal stores; 1 = always non-temporal (where the kernel writes whole 128-byte lines).  Alone a
 * transform is about as fast either way; the pass that follows is not.  Results do not depend on it. */
int fbfc_debug_force_spectrum_streaming(int mode);
/* Stand-alone stages ------------------------------------------------------------
 * Replaces FFTWrapper_fft with fbfft (src/fft/FFTWrapperLua.cpp:209-272 ->
 * fbfft2dHost, src/fft/FBFFTHost.cpp:39-116): batched 2-D real-to-complex FFT of
 * `planes` h x w planes, each implicitly zero-padded into an N x N canvas at
 * row pad_u, column pad_l.  N in {2,4,8,16,32,64,128} (the sizes the reference tests,
 * test/test_FFTModule.lua:170-260).  Output is frequency-major (fbfc_fft2d_planes gives the
 * reference's plane-major buffer). */
int fbfc_fft2d(const float *real, long planes, int h, int w, int pad_u, int pad_l,
               int fft_size, float *freq, void *stream);

/* Replaces FFTWrapper_ffti (same files): UNNORMALISED complex-to-real inverse;
 * writes real[plane][r][s] = y[r+pad_u][s+pad_l] for r<h, s<w of the N x N result.
 * If bias != NULL, bias[plane % bias_period] is added to every element of the
 * plane (the fused form of updateOutputBiasFFI, src/ConvolutionBias.cu:39-51).
 * As in any complex-to-real transform the input is taken to be the spectrum of a real
 * plane: the entries (ky > N/2, kx in {0, N/2}) are not read but taken as the
 * conjugates of (N - ky, kx) (sizes 8 to 128; sizes 2 and 4 read every entry).  Every entry that
 * is read is used as given: where the buffer deviates from the spectrum of a real plane (say by
 * imaginary parts in the four self-conjugate entries, ky and kx in {0, N/2}) the deviation passes
 * linearly into the result, it is not filtered out. */
int fbfc_ifft2d(const float *freq, long planes, int h, int w, int pad_u, int pad_l,
                int fft_size, float *real, const float *bias, int bias_period, void *stream);

/* The same two transforms on the reference's own buffer layout, for callers at the nn.FFTWrapper
 * level (fbcunn/FFTWrapper.lua:53-132, test/test_FFTModule.lua:238-342): freq_planes is
 * (planes, N/2+1, N, 2), plane-major, the first of the two frequency axes halved.  As fbfft leaves
 * it, buf[a][c] = X[ky = a][kx = c] for 8 <= N <= 32 and buf[a][c] = X[ky = c][kx = a] for N < 8 or
 * N > 32 (test/test_FFTModule.lua:238-241).  workspace: fbfc_planes_layout_workspace_bytes(planes, N)
 * bytes of device memory, the counterpart of the buffer tensor the reference passes for sizes above
 * 32 (fbcunn/FFTWrapper.lua:73-79, 114-122); the transform runs frequency-major in it and one more
 * kernel converts the layout.  The inverse is unnormalised and, like fbfc_ifft2d, takes its input
 * to be the spectrum of a real plane: of the half plane given, the entries the frequency-major
 * spectrum holds twice over -- (ky > N/2, kx in {0, N/2}), which repeat (N - ky, kx) as conjugates --
 * are not used, so the result equals the reference's exactly when the buffer is Hermitian (as every
 * spectrum or product of spectra of real planes is, up to rounding). */
size_t fbfc_planes_layout_workspace_bytes(long planes, int fft_size);
int fbfc_fft2d_planes(const float *real, long planes, int h, int w, int pad_u, int pad_l,
                      int fft_size, float *freq_planes, float *workspace, void *stream);
int fbfc_ifft2d_planes(const float *freq_planes, long planes, int h, int w, int pad_u, int pad_l,
                       int fft_size, float *real, float *workspace, void *stream);

/* Replaces FFTWrapper_fft / FFTWrapper_ffti on tensors with ONE transform dimension
 * (fbfft1dHost, src/fft/FBFFTHost.cpp:119-131): `rows` real sequences of n values, each
 * zero-padded into fft_size points at pad_l, <-> freq (rows, fft_size/2+1, 2), row-major as in
 * the reference.  fft_size in {2,4,...,128}; the inverse is unnormalised and writes
 * real[row][i] = y[i + pad_l], i < n. */
int fbfc_fft1d(const float *real, long rows, int n, int pad_l, int fft_size, float *freq, void *stream);
int fbfc_ifft1d(const float *freq, long rows, int n, int pad_l, int fft_size, float *real, void *stream);

/* Replaces transposeMMFFI (src/MM.cu:54-73): for each of n_freq frequencies,
 *   C (m x n) (=|+=) inv_norm * op(A) * op(B),   op = conjugate transpose if flagged.
 * A is (m x k), or (k x m) when conj_trans_a; B is (k x n), or (n x k) when
 * conj_trans_b; all dense row-major complex, frequency-major
 * (X[freq][row][col][2]).  Both flags set is not supported (the reference does
 * not instantiate it either, src/MM.cu:34-39). */
int fbfc_transpose_mm(const float *A, const float *B, float *C, int n_freq,
                      int m, int n, int k, float inv_norm,
                      int conj_trans_a, int conj_trans_b, int accumulate, void *stream);

/* transposeMMFFI on the reference's operand layout (src/MM.cu:14-24, 54-73): A, B, C are
 * (rows, cols, n_freq, 2), plane-major, as the (d0, d1, N/2+1, N, 2) buffers of
 * fbcunn/SpatialConvolutionFFT.lua:710-721 are with their two frequency axes flattened.  Same
 * arithmetic as fbfc_transpose_mm; the operands are brought to frequency-major order in `workspace`
 * (fbfc_transpose_mm_planes_workspace_bytes bytes) and C is written back plane-major. */
size_t fbfc_transpose_mm_planes_workspace_bytes(int n_freq, int m, int n, int k);
int fbfc_transpose_mm_planes(const float *A, const float *B, float *C, int n_freq,
                             int m, int n, int k, float inv_norm, int conj_trans_a, int conj_trans_b,
                             int accumulate, float *workspace, void *stream);

/* Direct (spatial-domain) convolution: the three passes for ANY stride and padding, without a plan.
 * The role cudnn.SpatialConvolution plays for the reference's FFT path: the non-FFT candidate of the
 * tuning front (fbcunn/SpatialConvolution.lua:259-269), the path a layer falls back to when the FFT
 * modules cannot run it (fbcunn/SpatialConvolutionFFT.lua:323-393) and the result the self-check
 * compares with (:91-133, :387-399).  Plain kernels, correct for every shape, not tuned.  Output size
 * (in + 2 pad - k) / stride + 1; bias / grad_bias may be NULL; grad_weight and grad_bias are
 * assigned; scratch: fbfc_bias_grad_scratch_bytes(batch, out_planes) bytes, needed with grad_bias. */
int fbfc_direct_update_output(const fbfc_conv_desc *desc, const float *input, const float *weight,
                              const float *bias, float *output, void *stream);
int fbfc_direct_update_grad_input(const fbfc_conv_desc *desc, const float *grad_output,
                                  const float *weight, float *grad_input, void *stream);
int fbfc_direct_acc_grad_parameters(const fbfc_conv_desc *desc, const float *input,
                                    const float *grad_output, float *grad_weight, float *grad_bias,
                                    float scale, float *scratch, void *stream);

/* Replaces updateOutputBiasFFI (src/ConvolutionBias.cu:256-260): output[b][f][.][.] += bias[f]. */
int fbfc_update_output_bias(float *output, const float *bias, int batch, int planes,
                            int h, int w, void *stream);

/* The same on a non-contiguous feature-map tensor, which the reference's bias kernels accept
 * (src/ConvolutionBias.cu:39-51 takes strided DeviceTensors; test/BiasTest.cpp:38-63 transposes two
 * dimensions): element (b, f, r, c) lies at b*stride_b + f*stride_f + r*stride_h + c*stride_w floats
 * from `output`, bias[f] at f*bias_stride floats from `bias`. */
int fbfc_update_output_bias_strided(float *output, const float *bias, int batch, int planes,
                                    int h, int w, long stride_b, long stride_f, long stride_h,
                                    long stride_w, long bias_stride, void *stream);

/* Replaces accGradParametersBiasFFI (src/ConvolutionBias.cu:262-274):
 * grad_bias[f] = scale * sum_{b,r,c} grad_output[b][f][r][c] (assignment).
 * scratch must hold fbfc_bias_grad_scratch_bytes(batch, planes) bytes. */
size_t fbfc_bias_grad_scratch_bytes(int batch, int planes);
int fbfc_acc_grad_parameters_bias(const float *grad_output, float *grad_bias, float scale,
                                  int batch, int planes, int h, int w,
                                  float *scratch, void *stream);
/* The same on a non-contiguous grad_output (src/ConvolutionBias.cu:61-97; test/BiasTest.cpp:186-222);
 * strides in floats as for fbfc_update_output_bias_strided; scratch as above (dense). */
int fbfc_acc_grad_parameters_bias_strided(const float *grad_output, float *grad_bias, float scale,
                                          int batch, int planes, int h, int w, long stride_b,
                                          long stride_f, long stride_h, long stride_w,
                                          long bias_stride, float *scratch, void *stream);

/* fbfc_acc_grad_parameters_bias without the workspace argument, for callers that cannot allocate
 * device memory (code under HIP graph capture, tight serving loops, harnesses that forbid
 * hipMalloc).  It has no counterpart in the reference.  The partial sums live in a fixed 256 KB
 * array in device memory that every GPU the library runs on holds until the process ends; the call
 * allocates and frees nothing.  At most 4096 planes (FBFC_ERR_UNSUPPORTED_SIZE beyond, with the
 * limit in the message).  Results equal those of fbfc_acc_grad_parameters_bias bit for bit.  The
 * first call on a device looks the array's address up (a module query, not an allocation): make it
 * outside stream capture, or create any plan on that device first, which does the same lookup.  All
 * calls on one GPU share the array: calls that overlap in time on one GPU (two streams, two
 * threads) race and must be serialised by the caller. */
int fbfc_acc_grad_parameters_bias_noalloc(const float *grad_output, float *grad_bias, float scale,
                                          int batch, int planes, int h, int w, void *stream);

#ifdef __cplusplus
}
#endif
#endif /* FBFFTCONV_H */
