// Bias kernels (gfx950).
//
// bias_add_kernel replaces updateOutputBias (src/ConvolutionBias.cu:39-51) for
// callers that want the stand-alone form; the convolution itself adds the bias
// in the inverse-FFT epilogue instead.
// bias_grad_* replace accGradParametersBias (src/ConvolutionBias.cu:61-97):
// gradBias[f] = scale * sum_{b,r,c} gradOutput[b][f][r][c], ASSIGNED.  The
// reference uses one block per plane; here the batch is split over several
// workgroups per plane (enough to fill 256 CUs) and a second tiny kernel adds
// the partial sums in a fixed order, so the result is deterministic.
#include <hip/hip_runtime.h>

#include "bias_dc.h"
#include "kernels.h"

namespace fbfc {

constexpr int kMaxSplit = 16;

__global__ __launch_bounds__(256) void bias_add_kernel(float *__restrict__ out,
                                                       const float *__restrict__ bias, int planes,
                                                       int hw)
{
    const long plane = blockIdx.x;
    const float b = bias[plane % planes];
    float *o = out + plane * hw;
    for (int i = threadIdx.x; i < hw; i += 256) o[i] += b;
}

__device__ __forceinline__ float wave_sum(float v)
{
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) v += __shfl_down(v, off, 64);
    return v;
}

// grid (planes, split): workgroup (f, s) sums batches s, s+split, ... of plane f
__global__ __launch_bounds__(256) void bias_grad_partial_kernel(const float *__restrict__ g,
                                                                float *__restrict__ partial,
                                                                int batch, int planes, int hw,
                                                                int split)
{
    __shared__ float wsum[4];
    const int f = blockIdx.x, s = blockIdx.y;
    float acc = 0.0f;
    for (int b = s; b < batch; b += split) {
        const float *p = g + ((long)b * planes + f) * hw;
        for (int i = threadIdx.x; i < hw; i += 256) acc += p[i];
    }
    acc = wave_sum(acc);
    if ((threadIdx.x & 63) == 0) wsum[threadIdx.x >> 6] = acc;
    __syncthreads();
    if (threadIdx.x == 0) partial[f * split + s] = (wsum[0] + wsum[1]) + (wsum[2] + wsum[3]);
}

__global__ __launch_bounds__(256) void bias_grad_final_kernel(const float *__restrict__ partial,
                                                              float *__restrict__ grad_bias,
                                                              float scale, int planes, int split)
{
    const int f = blockIdx.x * 256 + threadIdx.x;
    if (f >= planes) return;
    float acc = 0.0f;
    for (int s = 0; s < split; ++s) acc += partial[f * split + s];
    grad_bias[f] = acc * scale;
}

// Stand-alone launch of the zero-frequency-row bias gradient (see bias_dc.h); the
// accGradParameters pass normally runs the same body inside its inverse-FFT launch.
__global__ __launch_bounds__(256) void bias_grad_dc_kernel(BiasGradJob job)
{
    __shared__ float part[4][64];
    bias_grad_dc_body(job, blockIdx.x, part);
}

hipError_t launch_bias_grad_dc(const float *freq, float *grad_bias, float scale, int batch, int planes,
                               hipStream_t s)
{
    BiasGradJob job = {reinterpret_cast<const float2 *>(freq), grad_bias, scale, batch, planes};
    FBFC_LAUNCH(bias_grad_dc_kernel, dim3(bias_grad_dc_blocks(planes)), dim3(256), 0, s, job);
    return hipGetLastError();
}

static int split_for(int batch) { return batch < kMaxSplit ? batch : kMaxSplit; }

size_t bias_grad_scratch_bytes(int batch, int planes)
{
    return (size_t)planes * split_for(batch) * sizeof(float);
}

hipError_t launch_bias_add(float *out, const float *bias, int batch, int planes, int hw,
                           hipStream_t s)
{
    FBFC_LAUNCH(bias_add_kernel, dim3((unsigned)((long)batch * planes)), dim3(256), 0, s, out,
                       bias, planes, hw);
    return hipGetLastError();
}

hipError_t launch_bias_grad(const float *grad_out, float *grad_bias, float scale, int batch,
                            int planes, int hw, float *scratch, hipStream_t s)
{
    const int split = split_for(batch);
    FBFC_LAUNCH(bias_grad_partial_kernel, dim3(planes, split), dim3(256), 0, s, grad_out,
                       scratch, batch, planes, hw, split);
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return e;
    FBFC_LAUNCH(bias_grad_final_kernel, dim3((planes + 255) / 256), dim3(256), 0, s, scratch,
                       grad_bias, scale, planes, split);
    return hipGetLastError();
}

// ---------------------------------------------------------------------------------
// Strided forms (the reference's bias kernels take non-contiguous tensors,
// src/ConvolutionBias.cu:39-97; test/BiasTest.cpp:38-63): element (b, f, r, c) of the
// feature-map tensor sits at b * sb + f * sf + r * sh + c * sw floats, bias[f] at f * bias_stride.
// ---------------------------------------------------------------------------------
struct Strides4 {
    long b, f, h, w;
};

__global__ __launch_bounds__(256) void bias_add_strided_kernel(float *__restrict__ out,
                                                               const float *__restrict__ bias, int planes,
                                                               int h, int w, Strides4 st, long bias_stride)
{
    const long plane = blockIdx.x;
    const long b = plane / planes, f = plane - b * planes;
    const float bv = bias[f * bias_stride];
    float *o = out + b * st.b + f * st.f;
    const int hw = h * w;
    for (int i = threadIdx.x; i < hw; i += 256) {
        const int r = i / w, c = i - r * w;
        o[r * st.h + c * st.w] += bv;
    }
}

__global__ __launch_bounds__(256) void bias_grad_partial_strided_kernel(const float *__restrict__ g,
                                                                        float *__restrict__ partial,
                                                                        int batch, int h, int w, Strides4 st,
                                                                        int split)
{
    __shared__ float wsum[4];
    const int f = blockIdx.x, s = blockIdx.y;
    const int hw = h * w;
    float acc = 0.0f;
    for (int b = s; b < batch; b += split) {
        const float *p = g + (long)b * st.b + (long)f * st.f;
        for (int i = threadIdx.x; i < hw; i += 256) {
            const int r = i / w, c = i - r * w;
            acc += p[r * st.h + c * st.w];
        }
    }
    acc = wave_sum(acc);
    if ((threadIdx.x & 63) == 0) wsum[threadIdx.x >> 6] = acc;
    __syncthreads();
    if (threadIdx.x == 0) partial[f * split + s] = (wsum[0] + wsum[1]) + (wsum[2] + wsum[3]);
}

__global__ __launch_bounds__(256) void bias_grad_final_strided_kernel(const float *__restrict__ partial,
                                                                      float *__restrict__ grad_bias,
                                                                      float scale, int planes, int split,
                                                                      long bias_stride)
{
    const int f = blockIdx.x * 256 + threadIdx.x;
    if (f >= planes) return;
    float acc = 0.0f;
    for (int s = 0; s < split; ++s) acc += partial[f * split + s];
    grad_bias[f * bias_stride] = acc * scale;
}

hipError_t launch_bias_add_strided(float *out, const float *bias, int batch, int planes, int h, int w,
                                   long sb, long sf, long sh, long sw, long bias_stride, hipStream_t s)
{
    const Strides4 st = {sb, sf, sh, sw};
    FBFC_LAUNCH(bias_add_strided_kernel, dim3((unsigned)((long)batch * planes)), dim3(256), 0, s, out,
                       bias, planes, h, w, st, bias_stride);
    return hipGetLastError();
}

hipError_t launch_bias_grad_strided(const float *grad_out, float *grad_bias, float scale, int batch,
                                    int planes, int h, int w, long sb, long sf, long sh, long sw,
                                    long bias_stride, float *scratch, hipStream_t s)
{
    const Strides4 st = {sb, sf, sh, sw};
    const int split = split_for(batch);
    FBFC_LAUNCH(bias_grad_partial_strided_kernel, dim3(planes, split), dim3(256), 0, s, grad_out,
                       scratch, batch, h, w, st, split);
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return e;
    FBFC_LAUNCH(bias_grad_final_strided_kernel, dim3((planes + 255) / 256), dim3(256), 0, s, scratch,
                       grad_bias, scale, planes, split, bias_stride);
    return hipGetLastError();
}

}  // namespace fbfc
