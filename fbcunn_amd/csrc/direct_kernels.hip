// Direct (spatial-domain) convolution for gfx950: the non-FFT candidate of the tuning front and the
// path a layer the FFT modules cannot run falls back to (strides above 1, sizes beyond the largest
// transform).  The reference uses cudnn.SpatialConvolution in both roles
// (fbcunn/SpatialConvolution.lua:259-269, fbcunn/SpatialConvolutionFFT.lua:323-393).  Plain kernels,
// one lane per result element, fp32 accumulation in the loop order of the reference's CPU
// convolutions (test/ReferenceConvolutions.cpp:86-200, 338-450, 452-554): they are there to be right
// for every shape, not to compete with the FFT path where that one runs.
#include <hip/hip_runtime.h>

#include "kernels.h"

namespace fbfc {

struct DirectGeom {
    int B, P, F, H, W, kH, kW, sH, sW, padH, padW, oH, oW;
};

__global__ __launch_bounds__(256) void direct_fprop_kernel(const float *__restrict__ in,
                                                           const float *__restrict__ w,
                                                           const float *__restrict__ bias,
                                                           float *__restrict__ out, DirectGeom g)
{
    const long total = (long)g.B * g.F * g.oH * g.oW;
    for (long i = (long)blockIdx.x * 256 + threadIdx.x; i < total; i += (long)gridDim.x * 256) {
        const int x = (int)(i % g.oW), y = (int)((i / g.oW) % g.oH);
        const int f = (int)((i / ((long)g.oW * g.oH)) % g.F), b = (int)(i / ((long)g.oW * g.oH * g.F));
        float acc = 0.0f;
        for (int p = 0; p < g.P; ++p) {
            const float *ip = in + ((long)b * g.P + p) * g.H * g.W;
            const float *wp = w + ((long)f * g.P + p) * g.kH * g.kW;
            for (int ky = 0; ky < g.kH; ++ky) {
                const int iy = y * g.sH - g.padH + ky;
                if (iy < 0 || iy >= g.H) continue;
                for (int kx = 0; kx < g.kW; ++kx) {
                    const int ix = x * g.sW - g.padW + kx;
                    if (ix < 0 || ix >= g.W) continue;
                    acc += ip[iy * g.W + ix] * wp[ky * g.kW + kx];
                }
            }
        }
        out[i] = acc + (bias != nullptr ? bias[f] : 0.0f);
    }
}

__global__ __launch_bounds__(256) void direct_bprop_kernel(const float *__restrict__ go,
                                                           const float *__restrict__ w,
                                                           float *__restrict__ gi, DirectGeom g)
{
    const long total = (long)g.B * g.P * g.H * g.W;
    for (long i = (long)blockIdx.x * 256 + threadIdx.x; i < total; i += (long)gridDim.x * 256) {
        const int ix = (int)(i % g.W), iy = (int)((i / g.W) % g.H);
        const int p = (int)((i / ((long)g.W * g.H)) % g.P), b = (int)(i / ((long)g.W * g.H * g.P));
        float acc = 0.0f;
        for (int f = 0; f < g.F; ++f) {
            const float *gp = go + ((long)b * g.F + f) * g.oH * g.oW;
            const float *wp = w + ((long)f * g.P + p) * g.kH * g.kW;
            for (int ky = 0; ky < g.kH; ++ky) {
                const int ty = iy + g.padH - ky;
                if (ty < 0 || ty % g.sH != 0) continue;
                const int y = ty / g.sH;
                if (y >= g.oH) continue;
                for (int kx = 0; kx < g.kW; ++kx) {
                    const int tx = ix + g.padW - kx;
                    if (tx < 0 || tx % g.sW != 0) continue;
                    const int x = tx / g.sW;
                    if (x >= g.oW) continue;
                    acc += gp[y * g.oW + x] * wp[ky * g.kW + kx];
                }
            }
        }
        gi[i] = acc;
    }
}

// one workgroup per weight element (f, p, ky, kx): its lanes share the sum over batch and output pixels
__global__ __launch_bounds__(256) void direct_accgrad_kernel(const float *__restrict__ in,
                                                             const float *__restrict__ go,
                                                             float *__restrict__ gw, float scale, DirectGeom g)
{
    __shared__ float part[256];
    const long e = blockIdx.x;
    const int kx = (int)(e % g.kW), ky = (int)((e / g.kW) % g.kH);
    const int p = (int)((e / ((long)g.kW * g.kH)) % g.P), f = (int)(e / ((long)g.kW * g.kH * g.P));
    const int opix = g.oH * g.oW;
    float acc = 0.0f;
    for (long j = threadIdx.x; j < (long)g.B * opix; j += 256) {
        const int b = (int)(j / opix), r = (int)(j % opix);
        const int y = r / g.oW, x = r % g.oW;
        const int iy = y * g.sH - g.padH + ky, ix = x * g.sW - g.padW + kx;
        if (iy < 0 || iy >= g.H || ix < 0 || ix >= g.W) continue;
        acc += go[((long)b * g.F + f) * opix + r] * in[(((long)b * g.P + p) * g.H + iy) * g.W + ix];
    }
    part[threadIdx.x] = acc;
    __syncthreads();
    for (int s = 128; s > 0; s >>= 1) {
        if (threadIdx.x < s) part[threadIdx.x] += part[threadIdx.x + s];
        __syncthreads();
    }
    if (threadIdx.x == 0) gw[e] = part[0] * scale;
}

static unsigned grid_for(long total)
{
    long blocks = (total + 255) / 256;
    if (blocks > 65536) blocks = 65536;
    return (unsigned)(blocks < 1 ? 1 : blocks);
}

static DirectGeom geom(const int *d)
{
    DirectGeom g;
    g.B = d[0]; g.P = d[1]; g.F = d[2]; g.H = d[3]; g.W = d[4]; g.kH = d[5]; g.kW = d[6];
    g.sH = d[7]; g.sW = d[8]; g.padH = d[9]; g.padW = d[10];
    g.oH = (g.H + 2 * g.padH - g.kH) / g.sH + 1;
    g.oW = (g.W + 2 * g.padW - g.kW) / g.sW + 1;
    return g;
}

hipError_t launch_direct_fprop(const int *desc, const float *in, const float *w, const float *bias, float *out,
                               hipStream_t s)
{
    const DirectGeom g = geom(desc);
    const long total = (long)g.B * g.F * g.oH * g.oW;
    kernel_log_add("direct_fprop_kernel", (long)grid_for(total) * 256);
    FBFC_LAUNCH(direct_fprop_kernel, dim3(grid_for(total)), dim3(256), 0, s, in, w, bias, out, g);
    return hipGetLastError();
}

hipError_t launch_direct_bprop(const int *desc, const float *go, const float *w, float *gi, hipStream_t s)
{
    const DirectGeom g = geom(desc);
    const long total = (long)g.B * g.P * g.H * g.W;
    kernel_log_add("direct_bprop_kernel", (long)grid_for(total) * 256);
    FBFC_LAUNCH(direct_bprop_kernel, dim3(grid_for(total)), dim3(256), 0, s, go, w, gi, g);
    return hipGetLastError();
}

hipError_t launch_direct_accgrad(const int *desc, const float *in, const float *go, float *gw, float scale,
                                 hipStream_t s)
{
    const DirectGeom g = geom(desc);
    const long total = (long)g.F * g.P * g.kH * g.kW;
    if (total > 0x7fffffffL) return hipErrorInvalidValue;
    kernel_log_add("direct_accgrad_kernel", total * 256);
    FBFC_LAUNCH(direct_accgrad_kernel, dim3((unsigned)total), dim3(256), 0, s, in, go, gw, scale, g);
    return hipGetLastError();
}

}  // namespace fbfc
