// Bias gradient from the spectrum of gradOutput.
//
// The zero-frequency bin of plane (b, f) is sum_{r,c} gradOutput[b][f][r][c], so
// gradBias[f] = scale * sum_b Re dc[b][f] with dc the first frequency row of the
// frequency-major spectrum (batch x planes complex numbers).  The first 256 lanes of a workgroup
// handle 64 planes x 4 batch slices; `part` is 4 x 64 floats of LDS.
#pragma once
#include <hip/hip_runtime.h>

namespace fbfc {

struct BiasGradJob {
    const float2 *dc;   // first frequency row of FFT(gradOutput); nullptr = no job
    float *grad_bias;
    float scale;
    int batch, planes;
};

__device__ __forceinline__ void bias_grad_dc_body(const BiasGradJob &j, unsigned block, float (*part)[64])
{
    const int fl = threadIdx.x & 63, slice = threadIdx.x >> 6;
    const int f = (int)block * 64 + fl;
    float acc = 0.0f;
    if (f < j.planes && slice < 4) {
        // eight loads in flight per lane: a tiled plan sums over batch * tiles planes
        float a[8] = {0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f};
        int b = slice;
        for (; b + 28 < j.batch; b += 32) {
#pragma unroll
            for (int u = 0; u < 8; ++u) a[u] += j.dc[(long)(b + 4 * u) * j.planes + f].x;
        }
        for (; b < j.batch; b += 4) a[0] += j.dc[(long)b * j.planes + f].x;
        acc = ((a[0] + a[1]) + (a[2] + a[3])) + ((a[4] + a[5]) + (a[6] + a[7]));
    }
    if (slice < 4) part[slice][fl] = acc;
    __syncthreads();
    if (slice == 0 && f < j.planes)
        j.grad_bias[f] = ((part[0][fl] + part[1][fl]) + (part[2][fl] + part[3][fl])) * j.scale;
}

inline unsigned bias_grad_dc_blocks(int planes) { return (unsigned)((planes + 63) / 64); }

}  // namespace fbfc
