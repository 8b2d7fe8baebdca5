// Window copies of the tiled convolution, shared by the three-kernel tiled passes (fft_kernels.hip) and
// the fused ones (fused_kernels.hip).
#pragma once
#include <hip/hip_runtime.h>

#include "fft_stage.h"
#include "kernels.h"

namespace fbfc {

// Moves the windows of planes [first, first + nph) of the workgroup between global memory and their
// nph * h canvas rows.  Each wave takes every fourth plane, so the window corner and the plane's base
// address are wave-uniform; its lanes sweep the window 64 elements (N <= 32: at least two rows) at a
// time with all loads of a plane in flight together.  pstride: floats between the canvases of two planes.
// The row pass reads a canvas row with 16-byte LDS accesses, 16 lanes (16 planes, same row) per cycle: they
// cover the 64 banks when pstride / 4 is odd, which h * LDR / 4 is for odd h only; window_plane_stride adds
// the four floats that make it so for even h (a window is as high as the tile: 16 x 16 windows had every
// plane's row on the same banks).
template <int N>
__device__ __host__ __forceinline__ constexpr int window_plane_stride(int h)
{
    return h * Canvas<N>::LDR + ((h & 1) ? 0 : 4);
}

template <int N, bool TO_LDS>
__device__ __forceinline__ void copy_windows(float *smem, float *g, const int4 *tbl, int first, int nph,
                                             int h, int w, int padL, const Window &win, int tid, int pstride)
{
    constexpr int LDR = Canvas<N>::LDR;
    constexpr int ITER = (N * N) / 64;
    const int wave = tid >> 6, lane = tid & 63;
    const int c = lane % N, r0 = lane / N;
    for (int tl = wave; tl < nph; tl += 4) {
        const int4 q = tbl[first + tl];
        const int off_lo = __builtin_amdgcn_readfirstlane(q.x), off_hi = __builtin_amdgcn_readfirstlane(q.y);
        const int y0 = __builtin_amdgcn_readfirstlane(q.z), x0 = __builtin_amdgcn_readfirstlane(q.w);
        float *gp = g + ((((long)off_hi) << 32) | (long)(unsigned)off_lo) + x0 + c;
        float *sp = smem + tl * pstride + padL + c;
        const bool xok = (c < w) && ((unsigned)(x0 + c) < (unsigned)win.img_w);
        float v[ITER];
        if (TO_LDS) {
#pragma unroll
            for (int i = 0; i < ITER; ++i) {
                const int r = r0 + i * (64 / N);
                const int y = y0 + r;
                const bool ok = xok && (r < h) && ((unsigned)y < (unsigned)win.img_h);
                v[i] = ok ? gp[(long)y * win.img_w] : 0.0f;
            }
#pragma unroll
            for (int i = 0; i < ITER; ++i) {
                const int r = r0 + i * (64 / N);
                if (r < h) sp[r * LDR] = v[i];
            }
        } else {
#pragma unroll
            for (int i = 0; i < ITER; ++i) {
                const int r = r0 + i * (64 / N);
                v[i] = (r < h) ? sp[r * LDR] : 0.0f;
            }
#pragma unroll
            for (int i = 0; i < ITER; ++i) {
                const int r = r0 + i * (64 / N);
                const int y = y0 + r;
                if (xok && (r < h) && ((unsigned)y < (unsigned)win.img_h)) gp[(long)y * win.img_w] = v[i];
            }
        }
    }
}

}  // namespace fbfc
