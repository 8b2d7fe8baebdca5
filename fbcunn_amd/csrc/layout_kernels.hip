// Conversions between the library's frequency-major spectra, freq[q][plane], and the plane-major
// buffers the reference's stand-alone wrappers hand around, buf[plane][q]:
//   * nn.FFTWrapper with fbfft: (planes, N/2+1, N, 2), the FIRST transform dimension halved; for
//     8 <= N <= 32 buf[a][c] = X[ky = a][kx = c], for N < 8 or N > 32 buf[a][c] = X[ky = c][kx = a]
//     (test/test_FFTModule.lua:238-241, 267-269 and the layout fbcunn/SpatialConvolutionFFT.lua:710-721
//     allocates);
//   * transposeMMFFI: (d0, d1, n_freq, 2) operands (src/MM.cu:54-73), any frequency order.
// The library keeps X[ky][kx], ky in [0,N), kx in [0,N/2]; where the reference's half plane needs
// a kx above N/2 the value is the conjugate of X[N - ky][N - kx].  Both directions go through a
// 32 x 32 LDS tile, so that reads and writes are contiguous on both sides.
#include <hip/hip_runtime.h>

#include "kernels.h"

namespace fbfc {

// layout modes: 0 = same frequency order on both sides; 1 = buf[a][c] = X[c][a];
// 2 = buf[a][c] = X[a][c] with a <= N/2 (the other half plane)
struct RefEntry {
    int q;      // index into the library's spectrum, ky * (N/2+1) + kx
    int conj;
};

// where entry (a, c) of the reference buffer comes from
__device__ __forceinline__ RefEntry ref_source(int mode, int N, int qref)
{
    const int nh = N / 2 + 1;
    if (mode == 0) return RefEntry{qref, 0};
    const int a = qref / N, c = qref - a * N;
    if (mode == 1) return RefEntry{c * nh + a, 0};
    if (c <= N / 2) return RefEntry{a * nh + c, 0};
    return RefEntry{((N - a) % N) * nh + (N - c), 1};
}

__global__ __launch_bounds__(256) void freq_to_planes_kernel(const float2 *__restrict__ freq,
                                                             float2 *__restrict__ buf, long planes, int nq,
                                                             int N, int mode)
{
    __shared__ float2 tile[32][33];
    const int tx = threadIdx.x & 31, ty = threadIdx.x >> 5;
    const int q0 = blockIdx.x * 32;
    // the grid's second dimension holds at most 65535 workgroups: each walks the plane tiles with that stride
    const long ptiles = (planes + 31) / 32;
    for (long pt = blockIdx.y; pt < ptiles; pt += gridDim.y) {
        const long p0 = pt * 32;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int ql = ty + 8 * i;   // entry of the reference buffer handled by this row of the tile
            if (q0 + ql < nq && p0 + tx < planes) {
                const RefEntry e = ref_source(mode, N, q0 + ql);
                float2 v = freq[(long)e.q * planes + p0 + tx];
                if (e.conj) v.y = -v.y;
                tile[ql][tx] = v;
            }
        }
        __syncthreads();
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int pl = ty + 8 * i;
            if (p0 + pl < planes && q0 + tx < nq) buf[(p0 + pl) * nq + q0 + tx] = tile[tx][pl];
        }
        __syncthreads();  // the tile is free for the next round
    }
}

// The other direction: every entry (ky, kx <= N/2) of the library's spectrum is written.  An entry
// (a, c) of the reference buffer feeds (a, c) itself when c <= N/2 (mode 2) and, as a conjugate, the
// row N - a above N/2 at column (N - c) mod N when that column is <= N/2.
__global__ __launch_bounds__(256) void planes_to_freq_kernel(const float2 *__restrict__ buf,
                                                             float2 *__restrict__ freq, long planes, int nq,
                                                             int N, int mode)
{
    __shared__ float2 tile[32][33];
    const int tx = threadIdx.x & 31, ty = threadIdx.x >> 5;
    const int q0 = blockIdx.x * 32;
    const int nh = N / 2 + 1;
    const long ptiles = (planes + 31) / 32;
    for (long pt = blockIdx.y; pt < ptiles; pt += gridDim.y) {
        const long p0 = pt * 32;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int pl = ty + 8 * i;
            if (p0 + pl < planes && q0 + tx < nq) tile[tx][pl] = buf[(p0 + pl) * nq + q0 + tx];
        }
        __syncthreads();
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int ql = ty + 8 * i;
            const int qref = q0 + ql;
            if (qref >= nq || p0 + tx >= planes) continue;
            const float2 v = tile[ql][tx];
            if (mode != 2) {
                freq[(long)ref_source(mode, N, qref).q * planes + p0 + tx] = v;
            } else {
                const int a = qref / N, c = qref - a * N;
                if (c <= N / 2) freq[(long)(a * nh + c) * planes + p0 + tx] = v;
                const int a2 = N - a, c2 = (N - c) % N;
                if (a > 0 && a2 > N / 2 && c2 <= N / 2)
                    freq[(long)(a2 * nh + c2) * planes + p0 + tx] = make_float2(v.x, -v.y);
            }
        }
        __syncthreads();  // the tile is free for the next round
    }
}

static bool layout_args_ok(long planes, int nq) { return planes > 0 && nq > 0; }
static unsigned plane_grid(long planes)
{
    const long ptiles = (planes + 31) / 32;
    return (unsigned)(ptiles < 65535 ? ptiles : 65535);
}

hipError_t launch_freq_to_planes(const float *freq, float *buf, long planes, int nq, int N, int mode,
                                 hipStream_t s)
{
    if (!layout_args_ok(planes, nq)) return hipErrorInvalidValue;
    kernel_log_add("freq_to_planes_kernel", (long)((nq + 31) / 32) * plane_grid(planes) * 256);
    FBFC_LAUNCH(freq_to_planes_kernel, dim3((nq + 31) / 32, plane_grid(planes)), dim3(256), 0, s,
                       reinterpret_cast<const float2 *>(freq), reinterpret_cast<float2 *>(buf), planes, nq, N, mode);
    return hipGetLastError();
}

hipError_t launch_planes_to_freq(const float *buf, float *freq, long planes, int nq, int N, int mode,
                                 hipStream_t s)
{
    if (!layout_args_ok(planes, nq)) return hipErrorInvalidValue;
    kernel_log_add("planes_to_freq_kernel", (long)((nq + 31) / 32) * plane_grid(planes) * 256);
    FBFC_LAUNCH(planes_to_freq_kernel, dim3((nq + 31) / 32, plane_grid(planes)), dim3(256), 0, s,
                       reinterpret_cast<const float2 *>(buf), reinterpret_cast<float2 *>(freq), planes, nq, N, mode);
    return hipGetLastError();
}

}  // namespace fbfc
