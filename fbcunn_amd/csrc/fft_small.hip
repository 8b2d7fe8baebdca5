// The transforms outside the convolution path that nn.FFTWrapper also offers with fbfft
// (fbcunn/FFTWrapper.lua:53-132 -> src/fft/FBFFTHost.cpp:39-175): batched 1-D real<->complex FFTs
// of sizes 2..128 (fbfft1dHost) and the 2-D sizes 2 and 4, which are below what the tiled 2-D
// kernels are built for.  These are simple kernels: a lane holds its whole problem in registers
// (two rows of a 1-D batch, packed as one complex sequence; one whole plane of a tiny 2-D batch)
// and talks to global memory directly.
#include <hip/hip_runtime.h>

#include "fft_regs.h"
#include "kernels.h"

namespace fbfc {

// ---------------------------------------------------------------------------------
// 1-D forward: rows of n reals, zero-padded into N at pad_l -> (rows, N/2+1) complex
// ---------------------------------------------------------------------------------
template <int N>
__global__ __launch_bounds__(256, (N >= 128) ? 1 : 2) void rfft1d_kernel(const float *__restrict__ in,
                                                                       float2 *__restrict__ out, long rows,
                                                                       int n, int pad_l)
{
    const long pair = (long)blockIdx.x * 256 + threadIdx.x;
    const long ra = 2 * pair, rb = ra + 1;
    if (ra >= rows) return;
    const bool has_b = rb < rows;
    float re[N], im[N];
    const float *pa = in + ra * n - pad_l;
    const float *pb = in + rb * n - pad_l;
    static_for<N>([&](auto ii) {
        constexpr int i = decltype(ii)::value;
        const bool ok = (i >= pad_l) && (i < pad_l + n);
        re[i] = ok ? pa[i] : 0.0f;
        im[i] = (ok && has_b) ? pb[i] : 0.0f;
    });
    fft_inplace<N, false>(re, im);
    float2 *oa = out + ra * (N / 2 + 1);
    float2 *ob = out + rb * (N / 2 + 1);
    // z = a + i b with a, b real: A[k] = (Z[k] + conj Z[N-k]) / 2, B[k] = -i (Z[k] - conj Z[N-k]) / 2
    static_for<N / 2 + 1>([&](auto kk) {
        constexpr int k = decltype(kk)::value;
        constexpr int kn = (N - k) % N;
        const float zr = re[brev<N>(k)], zi = im[brev<N>(k)];
        const float nr = re[brev<N>(kn)], ni = im[brev<N>(kn)];
        oa[k] = make_float2(0.5f * (zr + nr), 0.5f * (zi - ni));
        if (has_b) ob[k] = make_float2(0.5f * (zi + ni), 0.5f * (nr - zr));
    });
}

// 1-D inverse, unnormalised: (rows, N/2+1) complex -> rows of n reals read at pad_l of the N results
template <int N>
__global__ __launch_bounds__(256, (N >= 128) ? 1 : 2) void irfft1d_kernel(const float2 *__restrict__ in,
                                                                        float *__restrict__ out, long rows,
                                                                        int n, int pad_l)
{
    const long pair = (long)blockIdx.x * 256 + threadIdx.x;
    const long ra = 2 * pair, rb = ra + 1;
    if (ra >= rows) return;
    const bool has_b = rb < rows;
    float re[N], im[N];
    const float2 *ia = in + ra * (N / 2 + 1);
    const float2 *ib = in + rb * (N / 2 + 1);
    // Z[k] = A[k] + i B[k]; for k > N/2 the spectra of real rows continue as conjugates
    static_for<N / 2 + 1>([&](auto kk) {
        constexpr int k = decltype(kk)::value;
        const float2 a = ia[k];
        const float2 b = has_b ? ib[k] : make_float2(0.0f, 0.0f);
        if constexpr (k == 0 || 2 * k == N) {  // real-valued bins of a real row
            re[k] = a.x;
            im[k] = b.x;
        } else {
            re[k] = a.x - b.y;
            im[k] = a.y + b.x;
            re[N - k] = a.x + b.y;
            im[N - k] = b.x - a.y;
        }
    });
    fft_inplace<N, true>(re, im);
    float *oa = out + ra * n - pad_l;
    float *ob = out + rb * n - pad_l;
    static_for<N>([&](auto ii) {
        constexpr int i = decltype(ii)::value;
        if ((i >= pad_l) && (i < pad_l + n)) {
            oa[i] = re[brev<N>(i)];
            if (has_b) ob[i] = im[brev<N>(i)];
        }
    });
}

// ---------------------------------------------------------------------------------
// 2-D, N = 2 or 4: one lane per plane, frequency-major spectrum like the larger sizes
// ---------------------------------------------------------------------------------
template <int N>
__global__ __launch_bounds__(256) void rfft2d_tiny_kernel(const float *__restrict__ in, float2 *__restrict__ out,
                                                       long planes, int h, int w, int pad_u, int pad_l)
{
    constexpr int NH = N / 2 + 1;
    const long p = (long)blockIdx.x * 256 + threadIdx.x;
    if (p >= planes) return;
    float xr[N][N], xi[N][N];  // [row][col]
    const float *src = in + p * (long)h * w;
    static_for<N>([&](auto rr) {
        constexpr int r = decltype(rr)::value;
        static_for<N>([&](auto cc) {
            constexpr int c = decltype(cc)::value;
            const int y = r - pad_u, x = c - pad_l;
            const bool ok = (y >= 0) && (y < h) && (x >= 0) && (x < w);
            xr[r][c] = ok ? src[y * w + x] : 0.0f;
            xi[r][c] = 0.0f;
        });
        fft_inplace<N, false>(xr[r], xi[r]);  // row r: X1[r][kx] at column brev(kx)
    });
    static_for<NH>([&](auto kk) {
        constexpr int kx = decltype(kk)::value;
        float cr[N], ci[N];
        static_for<N>([&](auto rr) {
            constexpr int r = decltype(rr)::value;
            cr[r] = xr[r][brev<N>(kx)];
            ci[r] = xi[r][brev<N>(kx)];
        });
        fft_inplace<N, false>(cr, ci);
        static_for<N>([&](auto yy) {
            constexpr int ky = decltype(yy)::value;
            out[((long)ky * NH + kx) * planes + p] = make_float2(cr[brev<N>(ky)], ci[brev<N>(ky)]);
        });
    });
}

template <int N>
__global__ __launch_bounds__(256) void irfft2d_tiny_kernel(const float2 *__restrict__ in, float *__restrict__ out,
                                                        long planes, int h, int w, int pad_u, int pad_l,
                                                        const float *__restrict__ bias, int bias_period)
{
    constexpr int NH = N / 2 + 1;
    const long p = (long)blockIdx.x * 256 + threadIdx.x;
    if (p >= planes) return;
    float xr[N][N], xi[N][N];  // [ky][kx], all N columns
    static_for<N>([&](auto yy) {
        constexpr int ky = decltype(yy)::value;
        static_for<NH>([&](auto kk) {
            constexpr int kx = decltype(kk)::value;
            const float2 v = in[((long)ky * NH + kx) * planes + p];
            xr[ky][kx] = v.x;
            xi[ky][kx] = v.y;
        });
    });
    // columns above N/2 of the spectrum of a real plane: X[ky][N-kx] = conj X[(N-ky) % N][kx]
    static_for<N>([&](auto yy) {
        constexpr int ky = decltype(yy)::value;
        static_for<N - NH>([&](auto kk) {
            constexpr int kx = decltype(kk)::value + 1;  // 1 .. N/2-1
            xr[ky][N - kx] = xr[(N - ky) % N][kx];
            xi[ky][N - kx] = -xi[(N - ky) % N][kx];
        });
    });
    // inverse over ky for every column, then over kx for every row
    static_for<N>([&](auto kk) {
        constexpr int kx = decltype(kk)::value;
        float cr[N], ci[N];
        static_for<N>([&](auto yy) { constexpr int ky = decltype(yy)::value; cr[ky] = xr[ky][kx]; ci[ky] = xi[ky][kx]; });
        fft_inplace<N, true>(cr, ci);
        static_for<N>([&](auto yy) {
            constexpr int y = decltype(yy)::value;
            xr[y][kx] = cr[brev<N>(y)];
            xi[y][kx] = ci[brev<N>(y)];
        });
    });
    const float bv = (bias != nullptr) ? bias[p % bias_period] : 0.0f;
    float *dst = out + p * (long)h * w;
    static_for<N>([&](auto yy) {
        constexpr int y = decltype(yy)::value;
        fft_inplace<N, true>(xr[y], xi[y]);
        static_for<N>([&](auto cc) {
            constexpr int c = decltype(cc)::value;
            const int r = y - pad_u, s = c - pad_l;
            if ((r >= 0) && (r < h) && (s >= 0) && (s < w)) dst[r * w + s] = xr[y][brev<N>(c)] + bv;
        });
    });
}

// ---------------------------------------------------------------------------------
// host launchers
// ---------------------------------------------------------------------------------
template <int N>
static hipError_t launch1d(bool inverse, const float *in, float *out, long rows, int n, int pad_l, hipStream_t s)
{
    const long pairs = (rows + 1) / 2;
    const long blocks = (pairs + 255) / 256;
    if (blocks > 0x7fffffffL) return hipErrorInvalidValue;
    if (!inverse)
        hipLaunchKernelGGL(rfft1d_kernel<N>, dim3((unsigned)blocks), dim3(256), 0, s, in,
                           reinterpret_cast<float2 *>(out), rows, n, pad_l);
    else
        hipLaunchKernelGGL(irfft1d_kernel<N>, dim3((unsigned)blocks), dim3(256), 0, s,
                           reinterpret_cast<const float2 *>(in), out, rows, n, pad_l);
    return hipGetLastError();
}

static hipError_t dispatch1d(bool inverse, int N, const float *in, float *out, long rows, int n, int pad_l,
                             hipStream_t s)
{
    switch (N) {
        case 2: return launch1d<2>(inverse, in, out, rows, n, pad_l, s);
        case 4: return launch1d<4>(inverse, in, out, rows, n, pad_l, s);
        case 8: return launch1d<8>(inverse, in, out, rows, n, pad_l, s);
        case 16: return launch1d<16>(inverse, in, out, rows, n, pad_l, s);
        case 32: return launch1d<32>(inverse, in, out, rows, n, pad_l, s);
        case 64: return launch1d<64>(inverse, in, out, rows, n, pad_l, s);
        case 128: return launch1d<128>(inverse, in, out, rows, n, pad_l, s);
        default: return hipErrorInvalidValue;
    }
}

hipError_t launch_rfft1d(int N, const float *in, float *out, long rows, int n, int pad_l, hipStream_t s)
{
    return dispatch1d(false, N, in, out, rows, n, pad_l, s);
}

hipError_t launch_irfft1d(int N, const float *in, float *out, long rows, int n, int pad_l, hipStream_t s)
{
    return dispatch1d(true, N, in, out, rows, n, pad_l, s);
}

hipError_t launch_rfft2d_tiny(int N, const float *in, float *out, long planes, int h, int w, int pad_u,
                              int pad_l, hipStream_t s)
{
    const long blocks = (planes + 255) / 256;
    if (blocks > 0x7fffffffL) return hipErrorInvalidValue;
    if (N == 2)
        hipLaunchKernelGGL(rfft2d_tiny_kernel<2>, dim3((unsigned)blocks), dim3(256), 0, s, in,
                           reinterpret_cast<float2 *>(out), planes, h, w, pad_u, pad_l);
    else if (N == 4)
        hipLaunchKernelGGL(rfft2d_tiny_kernel<4>, dim3((unsigned)blocks), dim3(256), 0, s, in,
                           reinterpret_cast<float2 *>(out), planes, h, w, pad_u, pad_l);
    else
        return hipErrorInvalidValue;
    return hipGetLastError();
}

hipError_t launch_irfft2d_tiny(int N, const float *in, float *out, long planes, int h, int w, int pad_u,
                               int pad_l, const float *bias, int bias_period, hipStream_t s)
{
    const long blocks = (planes + 255) / 256;
    if (blocks > 0x7fffffffL) return hipErrorInvalidValue;
    const int period = bias_period > 0 ? bias_period : 1;
    if (N == 2)
        hipLaunchKernelGGL(irfft2d_tiny_kernel<2>, dim3((unsigned)blocks), dim3(256), 0, s,
                           reinterpret_cast<const float2 *>(in), out, planes, h, w, pad_u, pad_l, bias, period);
    else if (N == 4)
        hipLaunchKernelGGL(irfft2d_tiny_kernel<4>, dim3((unsigned)blocks), dim3(256), 0, s,
                           reinterpret_cast<const float2 *>(in), out, planes, h, w, pad_u, pad_l, bias, period);
    else
        return hipErrorInvalidValue;
    return hipGetLastError();
}

}  // namespace fbfc
