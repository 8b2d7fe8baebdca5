// Batched 2-D real<->complex FFT kernels for gfx950 (power-of-two N, 8..64).
//
// Replaces what the reference asks of fbcuda's fbfft2D / fbifft2D through
// src/fft/FBFFTHost.cpp:39-116 (call sites :86-88, :93, :101-111): implicit zero
// padding at (padU, padL) on the way in, crop at (padU, padL) on the way out,
// Hermitian half spectrum, unnormalised inverse.
//
// Design (one workgroup = T consecutive planes, T*N/2 = 256 lanes):
//   * the T planes are one contiguous chunk of the real tensor: it is copied to
//     LDS with fully coalesced loads;
//   * row pass: one lane transforms TWO real rows at once as one complex
//     length-N FFT held entirely in registers (z = rowA + i rowB) and untangles
//     the two Hermitian spectra; columns 0 and N/2 of a real row spectrum are
//     real, so they share one complex slot and the tile is exactly N/2 wide;
//   * the tile R[y][kx][t] (plane index t fastest) lives in LDS, aliasing the
//     staging chunk; rows of the canvas that are known to be zero are neither
//     stored nor read back;
//   * column pass: one lane transforms one column (N complex points) in
//     registers; the lane owning slot 0 untangles columns 0 and N/2;
//   * results go straight from registers to the frequency-major buffer
//     freq[(ky*(N/2+1)+kx)*planes + plane]: the T lanes that share a frequency
//     write T consecutive complex numbers (T*8 bytes, 128 B for N=32).
// The inverse kernel is the mirror image and adds the bias while cropping.
#include <hip/hip_runtime.h>

#include "fft_regs.h"
#include "kernels.h"

namespace fbfc {

template <int N>
struct FftShape {
    static constexpr int T = 512 / N;       // planes per workgroup
    static constexpr int THREADS = 256;     // T * N / 2
    static constexpr int NH2 = N / 2;       // complex slots per tile row
    static constexpr int NH = N / 2 + 1;    // stored column frequencies
    // Phases: the LDS tile holds NH2/PH of the tile columns at a time and the input /
    // output staging area T/PH planes at a time, so that two workgroups fit one CU's
    // 160 KB LDS even for N = 64 (a full 8-plane tile would need 117 KB).
    static constexpr int PH = (N >= 64) ? 2 : 1;
    static constexpr int KXP = NH2 / PH;    // tile columns per phase
    static constexpr int TP = T / PH;       // planes per staging round
    // padding (in complex elements) between tile rows: keeps the T-lane groups
    // of one wave on different LDS banks when T*8 bytes is below 128
    static constexpr int ROWPAD = (T * 8 < 128) ? (64 / 8) / 2 : 0;
    static constexpr int ROWSTRIDE = KXP * T + ROWPAD;  // complex elements
};

// Copies np whole planes of hw floats between a contiguous global chunk and an
// LDS staging area whose plane stride hwp = hw|1 is odd, so that lanes reading
// the same (row, column) of consecutive planes hit different banks.
template <bool TO_LDS>
__device__ __forceinline__ void copy_planes(float *smem, float *g, int np, int hw, int hwp,
                                            int vec4, int tid)
{
    const int total = np * hw;
    if (vec4 && hwp == hw) {  // same layout on both sides: flat 16-byte copy
        const int n4 = total >> 2;
        float4 *g4 = reinterpret_cast<float4 *>(g);
        float4 *s4 = reinterpret_cast<float4 *>(smem);
        for (int i = tid; i < n4; i += 256) {
            if (TO_LDS) s4[i] = g4[i]; else g4[i] = s4[i];
        }
        for (int i = (n4 << 2) + tid; i < total; i += 256) {
            if (TO_LDS) smem[i] = g[i]; else g[i] = smem[i];
        }
    } else if (vec4 && (hw & 3) == 0) {  // 16-byte global accesses never straddle a plane
        const int n4 = total >> 2;
        float4 *g4 = reinterpret_cast<float4 *>(g);
        int e = tid * 4;
        int p = e / hw, off = e - p * hw;
        const int dp = 1024 / hw, doff = 1024 - dp * hw;
        for (int i = tid; i < n4; i += 256) {
            float *s = smem + p * hwp + off;
            if (TO_LDS) {
                const float4 v = g4[i];
                s[0] = v.x; s[1] = v.y; s[2] = v.z; s[3] = v.w;
            } else {
                g4[i] = make_float4(s[0], s[1], s[2], s[3]);
            }
            p += dp;
            off += doff;
            if (off >= hw) { off -= hw; ++p; }
        }
    } else {
        int p = tid / hw, off = tid - p * hw;
        const int dp = 256 / hw, doff = 256 - dp * hw;
        for (int i = tid; i < total; i += 256) {
            if (TO_LDS) smem[p * hwp + off] = g[i]; else g[i] = smem[p * hwp + off];
            p += dp;
            off += doff;
            if (off >= hw) { off -= hw; ++p; }
        }
    }
}

// ---------------------------------------------------------------------------------
// forward: real (planes,h,w) -> freq [N*(N/2+1)][planes] complex
// ---------------------------------------------------------------------------------
template <int N>
__global__ __launch_bounds__(256, FftShape<N>::PH) void rfft2d_kernel(const float *__restrict__ in,
                                                     float2 *__restrict__ out, long planes,
                                                     int h, int w, int padU, int padL, int vec4)
{
    using S = FftShape<N>;
    constexpr int T = S::T;
    extern __shared__ __align__(16) float smem[];
    const int tid = threadIdx.x;
    const long x0 = (long)blockIdx.x * T;
    const int np = (int)((planes - x0 < (long)T) ? (planes - x0) : (long)T);
    const int hw = h * w;
    const int hwp = hw | 1;                           // odd plane stride in the staging area
    const int y_lo = padU & ~1;                       // first canvas row that can be non-zero (even)
    const int y_hi = (padU + h + 1) & ~1;             // one past the last, rounded up to even

    const int t = tid % T;
    float re[N], im[N];

    // ---- row pass: lane (t, rp) owns canvas rows 2rp and 2rp+1 of plane t ----
    const int rp = tid / T;
    const int ya = 2 * rp, yb = ya + 1;
    const int ia = ya - padU, ib = yb - padU;
    const bool va = (ia >= 0) && (ia < h);
    const bool vb = (ib >= 0) && (ib < h);
    const bool row_active = (t < np) && (va || vb);

    // ---- stage the contiguous chunk of planes, TP planes per round ----
    static_for<S::PH>([&](auto hh) {
        constexpr int hs = decltype(hh)::value;
        int nph = np - hs * S::TP;
        nph = nph < 0 ? 0 : (nph > S::TP ? S::TP : nph);
        if (hs > 0) __syncthreads();  // previous round fully read
        copy_planes<true>(smem, const_cast<float *>(in) + (x0 + hs * S::TP) * hw, nph, hw, hwp, vec4, tid);
        __syncthreads();
        if (row_active && (t / S::TP) == hs) {
            const float *pa = smem + (t - hs * S::TP) * hwp + ia * w - padL;
            const float *pb = smem + (t - hs * S::TP) * hwp + ib * w - padL;
            static_for<N>([&](auto cc) {
                constexpr int c = decltype(cc)::value;
                const bool vc = (c >= padL) && (c < padL + w);
                re[c] = (va && vc) ? pa[c] : 0.0f;
                im[c] = (vb && vc) ? pb[c] : 0.0f;
            });
        }
    });

    // ---- row FFT and untangling ----
    // A[k] / B[k]: spectra of rows ya / yb; slot 0 carries the real-valued columns 0 and N/2.
    // The first phase's columns go straight to the LDS tile, later ones wait in registers.
    constexpr int NLATE = S::NH2 - S::KXP;  // 0 when there is a single phase
    float ar[NLATE > 0 ? NLATE : 1], ai[NLATE > 0 ? NLATE : 1], br[NLATE > 0 ? NLATE : 1], bi[NLATE > 0 ? NLATE : 1];
    float2 *R = reinterpret_cast<float2 *>(smem);
    const int kx = tid / T;  // column pass: lane (t, kx) owns tile column kx of plane t
    __syncthreads();  // staging area fully consumed; the tile may overwrite it
    if (row_active) {
        fft_inplace<N, false>(re, im);
        float2 *Ra = R + (ya - y_lo) * S::ROWSTRIDE + t;
        float2 *Rb = Ra + S::ROWSTRIDE;
        Ra[0] = make_float2(re[brev<N>(0)], re[brev<N>(N / 2)]);
        Rb[0] = make_float2(im[brev<N>(0)], im[brev<N>(N / 2)]);
        static_for<N / 2 - 1>([&](auto kk) {
            constexpr int k = decltype(kk)::value + 1;
            const float zr = re[brev<N>(k)], zi = im[brev<N>(k)];
            const float nr = re[brev<N>(N - k)], ni = im[brev<N>(N - k)];
            // A = (Z[k] + conj Z[N-k]) / 2 ; B = -i (Z[k] - conj Z[N-k]) / 2
            if constexpr (k < S::KXP) {
                Ra[k * T] = make_float2(0.5f * (zr + nr), 0.5f * (zi - ni));
                Rb[k * T] = make_float2(0.5f * (zi + ni), 0.5f * (nr - zr));
            } else {
                ar[k - S::KXP] = 0.5f * (zr + nr);  ai[k - S::KXP] = 0.5f * (zi - ni);
                br[k - S::KXP] = 0.5f * (zi + ni);  bi[k - S::KXP] = 0.5f * (nr - zr);
            }
        });
    }

    // Each phase: (later phases first refill the tile from registers) then the lanes whose
    // column belongs to the phase pull it into registers, which frees the tile again.
    static_for<S::PH>([&](auto pp) {
        constexpr int ph = decltype(pp)::value;
        if constexpr (ph > 0) {
            __syncthreads();  // previous phase's columns are in registers
            if (row_active) {
                float2 *Ra = R + (ya - y_lo) * S::ROWSTRIDE + t;
                float2 *Rb = Ra + S::ROWSTRIDE;
                static_for<S::KXP>([&](auto kk) {
                    constexpr int kl = decltype(kk)::value;
                    constexpr int k = ph * S::KXP + kl - S::KXP;
                    Ra[kl * T] = make_float2(ar[k], ai[k]);
                    Rb[kl * T] = make_float2(br[k], bi[k]);
                });
            }
        }
        __syncthreads();
        if ((t < np) && (kx / S::KXP) == ph) {
            const int kl = kx - ph * S::KXP;
            static_for<N>([&](auto yy) {
                constexpr int y = decltype(yy)::value;
                const bool vy = (y >= y_lo) && (y < y_hi);
                float2 v = make_float2(0.0f, 0.0f);
                if (vy) v = R[(y - y_lo) * S::ROWSTRIDE + kl * T + t];
                re[y] = v.x;
                im[y] = v.y;
            });
        }
    });

    // ---- column FFT and frequency-major store, all lanes at once ----
    if (t < np) {
        fft_inplace<N, false>(re, im);
        float2 *o = out + x0 + t;
        if (kx != 0) {
            static_for<N>([&](auto kk) {
                constexpr int ky = decltype(kk)::value;
                o[(long)(ky * S::NH + kx) * planes] = make_float2(re[brev<N>(ky)], im[brev<N>(ky)]);
            });
        } else {
            // C = FFT(col0 + i colNyq), both real sequences: untangle
            static_for<N>([&](auto kk) {
                constexpr int ky = decltype(kk)::value;
                constexpr int kn = (N - ky) % N;
                const float zr = re[brev<N>(ky)], zi = im[brev<N>(ky)];
                const float nr = re[brev<N>(kn)], ni = im[brev<N>(kn)];
                o[(long)(ky * S::NH + 0) * planes] = make_float2(0.5f * (zr + nr), 0.5f * (zi - ni));
                o[(long)(ky * S::NH + N / 2) * planes] = make_float2(0.5f * (zi + ni), 0.5f * (nr - zr));
            });
        }
    }
}

// ---------------------------------------------------------------------------------
// inverse: freq [N*(N/2+1)][planes] complex -> real (planes,h,w), unnormalised,
// real[r][s] = y[r+padU][s+padL] (+ bias[plane % bias_period])
// ---------------------------------------------------------------------------------
template <int N>
__global__ __launch_bounds__(256, FftShape<N>::PH) void irfft2d_kernel(const float2 *__restrict__ in,
                                                      float *__restrict__ out, long planes,
                                                      int h, int w, int padU, int padL,
                                                      const float *__restrict__ bias,
                                                      int bias_period, int vec4)
{
    using S = FftShape<N>;
    constexpr int T = S::T;
    extern __shared__ __align__(16) float smem[];
    const int tid = threadIdx.x;
    const long x0 = (long)blockIdx.x * T;
    const int np = (int)((planes - x0 < (long)T) ? (planes - x0) : (long)T);
    const int hw = h * w;
    const int hwp = hw | 1;                           // odd plane stride in the staging area
    const int y_lo = padU & ~1;                       // canvas rows the crop needs
    const int y_hi = (padU + h + 1) & ~1;

    const int t = tid % T;
    float re[N], im[N];
    float2 *R = reinterpret_cast<float2 *>(smem);

    // ---- column pass: lane (t, kx) fetches its whole column and transforms it, all lanes at once ----
    const int kx = tid / T;
    if (t < np) {
        const float2 *src = in + x0 + t;
        if (kx != 0) {
            static_for<N>([&](auto kk) {
                constexpr int ky = decltype(kk)::value;
                const float2 v = src[(long)(ky * S::NH + kx) * planes];
                re[ky] = v.x;
                im[ky] = v.y;
            });
        } else {
            // pack columns 0 and N/2 (each the spectrum of a real sequence): C = X0 + i XN
            static_for<N>([&](auto kk) {
                constexpr int ky = decltype(kk)::value;
                const float2 a = src[(long)(ky * S::NH + 0) * planes];
                const float2 b = src[(long)(ky * S::NH + N / 2) * planes];
                re[ky] = a.x - b.y;
                im[ky] = a.y + b.x;
            });
        }
        fft_inplace<N, true>(re, im);
    }

    // ---- row pass bookkeeping: lane (t, rp) rebuilds canvas rows 2rp, 2rp+1 ----
    const int rp = tid / T;
    const int ya = 2 * rp, yb = ya + 1;
    const int ia = ya - padU, ib = yb - padU;
    const bool va = (ia >= 0) && (ia < h);
    const bool vb = (ib >= 0) && (ib < h);
    const bool row_active = (t < np) && (va || vb);
    // Z[k] = Ya[k] + i Yb[k], k = 0..N-1, with Y[N-k] = conj Y[k]
    float zr[N], zi[N];

    static_for<S::PH>([&](auto pp) {
        constexpr int ph = decltype(pp)::value;
        if (ph > 0) __syncthreads();  // previous phase's tile fully read
        if ((t < np) && (kx / S::KXP) == ph) {
            const int kl = kx - ph * S::KXP;
            static_for<N>([&](auto yy) {
                constexpr int y = decltype(yy)::value;
                if ((y >= y_lo) && (y < y_hi))
                    R[(y - y_lo) * S::ROWSTRIDE + kl * T + t] = make_float2(re[brev<N>(y)], im[brev<N>(y)]);
            });
        }
        __syncthreads();
        if (row_active) {
            const float2 *Ra = R + (ya - y_lo) * S::ROWSTRIDE + t;
            const float2 *Rb = Ra + S::ROWSTRIDE;
            static_for<S::KXP>([&](auto kk) {
                constexpr int kl = decltype(kk)::value;
                constexpr int k = ph * S::KXP + kl;
                const float2 a = Ra[kl * T], b = Rb[kl * T];
                if constexpr (k == 0) {
                    zr[0] = a.x;      zi[0] = b.x;        // k = 0   : both real
                    zr[N / 2] = a.y;  zi[N / 2] = b.y;    // k = N/2 : both real
                } else {
                    zr[k] = a.x - b.y;      zi[k] = a.y + b.x;
                    zr[N - k] = a.x + b.y;  zi[N - k] = b.x - a.y;
                }
            });
        }
    });
    __syncthreads();  // tile fully consumed; the staging area may overwrite it

    float bv = 0.0f;
    if (row_active) {
        fft_inplace<N, true>(zr, zi);
        if (bias != nullptr) bv = bias[(x0 + t) % bias_period];
    }
    // ---- crop (+bias) into the staging area and coalesced copy-out, TP planes per round ----
    static_for<S::PH>([&](auto hh) {
        constexpr int hs = decltype(hh)::value;
        int nph = np - hs * S::TP;
        nph = nph < 0 ? 0 : (nph > S::TP ? S::TP : nph);
        if (hs > 0) __syncthreads();  // previous round copied out
        if (row_active && (t / S::TP) == hs) {
            float *pa = smem + (t - hs * S::TP) * hwp + ia * w - padL;
            float *pb = smem + (t - hs * S::TP) * hwp + ib * w - padL;
            static_for<N>([&](auto cc) {
                constexpr int c = decltype(cc)::value;
                const bool vc = (c >= padL) && (c < padL + w);
                if (va && vc) pa[c] = zr[brev<N>(c)] + bv;
                if (vb && vc) pb[c] = zi[brev<N>(c)] + bv;
            });
        }
        __syncthreads();
        copy_planes<false>(smem, out + (x0 + hs * S::TP) * hw, nph, hw, hwp, vec4, tid);
    });
}

// ---------------------------------------------------------------------------------
// host launchers
// ---------------------------------------------------------------------------------
template <int N>
static size_t fft_lds_bytes(int h, int w, int padU, bool inverse)
{
    using S = FftShape<N>;
    const int y_lo = padU & ~1, y_hi = (padU + h + 1) & ~1;
    const size_t tile = (size_t)(y_hi - y_lo) * S::ROWSTRIDE * sizeof(float2);
    (void)inverse;
    const size_t plane = (size_t)((h * w) | 1);
    const size_t stage = (size_t)S::TP * plane * sizeof(float);
    return ((tile > stage ? tile : stage) + 15) & ~(size_t)15;
}

template <int N>
static hipError_t launch_fwd(const float *in, float *out, long planes, int h, int w, int padU,
                             int padL, hipStream_t s)
{
    using S = FftShape<N>;
    static bool attr_done = false;
    if (!attr_done) {
        hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(&rfft2d_kernel<N>),
                                           hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
        if (e != hipSuccess) return e;
        attr_done = true;
    }
    const size_t lds = fft_lds_bytes<N>(h, w, padU, false);
    const long blocks = (planes + S::T - 1) / S::T;
    const int vec4 = ((reinterpret_cast<uintptr_t>(in) & 15) == 0) && (((long)S::T * h * w) % 4 == 0);
    hipLaunchKernelGGL(rfft2d_kernel<N>, dim3((unsigned)blocks), dim3(256), lds, s, in,
                       reinterpret_cast<float2 *>(out), planes, h, w, padU, padL, vec4);
    return hipGetLastError();
}

template <int N>
static hipError_t launch_inv(const float *in, float *out, long planes, int h, int w, int padU,
                             int padL, const float *bias, int bias_period, hipStream_t s)
{
    using S = FftShape<N>;
    static bool attr_done = false;
    if (!attr_done) {
        hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(&irfft2d_kernel<N>),
                                           hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
        if (e != hipSuccess) return e;
        attr_done = true;
    }
    const size_t lds = fft_lds_bytes<N>(h, w, padU, true);
    const long blocks = (planes + S::T - 1) / S::T;
    const int vec4 = ((reinterpret_cast<uintptr_t>(out) & 15) == 0) && (((long)S::T * h * w) % 4 == 0);
    hipLaunchKernelGGL(irfft2d_kernel<N>, dim3((unsigned)blocks), dim3(256), lds, s,
                       reinterpret_cast<const float2 *>(in), out, planes, h, w, padU, padL, bias,
                       bias_period > 0 ? bias_period : 1, vec4);
    return hipGetLastError();
}

hipError_t launch_rfft2d(int N, const float *in, float *out, long planes, int h, int w, int padU,
                         int padL, hipStream_t s)
{
    switch (N) {
        case 8: return launch_fwd<8>(in, out, planes, h, w, padU, padL, s);
        case 16: return launch_fwd<16>(in, out, planes, h, w, padU, padL, s);
        case 32: return launch_fwd<32>(in, out, planes, h, w, padU, padL, s);
        case 64: return launch_fwd<64>(in, out, planes, h, w, padU, padL, s);
        default: return hipErrorInvalidValue;
    }
}

hipError_t launch_irfft2d(int N, const float *in, float *out, long planes, int h, int w, int padU,
                          int padL, const float *bias, int bias_period, hipStream_t s)
{
    switch (N) {
        case 8: return launch_inv<8>(in, out, planes, h, w, padU, padL, bias, bias_period, s);
        case 16: return launch_inv<16>(in, out, planes, h, w, padU, padL, bias, bias_period, s);
        case 32: return launch_inv<32>(in, out, planes, h, w, padU, padL, bias, bias_period, s);
        case 64: return launch_inv<64>(in, out, planes, h, w, padU, padL, bias, bias_period, s);
        default: return hipErrorInvalidValue;
    }
}

}  // namespace fbfc
