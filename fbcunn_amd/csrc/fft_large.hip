// Batched 2-D real<->complex FFT kernels for the large sizes (N = 64, 128) on gfx950.
//
// Same job as fft_kernels.hip (what the reference asks of fbcuda's fbfft2D / fbifft2D through
// src/fft/FBFFTHost.cpp:39-116: implicit zero padding, crop, Hermitian half spectrum, unnormalised
// inverse, frequency-major spectrum), same staging and tile, but the transforms are cut finer so
// that a lane holds N/2 complex values instead of N:
//   * row pass: one lane owns ONE real canvas row.  z[n] = x[2n] + i x[2n+1] is a complex
//     sequence of length N/2; the lane transforms it in registers and splits the result into the
//     row's Hermitian half spectrum X[0..N/2] (the textbook real transform by a half-length
//     complex one).  Columns 0 and N/2 are real and share tile slot 0, so a tile row is N/2 slots.
//   * column pass: a column of N complex values is split over TWO lanes, the "roles", which sit
//     in different waves so that everything that depends on the role is wave-uniform.
//     Forward: both roles read the whole column from the LDS tile; role r forms
//     y_r[n] = c[n] + (-1)^r c[n + N/2] and transforms it with the twisted block of fft_regs.h
//     (theta = r / 2), which yields the outputs ky = 2 k' + r.
//     Inverse: role r loads the inputs ky = 2 m + r from global memory, transforms them, role 1
//     multiplies by exp(+2 pi i k / N), and the tile receives E (rows 0..N/2-1) and T (rows
//     N/2..N-1); canvas row y is E[y mod N/2] +/- T[y mod N/2], which the row lane forms on reading.
// A workgroup of T planes has T * N lanes: 1024 at N = 64 with T = 16 (whole 128-byte runs per
// frequency, 128 registers per lane, 16 waves per CU) where the earlier design had 512 lanes at
// 256 registers; 512 at N = 128 with T = 4, where a lane held 256 values and spilled.
#include <hip/hip_runtime.h>

#include <cstdio>

#include "bias_dc.h"
#include "fft_regs.h"
#include "fft_stage.h"
#include "kernels.h"
#include "store_nt.h"

namespace fbfc {

template <int N, int T_, bool SMALL = false>
struct RowShape {
    static constexpr int T = T_;               // planes per workgroup
    static constexpr int THREADS = T * N;      // one lane per canvas row of every plane
    static constexpr int M = N / 2;            // complex length of a row lane's transform = tile slots per row
    static constexpr int NH = N / 2 + 1;       // stored column frequencies
    // Phases: the tile holds M / PH slots of every row at a time (the others wait in registers) and
    // the staging area T / PH planes.  Small planes (at most 16 rows) fit at once.
    static constexpr int PH = SMALL ? 1 : 2;
    static constexpr int KXP = M / PH;
    static constexpr int TP = T / PH;
    static constexpr int LPR = THREADS / PH;   // lanes of one staging round: whole waves
    // A wave of the row pass writes 64 / T tile rows of T consecutive complex values each; with the
    // row stride = T (mod 32) complex the rows of a wave tile the 64 banks.
    static constexpr int ROWPAD = (T < 32) ? T : 0;
    static constexpr int ROWSTRIDE = KXP * T + ROWPAD;
    // plane groups that share a 128-byte line of a frequency's run
    static constexpr int G = (T * 8 >= 128) ? 1 : 16 / T;
    // waves per SIMD the register budget is sized for: 1024 lanes fill a CU at 128 registers; 512
    // lanes get 128 registers at N = 64 (two workgroups per CU) and 256 at N = 128 (one)
    static constexpr int MIN_WAVES = (THREADS >= 1024) ? 4 : (N >= 128) ? 2 : 4;
};

// ---------------------------------------------------------------------------------
// forward: real (planes,h,w) -> freq [N*(N/2+1)][planes] complex
// ---------------------------------------------------------------------------------
// Stores the outputs ky = 2 k' + ROLE of one tile column (X[2 k' + ROLE] sits at brev(k')).
template <int N, int WHOLE, int ROLE>
__device__ __forceinline__ void store_column(const float (&re)[N / 2], const float (&im)[N / 2], char *obase,
                                             long rowbytes, unsigned voff, unsigned vnyq, bool slot0, int herm)
{
    constexpr int M = N / 2;
    if (!slot0) {
        static_for<M>([&](auto kk) {
            constexpr int k = decltype(kk)::value;
            store_freq_at<WHOLE>(obase + (2 * k + ROLE) * rowbytes, voff,
                                  make_float2(re[brev<M>(k)], im[brev<M>(k)]));
        });
    } else {
        // slot 0 carries C = FFT(col0 + i colNyq), both real sequences: untangle.  The partner of
        // ky = 2 k + ROLE is N - ky = 2 k2 + ROLE with k2 = (M - k - ROLE) mod M: the same role.
        // Rows 0 .. N/2 come from k <= KLOW; the rows above N/2 repeat the rows below it as conjugates
        // (both columns are spectra of real sequences) and are written, unless the caller leaves them
        // out, right beside their partner, so that nothing is kept for later.
        constexpr int KLOW = (N / 2 - ROLE) / 2;
        static_for<KLOW + 1>([&](auto kk) {
            constexpr int k = decltype(kk)::value;
            constexpr int ky = 2 * k + ROLE;
            constexpr int k2 = (M - k - ROLE) % M;
            const float zr = re[brev<M>(k)], zi = im[brev<M>(k)];
            const float nr = re[brev<M>(k2)], ni = im[brev<M>(k2)];
            const float2 c0 = make_float2(0.5f * (zr + nr), 0.5f * (zi - ni));
            const float2 cn = make_float2(0.5f * (zi + ni), 0.5f * (nr - zr));
            store_freq_at<WHOLE>(obase + ky * rowbytes, voff, c0);
            store_freq_at<WHOLE>(obase + ky * rowbytes, vnyq, cn);
            if constexpr (ky > 0 && ky < N / 2) {
                if (!herm) {
                    store_freq_at<WHOLE>(obase + (N - ky) * rowbytes, voff,
                                          make_float2(c0.x, -c0.y));
                    store_freq_at<WHOLE>(obase + (N - ky) * rowbytes, vnyq,
                                          make_float2(cn.x, -cn.y));
                }
            }
        });
    }
}

// NZ < N: planes of at most NZ x NZ at the canvas origin (convolution kernels): the transforms skip
// the inputs that are known to be zero and the tile keeps NZ rows.
template <int N, int T, int NZ, bool RAW>
__global__ __launch_bounds__((RowShape<N, T, (NZ < N)>::THREADS), (RowShape<N, T, (NZ < N)>::MIN_WAVES)) void
rfft2d_rows_kernel(FwdJob job0, FwdJob job1, FwdJob job2, unsigned blocks0, unsigned blocks01)
{
    constexpr bool SMALL = NZ < N;
    using S = RowShape<N, T, SMALL>;
    constexpr int M = S::M;
    constexpr bool WHOLE = (T * 8 >= 128);
    extern __shared__ __align__(16) float smem[];
    const int tid = threadIdx.x;
    const unsigned v = blockIdx.x;
    // up to three tensors per launch: workgroups [0, blocks0) work on job 0, [blocks0, blocks01) on
    // job 1, the rest on job 2
    const bool second = v >= blocks0, third = v >= blocks01;
    const FwdJob &job = third ? job2 : (second ? job1 : job0);
    const float *__restrict__ in = job.in;
    float2 *__restrict__ out = job.out;
    const long planes = job.planes;
    const int h = job.h, w = job.w;
    const int padU = job.padU, padL = job.padL;
    const int vec4 = job.vec4;
    const int herm = job.herm;
    const int stream = job.stream;
    const long x0 = plane_group<T, S::G>(v - (third ? blocks01 : (second ? blocks0 : 0u))) * T;
    if (x0 >= planes) return;
    const int np = (int)((planes - x0 < (long)T) ? (planes - x0) : (long)T);
    const int hw = h * w;

    // ---- row pass: lane (t, y) owns canvas row y of plane t.  The planes are staged TP at a time;
    // the lanes of round r are LPR consecutive ones (whole waves) ----
    const int round_of_lane = tid / S::LPR, rl = tid % S::LPR;
    const int t = round_of_lane * S::TP + rl % S::TP;
    const int y = rl / S::TP;
    const int iy = y - padU;
    const bool row_active = (t < np) && (iy >= 0) && (iy < h);
    constexpr int NZH = SMALL ? NZ / 2 : M;  // complex inputs z[n] that can be non-zero
    float re[M], im[M];

    constexpr int LDR = Canvas<N>::LDR;
    static_assert(!RAW || N <= 64, "raw staging masks the row with a 64-bit column mask");
    // raw staging: bit x of colmask = canvas column x lies inside the plane
    [[maybe_unused]] const unsigned long long colmask = ((w >= 64) ? ~0ull : ((1ull << w) - 1ull)) << padL;
    static_for<S::PH>([&](auto hh) {
        constexpr int hs = decltype(hh)::value;
        int nph = np - hs * S::TP;
        nph = nph < 0 ? 0 : (nph > S::TP ? S::TP : nph);
        if (hs > 0) __syncthreads();  // previous round fully read
        if constexpr (RAW) {
            // the chunk as it lies, N floats of slack on either side (the first row is read from
            // -padL on, the last one up to N - 1 - padL); what lies left and right of a row is masked off
            float *raw = smem + N;
            stage_raw<(N >= 64) ? 2 : 0, S::THREADS>(raw, in + (x0 + hs * S::TP) * hw, nph * hw, vec4 != 0, tid);
            __builtin_amdgcn_s_waitcnt(0x0f70);  // vmcnt(0): this wave's pieces have landed
            __syncthreads();
            if (row_active && round_of_lane == hs) {
                const float *p = raw + ((t - hs * S::TP) * h + iy) * w - padL;
                static_for<M>([&](auto nn) {
                    constexpr int n = decltype(nn)::value;
                    if constexpr (n < NZH) {
                        const unsigned m0 = ((colmask >> (2 * n)) & 1ull) ? 0xffffffffu : 0u;
                        const unsigned m1 = ((colmask >> (2 * n + 1)) & 1ull) ? 0xffffffffu : 0u;
                        re[n] = __uint_as_float(__float_as_uint(p[2 * n]) & m0);
                        im[n] = __uint_as_float(__float_as_uint(p[2 * n + 1]) & m1);
                    } else {
                        re[n] = 0.0f;
                        im[n] = 0.0f;
                    }
                });
            }
        } else {
            zero_canvas_margins<N, S::THREADS>(smem, nph * h, w, padL, S::TP * h * LDR, tid);
            copy_canvas<N, true, S::THREADS>(smem, const_cast<float *>(in) + (x0 + hs * S::TP) * hw, nph * h, w, padL,
                                             vec4, tid);
            __syncthreads();
            if (row_active && round_of_lane == hs) {
                const float4 *p = reinterpret_cast<const float4 *>(smem + ((t - hs * S::TP) * h + iy) * LDR);
                static_for<N / 4>([&](auto jj) {
                    constexpr int j = decltype(jj)::value;
                    if constexpr (2 * j < NZH) {
                        const float4 q = p[j];
                        re[2 * j] = q.x; im[2 * j] = q.y; re[2 * j + 1] = q.z; im[2 * j + 1] = q.w;
                    } else {
                        re[2 * j] = im[2 * j] = re[2 * j + 1] = im[2 * j + 1] = 0.0f;
                    }
                });
            }
        }
    });

    // ---- row transform.  Z = FFT(z) gives the row spectrum by
    //   E = (Z[k] + conj Z[M-k]) / 2,  O = -i (Z[k] - conj Z[M-k]) / 2,  W = exp(-2 pi i k / N)
    //   X[k] = E + W O,   X[M-k] = conj(E - W O),   X[0] = Re Z0 + Im Z0,  X[M] = Re Z0 - Im Z0.
    // Slot k of the tile row holds X[k]; slot 0 the two real values (X[0], X[M]).  The first phase's
    // slots go straight to the tile, later ones wait in registers ----
    constexpr int NLATE = M - S::KXP;
    constexpr int TROWS = SMALL ? NZ : N;
    float lr[NLATE > 0 ? NLATE : 1], li[NLATE > 0 ? NLATE : 1];
    float2 *R = reinterpret_cast<float2 *>(smem);
    float2 *Rr = R + y * S::ROWSTRIDE + t;
    __syncthreads();  // staging area fully consumed; the tile may overwrite it
    if (row_active) {
        fft_inplace_nz<M, NZH, false>(re, im);
        auto put = [&](auto kk, float xr, float xi) {
            constexpr int k = decltype(kk)::value;
            if constexpr (k < S::KXP) {
                Rr[k * T] = make_float2(xr, xi);
            } else {
                lr[k - S::KXP] = xr;
                li[k - S::KXP] = xi;
            }
        };
        put(std::integral_constant<int, 0>{}, re[0] + im[0], re[0] - im[0]);
        put(std::integral_constant<int, M / 2>{}, re[brev<M>(M / 2)], -im[brev<M>(M / 2)]);
        static_for<M / 2 - 1>([&](auto kk) {
            constexpr int k = decltype(kk)::value + 1;
            const float a = re[brev<M>(k)], b = im[brev<M>(k)];
            const float c = re[brev<M>(M - k)], d = im[brev<M>(M - k)];
            const float t1 = a + c, t2 = b - d, t3 = b + d, t4 = c - a;
            constexpr float wr = (float)(0.5 * cos2pi(k, N)), wi = (float)(-0.5 * sin2pi(k, N));
            // every multiply-add is spelt out: the file is compiled without implicit contraction, so that
            // the instantiations of this kernel (raw / canvas staging) round alike
            const float pr = __builtin_fmaf(wr, t3, -(wi * t4)), pi_ = __builtin_fmaf(wr, t4, wi * t3);
            put(std::integral_constant<int, k>{}, __builtin_fmaf(0.5f, t1, pr), __builtin_fmaf(0.5f, t2, pi_));
            put(std::integral_constant<int, M - k>{}, __builtin_fmaf(0.5f, t1, -pr), __builtin_fmaf(-0.5f, t2, pi_));
        });
    } else if (t < np && y < TROWS) {
        // a canvas row outside the plane is zero in every phase: written once, the refills below
        // leave it alone
        static_for<S::KXP>([&](auto kk) {
            constexpr int k = decltype(kk)::value;
            Rr[k * T] = make_float2(0.0f, 0.0f);
        });
    }

    // ---- column pass: lane (role, tc, kx) computes the outputs ky = 2 k' + role of tile column kx
    // of plane tc.  Each phase: (later phases first refill the tile from registers) then the lanes
    // whose column belongs to the phase pull it into registers, already folded to half length ----
    const int role = __builtin_amdgcn_readfirstlane(tid / (S::THREADS / 2));
    const int cl = tid % (S::THREADS / 2);
    const int tc = cl % T, kx = cl / T;
    const float sgn = role ? -1.0f : 1.0f;
    static_for<S::PH>([&](auto pp) {
        constexpr int ph = decltype(pp)::value;
        if constexpr (ph > 0) {
            __syncthreads();  // previous phase's columns are in registers
            if (row_active) {
                static_for<S::KXP>([&](auto kk) {
                    constexpr int kl = decltype(kk)::value;
                    constexpr int k = ph * S::KXP + kl - S::KXP;
                    Rr[kl * T] = make_float2(lr[k], li[k]);
                });
            }
        }
        __syncthreads();
        if ((tc < np) && (kx / S::KXP) == ph) {
            const float2 *col = R + (kx - ph * S::KXP) * T + tc;
            static_for<M>([&](auto nn) {
                constexpr int n = decltype(nn)::value;
                if constexpr (SMALL) {
                    // rows from NZ on are zero: both roles start from the column itself
                    if constexpr (n < NZ) {
                        const float2 a = col[n * S::ROWSTRIDE];
                        re[n] = a.x;
                        im[n] = a.y;
                    } else {
                        re[n] = 0.0f;
                        im[n] = 0.0f;
                    }
                } else {
                    const float2 a = col[n * S::ROWSTRIDE], b = col[(n + M) * S::ROWSTRIDE];
                    re[n] = __builtin_fmaf(sgn, b.x, a.x);
                    im[n] = __builtin_fmaf(sgn, b.y, a.y);
                    // the column arrives as 2 M values and leaves as M: keep the scheduler from
                    // issuing all loads before the first fold (it would hold 2 M values and spill)
                    if constexpr (n % 8 == 7) __builtin_amdgcn_sched_barrier(0);
                }
            });
        }
    });

    // ---- column transform and frequency-major store, all lanes at once ----
    if (tc < np) {
        constexpr int NZC = SMALL ? NZ : M;
        // address = uniform base (frequency row ky, first plane of the group) + 32-bit lane offset
        const unsigned voff = (unsigned)(((long)kx * planes + tc) * (long)sizeof(float2));
        const unsigned vnyq = (unsigned)(((long)(N / 2) * planes + tc) * (long)sizeof(float2));
        char *obase = reinterpret_cast<char *>(out + x0);
        const long rowbytes = (long)S::NH * planes * (long)sizeof(float2);
        if (role == 0) {
            fft_block_nz<M, 0, 0, 2, false, NZC>(re, im);
            with_store_mode<WHOLE>(stream, [&](auto mode_tag) {
                store_column<N, decltype(mode_tag)::value, 0>(re, im, obase, rowbytes, voff, vnyq, kx == 0, herm);
            });
        } else {
            fft_block_nz<M, 0, 1, 2, false, NZC>(re, im);
            with_store_mode<WHOLE>(stream, [&](auto mode_tag) {
                store_column<N, decltype(mode_tag)::value, 1>(re, im, obase, rowbytes, voff, vnyq, kx == 0, herm);
            });
        }
    }
}

// ---------------------------------------------------------------------------------
// inverse: freq [N*(N/2+1)][planes] complex -> real (planes,h,w), unnormalised,
// real[r][s] = y[r+padU][s+padL] (+ bias[plane % bias_period])
// ---------------------------------------------------------------------------------
// Loads the inputs ky = 2 m + ROLE of one column into position m.
template <int N, int ROLE>
__device__ __forceinline__ void load_column(float (&re)[N / 2], float (&im)[N / 2], const char *ibase,
                                            long rowbytes, unsigned voff, unsigned vnyq, bool slot0)
{
    constexpr int M = N / 2;
    if (!slot0) {
        static_for<M>([&](auto mm) {
            constexpr int m = decltype(mm)::value;
            const float2 v = *reinterpret_cast<const float2 *>(ibase + (2 * m + ROLE) * rowbytes + voff);
            re[m] = v.x;
            im[m] = v.y;
        });
    } else {
        // pack columns 0 and N/2 (each the spectrum of a real sequence): C = X0 + i XN.  Rows above
        // N/2 are the conjugates of the rows below it and are not read: row j <= N/2 gives C[j] and
        // C[N - j], both of the parity of j.
        static_for<(ROLE == 0) ? M / 2 + 1 : M / 2>([&](auto jj) {
            constexpr int j = 2 * decltype(jj)::value + ROLE;
            const float2 a = *reinterpret_cast<const float2 *>(ibase + j * rowbytes + voff);
            const float2 b = *reinterpret_cast<const float2 *>(ibase + j * rowbytes + vnyq);
            re[(j - ROLE) / 2] = a.x - b.y;
            im[(j - ROLE) / 2] = a.y + b.x;
            if constexpr (j > 0 && j < N / 2) {
                re[(N - j - ROLE) / 2] = a.x + b.y;
                im[(N - j - ROLE) / 2] = b.x - a.y;
            }
        });
    }
}

template <int N, int T>
__global__ __launch_bounds__((RowShape<N, T>::THREADS), (RowShape<N, T>::MIN_WAVES)) void
irfft2d_rows_kernel(const float2 *__restrict__ in, float *__restrict__ out, long planes, int h, int w, int padU,
                    int padL, const float *__restrict__ bias, int bias_period, int vec4, int ppad, BiasGradJob bgrad,
                    unsigned bgrad_blocks)
{
    using S = RowShape<N, T>;
    constexpr int M = S::M;
    extern __shared__ __align__(16) float smem[];
    if (blockIdx.x < bgrad_blocks) {
        // an independent small job riding on this launch: the bias gradient of the same pass
        // (1 KB of the dynamic LDS, which is never smaller than one tile row)
        bias_grad_dc_body(bgrad, blockIdx.x, reinterpret_cast<float (*)[64]>(smem));
        return;
    }
    const int tid = threadIdx.x;
    const long x0 = plane_group<T, S::G>(blockIdx.x - bgrad_blocks) * T;
    if (x0 >= planes) return;
    const int np = (int)((planes - x0 < (long)T) ? (planes - x0) : (long)T);
    const int hw = h * w;
    float2 *R = reinterpret_cast<float2 *>(smem);

    // ---- column pass: lane (role, tc, kx) takes the inputs ky = 2 m + role of its column.  With
    // E_r = transform of those, the column's result is X[k] = E_0[k] + V^k E_1[k],
    // X[k + M] = E_0[k] - V^k E_1[k], V = exp(+2 pi i / N): role 1 multiplies by V^k, the sum and
    // the difference are formed by the row lanes that read the tile ----
    const int role = __builtin_amdgcn_readfirstlane(tid / (S::THREADS / 2));
    const int cl = tid % (S::THREADS / 2);
    const int tc = cl % T, kx = cl / T;
    float re[M], im[M];
    if (tc < np) {
        const unsigned voff = (unsigned)(((long)kx * planes + tc) * (long)sizeof(float2));
        const unsigned vnyq = (unsigned)(((long)(N / 2) * planes + tc) * (long)sizeof(float2));
        const char *ibase = reinterpret_cast<const char *>(in + x0);
        const long rowbytes = (long)S::NH * planes * (long)sizeof(float2);
        if (role == 0) {
            load_column<N, 0>(re, im, ibase, rowbytes, voff, vnyq, kx == 0);
            fft_inplace<M, true>(re, im);
        } else {
            load_column<N, 1>(re, im, ibase, rowbytes, voff, vnyq, kx == 0);
            fft_inplace<M, true>(re, im);
            static_for<M - 1>([&](auto kk) {
                constexpr int k = decltype(kk)::value + 1;
                constexpr int p = brev<M>(k);
                const float xr = re[p], xi = im[p];
                if constexpr (2 * k == M) {  // V^k = i
                    re[p] = -xi;
                    im[p] = xr;
                } else {
                    constexpr float vr = (float)cos2pi(k, N), vi = (float)sin2pi(k, N);
                    re[p] = __builtin_fmaf(xr, vr, -(xi * vi));
                    im[p] = __builtin_fmaf(xr, vi, xi * vr);
                }
            });
        }
    }

    // ---- row pass: lane (tr, y) rebuilds canvas row y of plane tr.  Its spectrum is
    // Y[k] = E[y mod M][k] + s T[y mod M][k], s = +1 for y < M and -1 above; the half-length sequence
    //   Z'[k] = (Y[k] + conj Y[M-k]) + i V^k (Y[k] - conj Y[M-k]),  k < M
    // transforms into z[n] = y[2n] + i y[2n+1] ----
    const int round_of_lane = tid / S::LPR, rl = tid % S::LPR;
    const int tr = round_of_lane * S::TP + rl % S::TP;
    const int y = rl / S::TP;
    const int iy = y - padU;
    const bool row_active = (tr < np) && (iy >= 0) && (iy < h);
    const float sgn = (y >= M) ? -1.0f : 1.0f;
    float zr[M], zi[M];

    static_for<S::PH>([&](auto pp) {
        constexpr int ph = decltype(pp)::value;
        if (ph > 0) __syncthreads();  // previous phase's tile fully read
        if ((tc < np) && (kx / S::KXP) == ph) {
            float2 *col = R + (role * M) * S::ROWSTRIDE + (kx - ph * S::KXP) * T + tc;
            static_for<M>([&](auto kk) {
                constexpr int k = decltype(kk)::value;
                col[k * S::ROWSTRIDE] = make_float2(re[brev<M>(k)], im[brev<M>(k)]);
            });
        }
        __syncthreads();
        if (row_active) {
            const float2 *Re = R + (y & (M - 1)) * S::ROWSTRIDE + tr;
            const float2 *Rt = Re + M * S::ROWSTRIDE;
            static_for<S::KXP>([&](auto kk) {
                constexpr int kl = decltype(kk)::value;
                constexpr int k = ph * S::KXP + kl;
                const float2 e = Re[kl * T], tt = Rt[kl * T];
                // slot 0 carries the two real values Y[0] and Y[M]
                zr[k] = __builtin_fmaf(sgn, tt.x, e.x);
                zi[k] = __builtin_fmaf(sgn, tt.y, e.y);
            });
        }
    });
    __syncthreads();  // tile fully consumed; the staging area may overwrite it

    float bv = 0.0f;
    if (row_active) {
        {
            const float y0 = zr[0], ym = zi[0];
            zr[0] = y0 + ym;
            zi[0] = y0 - ym;
            zr[M / 2] = 2.0f * zr[M / 2];
            zi[M / 2] = -2.0f * zi[M / 2];
        }
        static_for<M / 2 - 1>([&](auto kk) {
            constexpr int k = decltype(kk)::value + 1;
            const float a = zr[k], b = zi[k], c = zr[M - k], d = zi[M - k];
            const float sr = a + c, si = b - d, dr = a - c, di = b + d;
            constexpr float vr = (float)cos2pi(k, N), vi = (float)sin2pi(k, N);
            const float p = __builtin_fmaf(vr, dr, -(vi * di)), q = __builtin_fmaf(vr, di, vi * dr);
            zr[k] = sr - q;
            zi[k] = si + p;
            zr[M - k] = sr + q;
            zi[M - k] = p - si;
        });
        fft_inplace<M, true>(zr, zi);
        if (bias != nullptr) bv = bias[(x0 + tr) % bias_period];
    }
    // ---- canvas rows (+bias) into the staging area, cropped coalesced copy-out, TP planes per round ----
    constexpr int LDR = Canvas<N>::LDR;
    static_for<S::PH>([&](auto hh) {
        constexpr int hs = decltype(hh)::value;
        int nph = np - hs * S::TP;
        nph = nph < 0 ? 0 : (nph > S::TP ? S::TP : nph);
        if (hs > 0) __syncthreads();  // previous round copied out
        if (row_active && round_of_lane == hs) {
            float4 *p = reinterpret_cast<float4 *>(smem + (tr - hs * S::TP) * (h * LDR + ppad) + iy * LDR);
            static_for<N / 4>([&](auto jj) {
                constexpr int j = decltype(jj)::value;
                p[j] = make_float4(zr[brev<M>(2 * j)] + bv, zi[brev<M>(2 * j)] + bv,
                                   zr[brev<M>(2 * j + 1)] + bv, zi[brev<M>(2 * j + 1)] + bv);
            });
        }
        __syncthreads();
        copy_canvas<N, false, S::THREADS>(smem, out + (x0 + hs * S::TP) * hw, nph * h, w, padL, vec4, tid, h, ppad);
    });
}

// ---------------------------------------------------------------------------------
// host launchers
// ---------------------------------------------------------------------------------
template <int N, int T, bool SMALL>
static size_t rows_lds_bytes(int h, int w)
{
    using S = RowShape<N, T, SMALL>;
    const size_t tile = (size_t)(SMALL ? 16 : N) * S::ROWSTRIDE * sizeof(float2);
    // (+ up to 4 (32 / TP - 1) floats per plane: canvas_plane_pad with this kernel's lane order)
    const size_t canvas = ((size_t)S::TP * (h * Canvas<N>::LDR + 4 * (32 / S::TP - 1)) + Canvas<N>::LDR) * sizeof(float);
    const size_t raw = ((size_t)S::TP * h * w + 3 * N) * sizeof(float);
    const size_t stage = canvas > raw ? canvas : raw;
    return ((tile > stage ? tile : stage) + 15) & ~(size_t)15;
}

// one row per lane, TP planes fastest: 16 lanes are TP planes times 16 / TP consecutive rows
template <int TP>
static int rows_plane_pad(int ldr, int h, int w, int vec4)
{
    static_assert(TP == 2 || TP == 4 || TP == 8 || TP == 16, "planes per staging round");
    if (TP == 16) return canvas_plane_pad(ldr, h, w, vec4, 2, 1);
    return canvas_plane_pad(ldr, h, w, vec4, 32 / TP, 16 / TP);
}

template <int N, int T, bool SMALL>
static FwdJob make_rows_job(const FwdArgs &a)
{
    using S = RowShape<N, T, SMALL>;
    FwdJob j;
    j.in = a.in;
    j.out = reinterpret_cast<float2 *>(a.out);
    j.planes = a.planes;
    j.h = a.h; j.w = a.w; j.padU = a.padU; j.padL = a.padL;
    // every staging round starts TP planes after the previous one: all of them 16-byte aligned
    j.vec4 = ((reinterpret_cast<uintptr_t>(a.in) & 15) == 0) && (((long)S::TP * a.h * a.w) % 4 == 0);
    j.tbl_off = 0;
    j.herm = a.herm;
    j.stream = spectrum_store_mode(a.planes, N);
    j.win = a.win;
    return j;
}

template <int N, int T, int NZ, bool RAW>
static hipError_t launch_fwd_rows(const FwdArgs &a, const FwdArgs *second, hipStream_t s,
                                  const FwdArgs *third = nullptr)
{
    constexpr bool SMALL = NZ < N;
    using S = RowShape<N, T, SMALL>;
    size_t lds = rows_lds_bytes<N, T, SMALL>(a.h, a.w);
    const long blocks0 = plane_group_blocks<T, S::G>(a.planes);
    long blocks = blocks0;
    FwdJob j0 = make_rows_job<N, T, SMALL>(a);
    FwdJob j1 = j0, j2 = j0;
    if (second != nullptr) {
        const size_t lds1 = rows_lds_bytes<N, T, SMALL>(second->h, second->w);
        if (lds1 > lds) lds = lds1;
        blocks += plane_group_blocks<T, S::G>(second->planes);
        j1 = make_rows_job<N, T, SMALL>(*second);
    }
    const long blocks01 = blocks;
    if (third != nullptr) {
        const size_t lds2 = rows_lds_bytes<N, T, SMALL>(third->h, third->w);
        if (lds2 > lds) lds = lds2;
        blocks += plane_group_blocks<T, S::G>(third->planes);
        j2 = make_rows_job<N, T, SMALL>(*third);
    }
    if (blocks > 0x7fffffffL || lds > 160 * 1024) return hipErrorInvalidValue;
    {
        char name[64];
        snprintf(name, sizeof name, "rfft2d_rows_kernel<%d, %d, %d, %s>", N, T, NZ, RAW ? "true" : "false");
        kernel_log_add(name, blocks * S::THREADS);
    }
    FBFC_LAUNCH((rfft2d_rows_kernel<N, T, NZ, RAW>), dim3((unsigned)blocks), dim3(S::THREADS), lds, s, j0, j1,
                       j2, (unsigned)blocks0, (unsigned)blocks01);
    return hipGetLastError();
}

template <int N, int T>
static hipError_t launch_inv_rows(const InvArgs &a, hipStream_t s)
{
    using S = RowShape<N, T>;
    const size_t lds = rows_lds_bytes<N, T, false>(a.h, a.w);
    const long blocks = plane_group_blocks<T, S::G>(a.planes);
    // every copy-out round starts TP planes after the previous one: all of them 16-byte aligned
    const int vec4 = ((reinterpret_cast<uintptr_t>(a.out) & 15) == 0) && (((long)S::TP * a.h * a.w) % 4 == 0);
    const BiasGradJob bgrad = {reinterpret_cast<const float2 *>(a.go_freq), a.grad_bias, a.scale, a.batch,
                               a.out_planes};
    const unsigned bblocks = (bgrad.dc != nullptr) ? bias_grad_dc_blocks(bgrad.planes) : 0u;
    if (blocks + bblocks > 0x7fffffffL || lds > 160 * 1024) return hipErrorInvalidValue;
    {
        char name[64];
        snprintf(name, sizeof name, "irfft2d_rows_kernel<%d, %d>", N, T);
        kernel_log_add(name, (blocks + bblocks) * S::THREADS);
    }
    const int ppad = rows_plane_pad<S::TP>(Canvas<N>::LDR, a.h, a.w, vec4);
    FBFC_LAUNCH((irfft2d_rows_kernel<N, T>), dim3((unsigned)blocks + bblocks), dim3(S::THREADS), lds, s,
                       reinterpret_cast<const float2 *>(a.in), a.out, a.planes, a.h, a.w, a.padU, a.padL, a.bias,
                       a.bias_period > 0 ? a.bias_period : 1, vec4, ppad, bgrad, bblocks);
    return hipGetLastError();
}

// raw staging needs odd plane sizes in every operand of the launch (an even-sized plane staged raw
// puts every row on the same banks)
static bool raw_ok(const FwdArgs &a) { return (a.h & 1) && (a.w & 1); }

// N = 64.  Convolution kernels (planes of at most 16 x 16 at the origin, one operand per launch) take
// 16 planes per workgroup and the variant that skips the zero inputs: its tile has 16 rows and fits
// at once.  Other operands take 8 planes per workgroup (two workgroups per CU, half-line runs).
static hipError_t launch_fwd64(const FwdArgs &a, const FwdArgs *b, hipStream_t s)
{
    const bool raw = raw_ok(a) && (b == nullptr || raw_ok(*b));
    if (b == nullptr && a.h <= 16 && a.w <= 16 && a.padU == 0 && a.padL == 0)
        return raw ? launch_fwd_rows<64, 16, 16, true>(a, nullptr, s) : launch_fwd_rows<64, 16, 16, false>(a, nullptr, s);
    return raw ? launch_fwd_rows<64, 8, 64, true>(a, b, s) : launch_fwd_rows<64, 8, 64, false>(a, b, s);
}

hipError_t launch_rfft2d_large(int N, const FwdArgs &a, const FwdArgs *b, hipStream_t s, const FwdArgs *c)
{
    if (a.win.on || (b != nullptr && b->win.on) || (c != nullptr && (b == nullptr || c->win.on || N != 32)))
        return hipErrorInvalidValue;
    if (N == 32) {
        const bool raw = raw_ok(a) && (b == nullptr || raw_ok(*b)) && (c == nullptr || raw_ok(*c));
        return raw ? launch_fwd_rows<32, 16, 32, true>(a, b, s, c) : launch_fwd_rows<32, 16, 32, false>(a, b, s, c);
    }
    if (N == 64) return launch_fwd64(a, b, s);
    if (N == 128) return launch_fwd_rows<128, 4, 128, false>(a, b, s);
    return hipErrorInvalidValue;
}

hipError_t launch_irfft2d_large(int N, const InvArgs &a, hipStream_t s)
{
    if (a.win.on) return hipErrorInvalidValue;
    // N = 64: results of at most 16 x 16 (the gradWeight crop) have next to nothing to copy out and are all
    // spectrum loads: 16 planes per workgroup read whole lines (24 576 planes of 9 x 9: 105 us against 117 for
    // the two-rows-per-lane kernel; for large results the same kernel is 6-17 % slower than the 8-plane one)
    if (N == 64 && a.h <= 16 && a.w <= 16) return launch_inv_rows<64, 16>(a, s);
    if (N == 64) return launch_inv_rows<64, 8>(a, s);
    if (N == 128) return launch_inv_rows<128, 4>(a, s);
    return hipErrorInvalidValue;
}

template <class K>
static hipError_t raise_lds_limit(K *kernel)
{
    return hipFuncSetAttribute(reinterpret_cast<const void *>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize,
                               160 * 1024);
}

hipError_t fft_large_prepare_device()
{
    hipError_t e = raise_lds_limit(&rfft2d_rows_kernel<64, 8, 64, true>);
    if (e == hipSuccess) e = raise_lds_limit(&rfft2d_rows_kernel<64, 8, 64, false>);
    if (e == hipSuccess) e = raise_lds_limit(&rfft2d_rows_kernel<64, 16, 16, true>);
    if (e == hipSuccess) e = raise_lds_limit(&rfft2d_rows_kernel<64, 16, 16, false>);
    if (e == hipSuccess) e = raise_lds_limit(&irfft2d_rows_kernel<64, 8>);
    if (e == hipSuccess) e = raise_lds_limit(&irfft2d_rows_kernel<64, 16>);
    if (e == hipSuccess) e = raise_lds_limit(&rfft2d_rows_kernel<128, 4, 128, false>);
    if (e == hipSuccess) e = raise_lds_limit(&irfft2d_rows_kernel<128, 4>);
    return e;
}

}  // namespace fbfc
