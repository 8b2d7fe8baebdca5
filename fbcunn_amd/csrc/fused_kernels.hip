// Fused tiled FFT convolution for gfx950: one kernel per pass that transforms the windows of a block of
// tiles, multiplies the spectra and transforms back, without a spectrum of the feature maps ever
// reaching memory.
//
// Replaces what nn.SpatialConvolutionFFTTiledIterated asks of convolveIteratedFFI
// (fbcunn/SpatialConvolutionFFTTiledIterated.lua:79-123, 129-175, 180-229;
// src/fft/FFTIteratedConvolution.cu:23-95): tiles of 8, 16 or 32, the three passes, results those of
// the tiled modules.  Only the weight spectrum (small, shared by every tile) is formed beforehand by the
// ordinary forward transform.
//
// The three-kernel tiled pass writes and reads back batch x tiles x planes spectra (at 3 -> 64 planes,
// 112 x 112, tiles of 16: 302 MB each way for an output of 205 MB); here a workgroup keeps them in LDS
// and registers.  What it gives up is the matrix-core contraction: the sum over the contracted planes is
// vector arithmetic, one lane per (plane, frequency column), so the kernel is for layers in which one
// side has few planes (first and last layers); the tuning front times it against the other candidates.
//
// Naming: the "small" side is the contracted one (input planes in updateOutput, output planes in
// updateGradInput), the "big" side the one the result has (a lane owns one of its planes).
//   * forward batch: up to T windows of the small side (several tiles x several planes) go through the
//     two-rows-per-lane forward transform of fft_kernels.hip (canvas staging, row pass, LDS tile, column
//     pass) and leave their column spectra in an LDS array S[plane][kx][ky];
//   * product: lane (plane t of the big side, tile column kx) sums S[s][kx][.] x W[s][t][.][kx] over the
//     small planes s of the batch into a column spectrum held in registers (S is read by broadcast: all
//     lanes of a column read one address; the weights come from the weight spectrum in global memory, or
//     from registers when the small side has at most three planes);
//   * inverse: that column spectrum is exactly what the column pass of the inverse transform loads from
//     memory in the three-kernel pass, so the inverse transform runs from there (column pass, LDS tile,
//     row pass, bias, canvas staging, windowed store).
// accGradParameters keeps the running sum over tiles and images in registers instead (gradWeight
// spectrum of the lane's planes), transforms back once at the end and leaves a partial k x k result per
// range of tiles, which a second small kernel adds up in a fixed order.
#include <hip/hip_runtime.h>

#include <cstdio>

#include "fft_regs.h"
#include "fft_stage.h"
#include "fft_windows.h"
#include "kernels.h"
#include "store_nt.h"

namespace fbfc {

template <int N>
struct FusedShape {
    static constexpr int T = 512 / N;        // planes per batch: T * N / 2 = 256 lanes
    static constexpr int THREADS = 256;
    static constexpr int NH = N / 2 + 1;
    // LDS tile R[y][kx][t] of the transforms (see fft_kernels.hip); whole tile, one phase
    static constexpr int ROWPAD = (T >= 32) ? 0 : T / 2;
    static constexpr int ROWSTRIDE = (N / 2) * T + ROWPAD;   // complex
    // Column spectra of one small-side plane: [kx in 0..N/2][ky in 0..N) complex.  The plane stride is
    // 1 (mod 32) complex, so the T lanes that write the same (kx, ky) of consecutive planes hit
    // different banks.
    static constexpr int SPLANE = NH * N + (33 - (NH * N) % 32) % 32;
    // entries of a lane's column spectrum: N for an ordinary tile column; the lane of tile slot 0 holds
    // the columns kx = 0 and kx = N/2, rows 0 .. N/2 each (the rows above repeat them as conjugates)
    static constexpr int NE = N + 2;
};

// what a fused launch needs to know about one side's windows
struct FusedSide {
    Window win;      // d1 = planes of this side
    int h, w;        // window (tile) size on the canvas
    int padU, padL;  // inverse only: where the tile sits in the circular result
};

struct FusedJob {
    const float *small;    // real tensor of the contracted side
    float *big;            // real result tensor
    const float2 *wfreq;   // weight spectrum, frequency-major: [ky * NH + kx][f * P + p]
    const float *bias;     // nullptr: none
    FusedSide ss, bs;
    int Ns, Nb;            // planes of the small / big side
    int ws, wb, FP;        // weight plane of (small s, big b) = s * ws + b * wb; FP = F * P
    int vbatch;            // batch * tiles
    // blocking (chosen by the host, see fused_blocking): a group is VBF tiles; the forward batch takes SB small
    // planes of each (nsc chunks cover the small side); product and inverse take VBI tiles x BB big planes
    int VBF, VBI, SB, BB, nsc, nbb, ngroups;
    int bb_in_grid;        // 1: the big block comes from the grid (weights in registers), 0: loop inside
    float alpha;
    int s_off;             // LDS float offset of S; the tables sit behind it
    int tbl_off;
    int s_alias;           // S lies in region 0 (chunked small side: it is consumed before region 0 is used again)
};

// Window table: entry j describes virtual plane (tile vb_first + j / div, plane c0 + j % div); entries
// beyond the valid ones point outside the image, where loads give zero and stores are dropped.
__device__ __forceinline__ void fused_table(int4 *tbl, const Window &win, int slots, int div, int vb_first,
                                            int nvb, int c0, int cmax, int tid)
{
    if (tid < slots) {
        const int q = tid / div, r = tid - q * div;
        const int vb = vb_first + q, c = c0 + r;
        if (q < nvb && c < cmax) {
            const int b = vb / win.nt, tile = vb - b * win.nt;
            const int ty = tile / win.ntx, tx = tile - ty * win.ntx;
            const long off = ((long)b * win.d1 + c) * ((long)win.img_h * win.img_w);
            tbl[tid] = make_int4((int)(unsigned)(off & 0xffffffffL), (int)(off >> 32), ty * win.step_y + win.off_y,
                                 tx * win.step_x + win.off_x);
        } else {
            tbl[tid] = make_int4(0, 0, 0x3fffffff, 0);
        }
    }
}

// Forward transform of the `count` windows listed in tbl: on return lane (j = tid % T, kx = tid / T),
// j < count, holds tile column kx of window j in re / im (X[ky] at position brev(ky); for kx = 0 the
// transform of column 0 + i column N/2).  Region 0 of the LDS is used and must not be touched by
// the caller before its next barrier.
template <int N>
__device__ __forceinline__ void fused_forward(float *smem, const float *in, const int4 *tbl, int count,
                                              const FusedSide &sd, int tid, float (&re)[N], float (&im)[N])
{
    using S = FusedShape<N>;
    constexpr int T = S::T, LDR = Canvas<N>::LDR;
    const int t = tid % T, rp = tid / T;
    const int h = sd.h, w = sd.w;
    const int ya = 2 * rp, yb = ya + 1;
    const bool va = ya < h, vb = yb < h;
    const bool row_active = (t < count) && (va || vb);
    const int pstride = window_plane_stride<N>(h);
    const int zoff = T * pstride;  // an all-zero canvas row behind the staged windows
    if (tid < N) smem[zoff + tid] = 0.0f;
    copy_windows<N, true>(smem, const_cast<float *>(in), tbl, 0, count, h, w, 0, sd.win, tid, pstride);
    __syncthreads();
    if (row_active) {
        const float4 *pa = reinterpret_cast<const float4 *>(smem + (va ? t * pstride + ya * LDR : zoff));
        const float4 *pb = reinterpret_cast<const float4 *>(smem + (vb ? t * pstride + yb * LDR : zoff));
        static_for<N / 4>([&](auto jj) {
            constexpr int j = decltype(jj)::value;
            const float4 a = pa[j], b = pb[j];
            re[4 * j] = a.x; re[4 * j + 1] = a.y; re[4 * j + 2] = a.z; re[4 * j + 3] = a.w;
            im[4 * j] = b.x; im[4 * j + 1] = b.y; im[4 * j + 2] = b.z; im[4 * j + 3] = b.w;
        });
    }
    __syncthreads();  // staging consumed: the tile may overwrite it
    float2 *R = reinterpret_cast<float2 *>(smem);
    if (row_active) {
        fft_inplace<N, false>(re, im);
        float2 *Ra = R + ya * S::ROWSTRIDE + t;
        float2 *Rb = Ra + S::ROWSTRIDE;
        Ra[0] = make_float2(re[brev<N>(0)], re[brev<N>(N / 2)]);
        Rb[0] = make_float2(im[brev<N>(0)], im[brev<N>(N / 2)]);
        static_for<N / 2 - 1>([&](auto kk) {
            constexpr int k = decltype(kk)::value + 1;
            const float zr = re[brev<N>(k)], zi = im[brev<N>(k)];
            const float nr = re[brev<N>(N - k)], ni = im[brev<N>(N - k)];
            Ra[k * T] = make_float2(0.5f * (zr + nr), 0.5f * (zi - ni));
            Rb[k * T] = make_float2(0.5f * (zi + ni), 0.5f * (nr - zr));
        });
    } else if (t < count) {
        float2 *Ra = R + ya * S::ROWSTRIDE + t;
        float2 *Rb = Ra + S::ROWSTRIDE;
        static_for<N / 2>([&](auto kk) {
            constexpr int k = decltype(kk)::value;
            Ra[k * T] = make_float2(0.0f, 0.0f);
            Rb[k * T] = make_float2(0.0f, 0.0f);
        });
    }
    __syncthreads();
    if (t < count) {
        const float2 *col = R + rp * T + t;
        static_for<N>([&](auto yy) {
            constexpr int y = decltype(yy)::value;
            const float2 v = col[y * S::ROWSTRIDE];
            re[y] = v.x;
            im[y] = v.y;
        });
        fft_inplace<N, false>(re, im);
    }
}

// A column held as re / im (fused_forward's result) in entry order: entry e of an ordinary column is
// X[ky = e]; the slot-0 lane untangles its two columns into entries e <= N/2 (kx = 0, ky = e) and
// e = N/2 + 1 + ky (kx = N/2).  Entries N, N + 1 of an ordinary column are zero.
template <int N>
__device__ __forceinline__ void column_entries(const float (&re)[N], const float (&im)[N], bool slot0,
                                               float (&er)[N + 2], float (&ei)[N + 2])
{
    if (!slot0) {
        static_for<N>([&](auto kk) {
            constexpr int ky = decltype(kk)::value;
            er[ky] = re[brev<N>(ky)];
            ei[ky] = im[brev<N>(ky)];
        });
        er[N] = er[N + 1] = ei[N] = ei[N + 1] = 0.0f;
    } else {
        static_for<N / 2 + 1>([&](auto kk) {
            constexpr int ky = decltype(kk)::value;
            constexpr int kn = (N - ky) % N;
            const float zr = re[brev<N>(ky)], zi = im[brev<N>(ky)];
            const float nr = re[brev<N>(kn)], ni = im[brev<N>(kn)];
            er[ky] = 0.5f * (zr + nr);              ei[ky] = 0.5f * (zi - ni);
            er[N / 2 + 1 + ky] = 0.5f * (zi + ni);  ei[N / 2 + 1 + ky] = 0.5f * (nr - zr);
        });
    }
}

// where entry e of a lane's column lies in an S plane: (e <= N/2 ? lo : hi) + e complex
template <int N>
struct EntryMap {
    int lo, hi;       // S offsets
    int col_lo, col_hi, dhi;  // weight spectrum: column of the entry, row = e + (e > N/2 ? dhi : 0)
    __device__ __forceinline__ EntryMap(int kx)
    {
        if (kx != 0) {
            lo = hi = kx * N;
            col_lo = col_hi = kx;
            dhi = 0;
        } else {
            lo = 0;
            hi = (N / 2) * N - (N / 2 + 1);
            col_lo = 0;
            col_hi = N / 2;
            dhi = -(N / 2 + 1);
        }
    }
    template <int E>
    __device__ __forceinline__ int s_off() const { return (E <= N / 2 ? lo : hi) + E; }
    // index of the entry's frequency in the weight spectrum; the two spare entries of an ordinary column
    // stay inside the buffer (their products are never used)
    template <int E>
    __device__ __forceinline__ int w_freq() const
    {
        constexpr int NH = N / 2 + 1;
        if constexpr (E <= N / 2) return E * NH + col_lo;
        int row = E + dhi;
        if constexpr (E >= N) row = row > N - 1 ? N - 1 : row;
        return row * NH + col_hi;
    }
};

template <int N>
__device__ __forceinline__ void store_column_to_S(float2 *sp, int kx, const float (&re)[N], const float (&im)[N])
{
    float er[N + 2], ei[N + 2];
    column_entries<N>(re, im, kx == 0, er, ei);
    const EntryMap<N> em(kx);
    static_for<N + 2>([&](auto ee) {
        constexpr int e = decltype(ee)::value;
        // an ordinary column has N entries; the last two slots belong to the next column
        if (e < N || kx == 0) sp[em.template s_off<e>()] = make_float2(er[e], ei[e]);
    });
}

// Inverse transform of the column spectra the lanes hold (entry order, already scaled) and windowed store.
// valid: this lane's plane exists.  bias_v: added to every element of the plane.
template <int N>
__device__ __forceinline__ void fused_inverse(float *smem, float *out, const int4 *tbl, const FusedSide &sd, int tid,
                                              bool valid, float bias_v, const float (&er)[N + 2],
                                              const float (&ei)[N + 2])
{
    using S = FusedShape<N>;
    constexpr int T = S::T, LDR = Canvas<N>::LDR;
    const int t = tid % T, kx = tid / T;
    float2 *R = reinterpret_cast<float2 *>(smem);
    float re[N], im[N];
    if (valid) {
        if (kx != 0) {
            static_for<N>([&](auto kk) {
                constexpr int ky = decltype(kk)::value;
                re[ky] = er[ky];
                im[ky] = ei[ky];
            });
        } else {
            // pack columns 0 and N/2 (each the spectrum of a real sequence): C = X0 + i XN
            static_for<N / 2 + 1>([&](auto kk) {
                constexpr int ky = decltype(kk)::value;
                const float ax = er[ky], ay = ei[ky], bx = er[N / 2 + 1 + ky], by = ei[N / 2 + 1 + ky];
                re[ky] = ax - by;
                im[ky] = ay + bx;
                if constexpr (ky > 0 && ky < N / 2) {
                    re[N - ky] = ax + by;
                    im[N - ky] = bx - ay;
                }
            });
        }
        fft_inplace<N, true>(re, im);
        float2 *col = R + kx * T + t;
        static_for<N>([&](auto yy) {
            constexpr int y = decltype(yy)::value;
            col[y * S::ROWSTRIDE] = make_float2(re[brev<N>(y)], im[brev<N>(y)]);
        });
    }
    __syncthreads();
    const int rp = kx;
    const int ya = 2 * rp, yb = ya + 1;
    const int ia = ya - sd.padU, ib = yb - sd.padU;
    const bool va = (ia >= 0) && (ia < sd.h), vb = (ib >= 0) && (ib < sd.h);
    const bool row_active = valid && (va || vb);
    float zr[N], zi[N];
    if (row_active) {
        const float2 *Ra = R + ya * S::ROWSTRIDE + t;
        const float2 *Rb = Ra + S::ROWSTRIDE;
        static_for<N / 2>([&](auto kk) {
            constexpr int k = decltype(kk)::value;
            const float2 a = Ra[k * T], b = Rb[k * T];
            if constexpr (k == 0) {
                zr[0] = a.x;      zi[0] = b.x;
                zr[N / 2] = a.y;  zi[N / 2] = b.y;
            } else {
                zr[k] = a.x - b.y;      zi[k] = a.y + b.x;
                zr[N - k] = a.x + b.y;  zi[N - k] = b.x - a.y;
            }
        });
    }
    __syncthreads();  // tile consumed: the staging area may overwrite it
    const int pstride = window_plane_stride<N>(sd.h);
    if (row_active) {
        fft_inplace<N, true>(zr, zi);
        if (va) {
            float4 *pa = reinterpret_cast<float4 *>(smem + t * pstride + ia * LDR);
            static_for<N / 4>([&](auto jj) {
                constexpr int j = decltype(jj)::value;
                pa[j] = make_float4(zr[brev<N>(4 * j)] + bias_v, zr[brev<N>(4 * j + 1)] + bias_v,
                                    zr[brev<N>(4 * j + 2)] + bias_v, zr[brev<N>(4 * j + 3)] + bias_v);
            });
        }
        if (vb) {
            float4 *pb = reinterpret_cast<float4 *>(smem + t * pstride + ib * LDR);
            static_for<N / 4>([&](auto jj) {
                constexpr int j = decltype(jj)::value;
                pb[j] = make_float4(zi[brev<N>(4 * j)] + bias_v, zi[brev<N>(4 * j + 1)] + bias_v,
                                    zi[brev<N>(4 * j + 2)] + bias_v, zi[brev<N>(4 * j + 3)] + bias_v);
            });
        }
    }
    __syncthreads();
    copy_windows<N, false>(smem, out, tbl, 0, T, sd.h, sd.w, sd.padL, sd.win, tid, pstride);
}

// ---------------------------------------------------------------------------------------------------
// updateOutput (CONJ: O = sum_p I conj(W)) and updateGradInput (GI = sum_f GO W)
// ---------------------------------------------------------------------------------------------------
// WREG > 0: the small side has at most WREG planes, the big block comes from the grid and the lane keeps
// its weights (WREG x NE complex) in registers for all the tiles it works on.
template <int N, bool CONJ, int WREG>
__global__ __launch_bounds__(256, (N >= 32 ? 1 : 2)) void fused_conv_kernel(FusedJob jb)
{
    using S = FusedShape<N>;
    constexpr int T = S::T, NE = S::NE;
    extern __shared__ __align__(16) float smem[];
    float2 *Sbuf = reinterpret_cast<float2 *>(smem + jb.s_off);
    int4 *tbl_s = reinterpret_cast<int4 *>(smem + jb.tbl_off);
    int4 *tbl_b = tbl_s + T;
    const int tid = threadIdx.x;
    const int t = tid % T, kx = tid / T;
    const EntryMap<N> em(kx);
    // product / inverse role of the lane: tile vl of the sub-group, big plane bi of the block
    const int vl = t / jb.BB, bi = t - vl * jb.BB;

    int bb_first = 0, bb_last = jb.nbb, gw = blockIdx.x, ngw = gridDim.x;
    if (jb.bb_in_grid) {
        bb_first = (int)(blockIdx.x % (unsigned)jb.nbb);
        bb_last = bb_first + 1;
        gw = (int)(blockIdx.x / (unsigned)jb.nbb);
        ngw = (int)(gridDim.x / (unsigned)jb.nbb);
    }

    [[maybe_unused]] float wr[WREG > 0 ? WREG : 1][NE], wi[WREG > 0 ? WREG : 1][NE];
    if constexpr (WREG > 0) {
        const int b = bb_first * jb.BB + bi;
        const bool ok = vl < jb.VBI && b < jb.Nb;
        static_for<WREG>([&](auto ss) {
            constexpr int s = decltype(ss)::value;
            static_for<NE>([&](auto ee) {
                constexpr int e = decltype(ee)::value;
                float2 v = make_float2(0.0f, 0.0f);
                if (ok && s < jb.Ns) v = jb.wfreq[(long)em.template w_freq<e>() * jb.FP + s * jb.ws + b * jb.wb];
                wr[s][e] = v.x;
                wi[s][e] = v.y;
            });
        });
    }

    for (int g = gw; g < jb.ngroups; g += ngw) {
        const int vb0 = g * jb.VBF;
        const int nvb = (jb.vbatch - vb0 < jb.VBF) ? (jb.vbatch - vb0) : jb.VBF;
        // one chunk of the small side covers it (nsc == 1): transform once, then every big block and
        // sub-group of tiles multiplies from S.  Otherwise (VBF == VBI) the product runs chunk by chunk.
        const int nsub = (jb.nsc == 1) ? (nvb + jb.VBI - 1) / jb.VBI : 1;
        for (int bb = bb_first; bb < bb_last; ++bb) {
            const int b0 = bb * jb.BB;
            for (int sub = 0; sub < nsub; ++sub) {
                const int vsub = vb0 + sub * jb.VBI;
                const int nvs = (nvb - sub * jb.VBI < jb.VBI) ? (nvb - sub * jb.VBI) : jb.VBI;
                const bool valid = vl < nvs && bi < jb.BB && b0 + bi < jb.Nb;
                float ar[NE], ai[NE];
                static_for<NE>([&](auto ee) {
                    constexpr int e = decltype(ee)::value;
                    ar[e] = 0.0f;
                    ai[e] = 0.0f;
                });
                for (int sc = 0; sc < jb.nsc; ++sc) {
                    const int s0 = sc * jb.SB;
                    const int ns = (jb.Ns - s0 < jb.SB) ? (jb.Ns - s0) : jb.SB;
                    // ---- forward batch (once per group when one chunk covers the small side) ----
                    if (jb.nsc > 1 || (bb == bb_first && sub == 0)) {
                        __syncthreads();  // region 0, S and the tables are free
                        fused_table(tbl_s, jb.ss.win, T, ns, vb0, nvb, s0, jb.Ns, tid);
                        __syncthreads();
                        float re[N], im[N];
                        const int count = nvb * ns;
                        fused_forward<N>(smem, jb.small, tbl_s, count, jb.ss, tid, re, im);
                        if (jb.s_alias) __syncthreads();  // every column has left the tile S is about to overwrite
                        if (t < count) store_column_to_S<N>(Sbuf + t * S::SPLANE, kx, re, im);
                        __syncthreads();
                    }
                    // ---- product: small planes s0 .. s0 + ns of tile (sub * VBI + vl) ----
                    if (valid) {
                        const float2 *sp = Sbuf + (((jb.nsc == 1) ? sub * jb.VBI : 0) + vl) * ns * S::SPLANE;
                        auto mac = [&](auto ee, float sr, float si, float xr, float xi) {
                            constexpr int e = decltype(ee)::value;
                            if constexpr (CONJ) {   // s conj(w)
                                ar[e] = __builtin_fmaf(sr, xr, __builtin_fmaf(si, xi, ar[e]));
                                ai[e] = __builtin_fmaf(si, xr, __builtin_fmaf(-sr, xi, ai[e]));
                            } else {                // s w
                                ar[e] = __builtin_fmaf(sr, xr, __builtin_fmaf(-si, xi, ar[e]));
                                ai[e] = __builtin_fmaf(sr, xi, __builtin_fmaf(si, xr, ai[e]));
                            }
                        };
                        if constexpr (WREG > 0) {
                            static_for<WREG>([&](auto ss) {
                                constexpr int s = decltype(ss)::value;
                                if (s < ns) {
                                    static_for<NE>([&](auto ee) {
                                        constexpr int e = decltype(ee)::value;
                                        const float2 v = sp[s * S::SPLANE + em.template s_off<e>()];
                                        mac(ee, v.x, v.y, wr[s][e], wi[s][e]);
                                    });
                                }
                            });
                        } else {
                            const float2 *wq = jb.wfreq + (long)(b0 + bi) * jb.wb + (long)s0 * jb.ws;
                            for (int s = 0; s < ns; ++s) {
                                static_for<NE>([&](auto ee) {
                                    constexpr int e = decltype(ee)::value;
                                    const float2 v = sp[s * S::SPLANE + em.template s_off<e>()];
                                    const float2 x = wq[(long)em.template w_freq<e>() * jb.FP + (long)s * jb.ws];
                                    mac(ee, v.x, v.y, x.x, x.y);
                                });
                            }
                        }
                    }
                }
                // ---- inverse and windowed store of VBI tiles x BB big planes ----
                __syncthreads();  // region 0 is free (forward batch done; the previous store has been read out)
                fused_table(tbl_b, jb.bs.win, T, jb.BB, vsub, nvs, b0, jb.Nb, tid);
                static_for<NE>([&](auto ee) {
                    constexpr int e = decltype(ee)::value;
                    ar[e] *= jb.alpha;
                    ai[e] *= jb.alpha;
                });
                const float bias_v = (valid && jb.bias != nullptr) ? jb.bias[b0 + bi] : 0.0f;
                __syncthreads();  // table complete
                fused_inverse<N>(smem, jb.big, tbl_b, jb.bs, tid, valid, bias_v, ar, ai);
            }
        }
    }
}

// ---------------------------------------------------------------------------------------------------
// accGradParameters: GW[f][p] = sum over tiles and images of conj(GO[f]) I[p]
// ---------------------------------------------------------------------------------------------------
// The lane owns plane t of the big side (the side with more planes: gradOutput or input) and keeps the
// running sums for PCA planes of the other side in registers.  A workgroup = (block of T big planes,
// chunk of PCA small planes, range of tiles); its k x k results go to part[range][f][p].
struct FusedAccJob {
    const float *small, *big;   // real tensors: the side held in S (PCA planes at a time) / the lanes' side
    float *part;                // [nranges][F][P][kh][kw]
    FusedSide ss, bs;           // windows of the small / big side
    int Ns, Nb;
    int big_is_go;              // 1: big = gradOutput (conj on the lanes' columns), 0: big = input (conj on S)
    int F, P, kh, kw;
    int vbatch, nranges, VBS;   // tiles; ranges they are split into; tiles per forward batch of the small side
    int nbb, nsc;               // blocks of T big planes, chunks of PCA small planes
    float alpha;
    int s_off, tbl_off;
};

template <int N, int PCA>
__global__ __launch_bounds__(256, (N >= 32 ? 1 : 2)) void fused_accgrad_kernel(FusedAccJob jb)
{
    using S = FusedShape<N>;
    constexpr int T = S::T, NE = S::NE;
    extern __shared__ __align__(16) float smem[];
    float2 *Sbuf = reinterpret_cast<float2 *>(smem + jb.s_off);
    int4 *tbl_s = reinterpret_cast<int4 *>(smem + jb.tbl_off);
    int4 *tbl_b = tbl_s + T;
    const int tid = threadIdx.x;
    const int t = tid % T, kx = tid / T;
    const EntryMap<N> em(kx);
    unsigned w = blockIdx.x;
    const int bb = (int)(w % (unsigned)jb.nbb);
    w /= (unsigned)jb.nbb;
    const int sc = (int)(w % (unsigned)jb.nsc);
    const int range = (int)(w / (unsigned)jb.nsc);
    const int b0 = bb * T, s0 = sc * PCA;
    const int ns = (jb.Ns - s0 < PCA) ? (jb.Ns - s0) : PCA;
    const bool valid = b0 + t < jb.Nb;
    // tiles [v_first, v_last) of this range
    const int per = (jb.vbatch + jb.nranges - 1) / jb.nranges;
    const int v_first = range * per;
    const int v_last = (v_first + per < jb.vbatch) ? v_first + per : jb.vbatch;

    float ar[PCA][NE], ai[PCA][NE];
    static_for<PCA>([&](auto ss) {
        static_for<NE>([&](auto ee) {
            ar[decltype(ss)::value][decltype(ee)::value] = 0.0f;
            ai[decltype(ss)::value][decltype(ee)::value] = 0.0f;
        });
    });

    for (int v0 = v_first; v0 < v_last; v0 += jb.VBS) {
        const int nv = (v_last - v0 < jb.VBS) ? (v_last - v0) : jb.VBS;
        // ---- small side: nv tiles x ns planes into S ----
        __syncthreads();
        fused_table(tbl_s, jb.ss.win, T, ns, v0, nv, s0, jb.Ns, tid);
        __syncthreads();
        {
            float re[N], im[N];
            const int count = nv * ns;
            fused_forward<N>(smem, jb.small, tbl_s, count, jb.ss, tid, re, im);
            if (t < count) store_column_to_S<N>(Sbuf + t * S::SPLANE, kx, re, im);
        }
        // ---- big side, one tile at a time: T planes of tile v ----
        for (int vi = 0; vi < nv; ++vi) {
            __syncthreads();  // region 0 free; S complete (first round)
            fused_table(tbl_b, jb.bs.win, T, T, v0 + vi, 1, b0, jb.Nb, tid);
            __syncthreads();
            float re[N], im[N];
            const int count = (jb.Nb - b0 < T) ? (jb.Nb - b0) : T;
            fused_forward<N>(smem, jb.big, tbl_b, count, jb.bs, tid, re, im);
            if (valid) {
                float cr[NE], ci[NE];
                column_entries<N>(re, im, kx == 0, cr, ci);
                const float2 *sp = Sbuf + vi * ns * S::SPLANE;
                static_for<PCA>([&](auto ss) {
                    constexpr int s = decltype(ss)::value;
                    if (s < ns) {
                        static_for<NE>([&](auto ee) {
                            constexpr int e = decltype(ee)::value;
                            const float2 q = sp[s * S::SPLANE + em.template s_off<e>()];
                            // gradOutput's spectrum is the conjugated factor
                            const float gr = jb.big_is_go ? cr[e] : q.x, gi = jb.big_is_go ? ci[e] : q.y;
                            const float xr = jb.big_is_go ? q.x : cr[e], xi = jb.big_is_go ? q.y : ci[e];
                            ar[s][e] = __builtin_fmaf(gr, xr, __builtin_fmaf(gi, xi, ar[s][e]));
                            ai[s][e] = __builtin_fmaf(gr, xi, __builtin_fmaf(-gi, xr, ai[s][e]));
                        });
                    }
                });
            }
        }
    }

    // ---- back to the k x k kernels: inverse transform of each (big plane, small plane) sum ----
    float2 *R = reinterpret_cast<float2 *>(smem);
    static_for<PCA>([&](auto ss) {
        constexpr int s = decltype(ss)::value;
        if (s < ns) {   // uniform over the workgroup
            __syncthreads();
            float re[N], im[N];
            if (valid) {
                if (kx != 0) {
                    static_for<N>([&](auto kk) {
                        constexpr int ky = decltype(kk)::value;
                        re[ky] = ar[s][ky] * jb.alpha;
                        im[ky] = ai[s][ky] * jb.alpha;
                    });
                } else {
                    static_for<N / 2 + 1>([&](auto kk) {
                        constexpr int ky = decltype(kk)::value;
                        const float ax = ar[s][ky] * jb.alpha, ay = ai[s][ky] * jb.alpha;
                        const float bx = ar[s][N / 2 + 1 + ky] * jb.alpha, by = ai[s][N / 2 + 1 + ky] * jb.alpha;
                        re[ky] = ax - by;
                        im[ky] = ay + bx;
                        if constexpr (ky > 0 && ky < N / 2) {
                            re[N - ky] = ax + by;
                            im[N - ky] = bx - ay;
                        }
                    });
                }
                fft_inplace<N, true>(re, im);
                float2 *col = R + kx * T + t;
                static_for<N>([&](auto yy) {
                    constexpr int y = decltype(yy)::value;
                    col[y * S::ROWSTRIDE] = make_float2(re[brev<N>(y)], im[brev<N>(y)]);
                });
            }
            __syncthreads();
            const int ya = 2 * kx, yb = ya + 1;
            if (valid && ya < jb.kh) {
                float zr[N], zi[N];
                const float2 *Ra = R + ya * S::ROWSTRIDE + t;
                const float2 *Rb = Ra + S::ROWSTRIDE;
                static_for<N / 2>([&](auto kk) {
                    constexpr int k = decltype(kk)::value;
                    const float2 a = Ra[k * T], b = Rb[k * T];
                    if constexpr (k == 0) {
                        zr[0] = a.x;      zi[0] = b.x;
                        zr[N / 2] = a.y;  zi[N / 2] = b.y;
                    } else {
                        zr[k] = a.x - b.y;      zi[k] = a.y + b.x;
                        zr[N - k] = a.x + b.y;  zi[N - k] = b.x - a.y;
                    }
                });
                fft_inplace<N, true>(zr, zi);
                const int f = jb.big_is_go ? b0 + t : s0 + s;
                const int p = jb.big_is_go ? s0 + s : b0 + t;
                float *dst = jb.part + (((long)range * jb.F + f) * jb.P + p) * (jb.kh * jb.kw);
                static_for<N>([&](auto cc) {
                    constexpr int c = decltype(cc)::value;
                    if (c < jb.kw) {
                        dst[ya * jb.kw + c] = zr[brev<N>(c)];
                        if (yb < jb.kh) dst[yb * jb.kw + c] = zi[brev<N>(c)];
                    }
                });
            }
        }
    });
}

// gradWeight[i] = sum over ranges of part[range][i], in a fixed order.  A workgroup takes 64 elements; its four
// waves each sum every fourth range with four independent chains (a lane summing all ranges one after the
// other waited for one load at a time: 60 us for 256 ranges), and the partial sums meet in LDS.
__global__ __launch_bounds__(256) void fused_accgrad_sum_kernel(const float *__restrict__ part, float *__restrict__ gw,
                                                                long n, int nranges)
{
    __shared__ float red[4][64];
    const int e = threadIdx.x & 63, sl = threadIdx.x >> 6;
    const long i = (long)blockIdx.x * 64 + e;
    float a[4] = {0.0f, 0.0f, 0.0f, 0.0f};
    if (i < n) {
        int r = sl;
        for (; r + 12 < nranges; r += 16) {
#pragma unroll
            for (int u = 0; u < 4; ++u) a[u] += part[(long)(r + 4 * u) * n + i];
        }
        for (; r < nranges; r += 4) a[0] += part[(long)r * n + i];
    }
    red[sl][e] = (a[0] + a[1]) + (a[2] + a[3]);
    __syncthreads();
    if (sl == 0 && i < n) gw[i] = (red[0][e] + red[1][e]) + (red[2][e] + red[3][e]);
}

// ---------------------------------------------------------------------------------------------------
// host side
// ---------------------------------------------------------------------------------------------------
template <int N>
static size_t fused_region0_floats(int h_small, int h_big)
{
    using S = FusedShape<N>;
    const size_t tile = (size_t)2 * N * S::ROWSTRIDE;
    const int h = h_small > h_big ? h_small : h_big;
    const size_t stage = (size_t)S::T * (h * Canvas<N>::LDR + 4) + Canvas<N>::LDR;
    return ((tile > stage ? tile : stage) + 3) & ~(size_t)3;
}

// LDS bytes the S array may take: what half a CU's LDS leaves beside the fixed part if the smallest S fits
// there (two workgroups per CU), otherwise what the whole LDS leaves
static long fused_s_budget(size_t fixed_bytes, size_t smallest_s_bytes)
{
    const long half = 80L * 1024 - (long)fixed_bytes, whole = 160L * 1024 - (long)fixed_bytes;
    return half >= (long)smallest_s_bytes ? half : whole;
}

// largest power of two <= v (v >= 1)
static int pow2_floor(int v)
{
    int p = 1;
    while (2 * p <= v) p *= 2;
    return p;
}

template <int N, bool CONJ>
static hipError_t launch_fused_conv_n(FusedJob jb, int wreg_ok, hipStream_t s)
{
    using S = FusedShape<N>;
    constexpr int T = S::T;
    // blocking: BB big planes x VBI tiles share the T plane slots of product and inverse; if the whole small
    // side of VBI tiles fits one forward batch it is transformed once per group of VBF tiles (a multiple of
    // VBI), otherwise chunk by chunk for VBF = VBI tiles
    jb.BB = jb.Nb < T ? jb.Nb : T;
    jb.VBI = pow2_floor(T / jb.BB);
    jb.nbb = (jb.Nb + jb.BB - 1) / jb.BB;
    const size_t r0 = fused_region0_floats<N>(jb.ss.h, jb.bs.h);
    size_t s_planes;
    if ((long)jb.Ns * jb.VBI <= T) {
        jb.SB = jb.Ns;
        jb.nsc = 1;
        jb.VBF = (T / jb.Ns) / jb.VBI * jb.VBI;
        // two workgroups per CU if a smaller group allows it
        const long budget = fused_s_budget(2 * T * sizeof(int4) + r0 * sizeof(float),
                                           (size_t)jb.VBI * jb.Ns * S::SPLANE * sizeof(float2));
        while (jb.VBF > jb.VBI && (long)jb.VBF * jb.Ns * S::SPLANE * (long)sizeof(float2) > budget) jb.VBF -= jb.VBI;
        s_planes = (size_t)jb.VBF * jb.Ns;
    } else {
        jb.VBF = jb.VBI;
        jb.SB = T / jb.VBF;
        jb.nsc = (jb.Ns + jb.SB - 1) / jb.SB;
        s_planes = (size_t)jb.VBF * jb.SB;
        jb.s_alias = 1;
    }
    jb.ngroups = (jb.vbatch + jb.VBF - 1) / jb.VBF;
    if (jb.s_alias) {
        // each chunk's spectra are multiplied before the next transform or the inverse touches region 0:
        // S shares it, and two workgroups fit a CU
        jb.s_off = 0;
        const size_t sfl = s_planes * S::SPLANE * 2;
        jb.tbl_off = (int)(sfl > r0 ? sfl : r0);
    } else {
        jb.s_off = (int)r0;
        jb.tbl_off = (int)(r0 + s_planes * S::SPLANE * 2);
    }
    jb.tbl_off = (jb.tbl_off + 3) & ~3;
    const size_t lds = (size_t)jb.tbl_off * sizeof(float) + 2 * T * sizeof(int4);
    if (lds > 160 * 1024) return hipErrorInvalidValue;
    // weights in registers: a small side of at most three planes at N <= 16, all in one chunk
    const bool wreg = wreg_ok && N <= 16 && jb.nsc == 1 && jb.Ns <= 3;
    jb.bb_in_grid = wreg ? 1 : 0;
    long per_bb = jb.ngroups;
    const long cap = 2048 / (wreg ? jb.nbb : 1);
    if (per_bb > cap) per_bb = cap > 0 ? cap : 1;
    const long grid = wreg ? per_bb * jb.nbb : per_bb;
    char name[64];
    snprintf(name, sizeof name, "fused_conv_kernel<%d, %s, %d>", N, CONJ ? "true" : "false", wreg ? 3 : 0);
    kernel_log_add(name, grid * 256);
    if (wreg) FBFC_LAUNCH((fused_conv_kernel<N, CONJ, (N <= 16 ? 3 : 0)>), dim3((unsigned)grid), dim3(256), lds, s, jb);
    else FBFC_LAUNCH((fused_conv_kernel<N, CONJ, 0>), dim3((unsigned)grid), dim3(256), lds, s, jb);
    return hipGetLastError();
}

static FusedSide make_side(const Window &win, int h, int w, int padU, int padL)
{
    FusedSide sd;
    sd.win = win;
    sd.win.remap = 0;
    sd.h = h;
    sd.w = w;
    sd.padU = padU;
    sd.padL = padL;
    return sd;
}

hipError_t launch_fused_conv(int N, const FusedConvArgs &a, hipStream_t s)
{
    if (a.vbatch <= 0 || a.n_small <= 0 || a.n_big <= 0 || !a.small_win.on || !a.big_win.on)
        return hipErrorInvalidValue;
    if (a.small_h > N || a.small_w > N || a.big_h + a.big_pad_u > N || a.big_w + a.big_pad_l > N) return hipErrorInvalidValue;
    FusedJob jb = {};
    jb.small = a.small;
    jb.big = a.big;
    jb.wfreq = reinterpret_cast<const float2 *>(a.w_freq);
    jb.bias = a.bias;
    jb.ss = make_side(a.small_win, a.small_h, a.small_w, 0, 0);
    jb.bs = make_side(a.big_win, a.big_h, a.big_w, a.big_pad_u, a.big_pad_l);
    jb.Ns = a.n_small;
    jb.Nb = a.n_big;
    jb.ws = a.w_stride_small;
    jb.wb = a.w_stride_big;
    jb.FP = a.out_planes * a.in_planes;
    jb.vbatch = a.vbatch;
    jb.alpha = a.alpha;
    const int wreg_ok = 1;
    switch (N) {
        case 8: return a.conj_w ? launch_fused_conv_n<8, true>(jb, wreg_ok, s) : launch_fused_conv_n<8, false>(jb, wreg_ok, s);
        case 16: return a.conj_w ? launch_fused_conv_n<16, true>(jb, wreg_ok, s) : launch_fused_conv_n<16, false>(jb, wreg_ok, s);
        case 32: return a.conj_w ? launch_fused_conv_n<32, true>(jb, wreg_ok, s) : launch_fused_conv_n<32, false>(jb, wreg_ok, s);
        default: return hipErrorInvalidValue;
    }
}

template <int N>
struct AccChunk {
    static constexpr int PCA = (N == 8) ? 6 : (N == 16) ? 3 : 1;  // small planes whose sums a lane keeps
};

int fused_accgrad_ranges(int N, int vbatch, int out_planes, int in_planes)
{
    const int T = 512 / N;
    const int pca = (N == 8) ? 6 : (N == 16) ? 3 : 1;
    const int nb = out_planes > in_planes ? out_planes : in_planes;
    const int ns = out_planes > in_planes ? in_planes : out_planes;
    const long blocks = (long)((nb + T - 1) / T) * ((ns + pca - 1) / pca);
    long r = 512 / blocks;  // two workgroups per CU, which is what the registers allow
    if (r < 1) r = 1;
    if (r > 512) r = 512;
    if (r > vbatch) r = vbatch;
    return (int)r;
}

template <int N>
static hipError_t launch_fused_accgrad_n(FusedAccJob jb, hipStream_t s)
{
    using S = FusedShape<N>;
    constexpr int T = S::T, PCA = AccChunk<N>::PCA;
    jb.nbb = (jb.Nb + T - 1) / T;
    jb.nsc = (jb.Ns + PCA - 1) / PCA;
    const int ns_max = jb.Ns < PCA ? jb.Ns : PCA;
    const size_t r0 = fused_region0_floats<N>(jb.ss.h, jb.bs.h);
    jb.VBS = T / ns_max;
    const long budget = fused_s_budget(2 * T * sizeof(int4) + r0 * sizeof(float),
                                       (size_t)ns_max * S::SPLANE * sizeof(float2));
    while (jb.VBS > 1 && (long)jb.VBS * ns_max * S::SPLANE * (long)sizeof(float2) > budget) --jb.VBS;
    jb.s_off = (int)r0;
    jb.tbl_off = (int)(r0 + (size_t)jb.VBS * ns_max * S::SPLANE * 2);
    jb.tbl_off = (jb.tbl_off + 3) & ~3;
    const size_t lds = (size_t)jb.tbl_off * sizeof(float) + 2 * T * sizeof(int4);
    if (lds > 160 * 1024) return hipErrorInvalidValue;
    const long grid = (long)jb.nbb * jb.nsc * jb.nranges;
    if (grid > 0x7fffffffL) return hipErrorInvalidValue;
    char name[64];
    snprintf(name, sizeof name, "fused_accgrad_kernel<%d, %d>", N, PCA);
    kernel_log_add(name, grid * 256);
    FBFC_LAUNCH((fused_accgrad_kernel<N, PCA>), dim3((unsigned)grid), dim3(256), lds, s, jb);
    return hipGetLastError();
}

template <class K>
static hipError_t raise_lds_limit(K *kernel)
{
    return hipFuncSetAttribute(reinterpret_cast<const void *>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize,
                               160 * 1024);
}

template <int N>
static hipError_t fused_prepare_n()
{
    hipError_t e = raise_lds_limit(&fused_conv_kernel<N, true, 0>);
    if (e == hipSuccess) e = raise_lds_limit(&fused_conv_kernel<N, false, 0>);
    if constexpr (N <= 16) {
        if (e == hipSuccess) e = raise_lds_limit(&fused_conv_kernel<N, true, 3>);
        if (e == hipSuccess) e = raise_lds_limit(&fused_conv_kernel<N, false, 3>);
    }
    if (e == hipSuccess) e = raise_lds_limit(&fused_accgrad_kernel<N, AccChunk<N>::PCA>);
    return e;
}

hipError_t fused_prepare_device()
{
    hipError_t e = fused_prepare_n<8>();
    if (e == hipSuccess) e = fused_prepare_n<16>();
    if (e == hipSuccess) e = fused_prepare_n<32>();
    return e;
}

hipError_t launch_fused_accgrad(int N, const FusedAccArgs &a, hipStream_t s)
{
    if (a.vbatch <= 0 || a.out_planes <= 0 || a.in_planes <= 0 || !a.in_win.on || !a.go_win.on || a.nranges < 1)
        return hipErrorInvalidValue;
    if (a.in_h > N || a.in_w > N || a.go_h > N || a.go_w > N || a.kh > N || a.kw > N) return hipErrorInvalidValue;
    FusedAccJob jb = {};
    const bool big_is_go = a.out_planes >= a.in_planes;
    const FusedSide go = make_side(a.go_win, a.go_h, a.go_w, 0, 0), in = make_side(a.in_win, a.in_h, a.in_w, 0, 0);
    jb.big = big_is_go ? a.grad_output : a.input;
    jb.small = big_is_go ? a.input : a.grad_output;
    jb.bs = big_is_go ? go : in;
    jb.ss = big_is_go ? in : go;
    jb.Nb = big_is_go ? a.out_planes : a.in_planes;
    jb.Ns = big_is_go ? a.in_planes : a.out_planes;
    jb.big_is_go = big_is_go ? 1 : 0;
    jb.part = a.part;
    jb.F = a.out_planes;
    jb.P = a.in_planes;
    jb.kh = a.kh;
    jb.kw = a.kw;
    jb.vbatch = a.vbatch;
    jb.nranges = a.nranges;
    jb.alpha = a.alpha;
    hipError_t e;
    switch (N) {
        case 8: e = launch_fused_accgrad_n<8>(jb, s); break;
        case 16: e = launch_fused_accgrad_n<16>(jb, s); break;
        case 32: e = launch_fused_accgrad_n<32>(jb, s); break;
        default: return hipErrorInvalidValue;
    }
    if (e != hipSuccess) return e;
    const long n = (long)a.out_planes * a.in_planes * a.kh * a.kw;
    kernel_log_add("fused_accgrad_sum_kernel", (n + 63) / 64 * 256);
    FBFC_LAUNCH(fused_accgrad_sum_kernel, dim3((unsigned)((n + 63) / 64)), dim3(256), 0, s, a.part, a.grad_weight, n,
                a.nranges);
    return hipGetLastError();
}

}  // namespace fbfc
