// The transforms outside the convolution path that nn.FFTWrapper also offers with fbfft
// (fbcunn/FFTWrapper.lua:53-132 -> src/fft/FBFFTHost.cpp:39-175): batched 1-D real<->complex FFTs
// of sizes 2..128 (fbfft1dHost) and the 2-D sizes 2 and 4, which are below what the tiled 2-D
// kernels are built for.
//
// 1-D, sizes 8 and 16: one lane owns one row.  A workgroup takes a contiguous chunk of rows, copies
// it with coalesced accesses into an LDS canvas (zero-padded rows, stride N + 4 floats: 16-byte
// aligned and rotating over the banks), every lane transforms its row in registers as ONE complex
// transform of half the length (z[m] = x[2m] + i x[2m+1], then the split into the row's half
// spectrum), writes the result over its own canvas row, and the workgroup copies the chunk out,
// again coalesced.  Bytes moved are the algorithmic ones: the rows once, the spectra once.
// 1-D, sizes 32..128: the same staging, but a row is shared by 2, 4 or 8 lanes of a wavefront: eight
// values per lane, an 8-point transform in registers and the remaining butterfly stages across the
// lanes by DPP exchanges (see Split1D below).
// Sizes 2 and 4 (1-D and 2-D) are simple kernels: a lane holds its whole problem in registers
// and talks to global memory directly.
#include <hip/hip_runtime.h>

#include <cstdint>
#include <type_traits>

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
// 1-D, N >= 8: one row per lane, chunk of rows per workgroup staged through LDS
// ---------------------------------------------------------------------------------
template <int N>
struct Rows1D {
    static constexpr int M = N / 2;        // complex length of a lane's transform
    static constexpr int NH = N / 2 + 1;   // stored frequencies of a row
    static constexpr int S = N + 4;        // canvas row stride in floats (holds the N + 2 floats of a spectrum too)
    static constexpr int LANES = (N <= 32) ? 256 : 8192 / N;  // rows per workgroup: at most 37 KB of LDS
};

// Rows [row0, row0 + nr) of `in` (n floats each) into canvas rows: value x[i] at column pad_l + i,
// zeros elsewhere.  V floats per piece (4 needs n, pad_l and the chunk address to be multiples of 4
// floats).  Column slot j of a row carries x[j] if j < n, else a zero for the column
// (j + pad_l) mod N: the columns left of the row wrap around to the slots right of it.
// ROWS canvas rows are staged by NT lanes (one lane per row unless said otherwise).
template <int N, int V, int ROWS = Rows1D<N>::LANES, int NT = Rows1D<N>::LANES>
__device__ __forceinline__ void stage_rows_in(float *smem, const float *__restrict__ src, int nr, int n, int pad_l,
                                              int tid)
{
    using G = Rows1D<N>;
    constexpr int PPR = N / V;                 // pieces per canvas row
    static_assert((ROWS * PPR) % NT == 0, "whole rounds of pieces");
    constexpr int PER_LANE = ROWS * PPR / NT;
    constexpr int CAP = (V == 4) ? 16 : 32;    // loads in flight per lane
    constexpr int CHUNK = (PER_LANE < CAP) ? PER_LANE : CAP;
    using Piece = typename std::conditional<V == 4, float4, float>::type;
    static_for<PER_LANE / CHUNK>([&](auto cc) {
        constexpr int c0 = decltype(cc)::value * CHUNK;
        Piece v[CHUNK];
        int dst[CHUNK];
        static_for<CHUNK>([&](auto ii) {
            constexpr int i = decltype(ii)::value;
            const int idx = (c0 + i) * NT + tid;
            const int row = idx / PPR, col = (idx % PPR) * V;
            const bool live = (row < nr) && (col < n);
            int c = col + pad_l;
            if (c >= N) c -= N;
            dst[i] = row * G::S + c;
            if constexpr (V == 4)
                v[i] = live ? *reinterpret_cast<const float4 *>(src + row * n + col) : make_float4(0.f, 0.f, 0.f, 0.f);
            else
                v[i] = live ? src[row * n + col] : 0.0f;
        });
        static_for<CHUNK>([&](auto ii) {
            constexpr int i = decltype(ii)::value;
            *reinterpret_cast<Piece *>(smem + dst[i]) = v[i];
        });
    });
}

// Canvas rows back to rows of n floats: real[row][i] = canvas[row][pad_l + i].
template <int N, int V, int ROWS = Rows1D<N>::LANES, int NT = Rows1D<N>::LANES>
__device__ __forceinline__ void stage_rows_out(const float *smem, float *__restrict__ dst, int nr, int n, int pad_l,
                                               int tid)
{
    using G = Rows1D<N>;
    constexpr int PPR = N / V;
    static_assert((ROWS * PPR) % NT == 0, "whole rounds of pieces");
    using Piece = typename std::conditional<V == 4, float4, float>::type;
    static_for<ROWS * PPR / NT>([&](auto ii) {
        constexpr int i = decltype(ii)::value;
        const int idx = i * NT + tid;
        const int row = idx / PPR, col = (idx % PPR) * V;
        if (row < nr && col < n)
            *reinterpret_cast<Piece *>(dst + row * n + col) =
                *reinterpret_cast<const Piece *>(smem + row * G::S + pad_l + col);
    });
}

// The spectra of rows [row0, row0 + nr), contiguous in global memory, into canvas rows (complex k of a
// row at floats 2k, 2k+1).  W complex numbers per piece; 2 needs the chunk to start on 16 bytes.  All
// loads of a lane are in flight together (up to 33 pieces of 16 bytes at N = 128): the lanes have no
// other work to hide the latency behind.
template <int N, int W, int ROWS = Rows1D<N>::LANES, int NT = Rows1D<N>::LANES>
__device__ __forceinline__ void stage_spectra_in(float *smem, const float2 *__restrict__ src, int nr, int tid)
{
    using G = Rows1D<N>;
    const int total = nr * G::NH;                       // complex numbers of the chunk
    constexpr int PIECES = ROWS * G::NH / W;            // ROWS is even
    constexpr int PER_LANE = (PIECES + NT - 1) / NT;
    if constexpr (W == 2) {
        float4 v[PER_LANE];
        static_for<PER_LANE>([&](auto ii) {
            constexpr int i = decltype(ii)::value;
            const int e = 2 * (i * NT + tid);
            v[i] = make_float4(0.f, 0.f, 0.f, 0.f);
            if (e + 1 < total) {
                v[i] = *reinterpret_cast<const float4 *>(src + e);
            } else if (e < total) {                     // the last number of a chunk with an odd count
                const float2 a = src[e];
                v[i].x = a.x;
                v[i].y = a.y;
            }
        });
        static_for<PER_LANE>([&](auto ii) {
            constexpr int i = decltype(ii)::value;
            const int e = 2 * (i * NT + tid);
            if (i * NT + tid < PIECES) {
                const int row = e / G::NH, k = e - row * G::NH;
                const bool wrap = (k + 1 == G::NH);     // the second number opens the next row
                *reinterpret_cast<float2 *>(smem + row * G::S + 2 * k) = make_float2(v[i].x, v[i].y);
                *reinterpret_cast<float2 *>(smem + (wrap ? (row + 1) * G::S : row * G::S + 2 * k + 2)) =
                    make_float2(v[i].z, v[i].w);
            }
        });
    } else {
        constexpr int CHUNK = (PER_LANE < 33) ? PER_LANE : 33;
        static_for<(PER_LANE + CHUNK - 1) / CHUNK>([&](auto cc) {
            constexpr int c0 = decltype(cc)::value * CHUNK;
            constexpr int CN = (PER_LANE - c0 < CHUNK) ? PER_LANE - c0 : CHUNK;
            float2 v[CN];
            static_for<CN>([&](auto ii) {
                constexpr int i = decltype(ii)::value;
                const int idx = (c0 + i) * NT + tid;
                v[i] = (idx < total) ? src[idx] : make_float2(0.0f, 0.0f);
            });
            static_for<CN>([&](auto ii) {
                constexpr int i = decltype(ii)::value;
                const int idx = (c0 + i) * NT + tid;
                if (idx >= ROWS * G::NH) return;
                const int row = idx / G::NH, k = idx - row * G::NH;
                *reinterpret_cast<float2 *>(smem + row * G::S + 2 * k) = v[i];
            });
        });
    }
}

template <int N, int V>
__global__ __launch_bounds__(Rows1D<N>::LANES) void rfft1d_rows_kernel(const float *__restrict__ in,
                                                                       float2 *__restrict__ out, long rows, int n,
                                                                       int pad_l)
{
    using G = Rows1D<N>;
    constexpr int M = G::M;
    __shared__ __attribute__((aligned(16))) float smem[G::LANES * G::S];
    const int tid = threadIdx.x;
    const long row0 = (long)blockIdx.x * G::LANES;
    const long left = rows - row0;
    const int nr = left < G::LANES ? (int)left : G::LANES;
    stage_rows_in<N, V>(smem, in + row0 * n, nr, n, pad_l, tid);
    __syncthreads();

    // z[m] = x[2m] + i x[2m+1]
    float re[M], im[M];
    float *mine = smem + tid * G::S;
    static_for<N / 4>([&](auto jj) {
        constexpr int j = decltype(jj)::value;
        const float4 p = reinterpret_cast<const float4 *>(mine)[j];
        re[2 * j] = p.x;
        im[2 * j] = p.y;
        re[2 * j + 1] = p.z;
        im[2 * j + 1] = p.w;
    });
    fft_inplace<M, false>(re, im);
    // X[k] = E[k] + W^k O[k],  E[k] = (Z[k] + conj Z[M-k]) / 2,  O[k] = -i (Z[k] - conj Z[M-k]) / 2,  Z[M] = Z[0]
    float xr[G::NH], xi[G::NH];
    xr[0] = re[0] + im[0];
    xi[0] = 0.0f;
    xr[M] = re[0] - im[0];
    xi[M] = 0.0f;
    xr[M / 2] = re[brev<M>(M / 2)];
    xi[M / 2] = -im[brev<M>(M / 2)];
    static_for<M / 2 - 1>([&](auto kk) {
        constexpr int k = decltype(kk)::value + 1;
        const float a = re[brev<M>(k)], b = im[brev<M>(k)];
        const float c = re[brev<M>(M - k)], d = im[brev<M>(M - k)];
        const float t1 = a + c, t2 = b - d, t3 = b + d, t4 = c - a;
        constexpr float wr = (float)(0.5 * cos2pi(k, N)), wi = (float)(-0.5 * sin2pi(k, N));
        // every multiply-add is spelt out (the file is compiled without implicit contraction: the 16-byte
        // and 4-byte staging variants of a kernel must round alike)
        const float pr = __builtin_fmaf(wr, t3, -(wi * t4)), pi_ = __builtin_fmaf(wr, t4, wi * t3);
        xr[k] = __builtin_fmaf(0.5f, t1, pr);
        xi[k] = __builtin_fmaf(0.5f, t2, pi_);
        xr[M - k] = __builtin_fmaf(0.5f, t1, -pr);
        xi[M - k] = __builtin_fmaf(-0.5f, t2, pi_);
    });
    // the spectrum over the lane's own canvas row (no other lane reads or writes it before the barrier)
    static_for<M / 2>([&](auto jj) {
        constexpr int j = decltype(jj)::value;
        reinterpret_cast<float4 *>(mine)[j] = make_float4(xr[2 * j], xi[2 * j], xr[2 * j + 1], xi[2 * j + 1]);
    });
    reinterpret_cast<float2 *>(mine)[M] = make_float2(xr[M], xi[M]);
    __syncthreads();

    // the chunk's spectra are contiguous in global memory: piece idx is complex number idx of the chunk
    float2 *dst = out + row0 * G::NH;
    const int total = nr * G::NH;
    static_for<G::NH>([&](auto ii) {
        constexpr int i = decltype(ii)::value;
        const int idx = i * G::LANES + tid;
        const int row = idx / G::NH, k = idx - row * G::NH;
        if (idx < total) dst[idx] = *reinterpret_cast<const float2 *>(smem + row * G::S + 2 * k);
    });
}

// Unnormalised inverse: (rows, N/2+1) complex -> real[row][i] = y[pad_l + i], i < n.  The imaginary
// parts of the bins 0 and N/2 of a row are not read, as in any complex-to-real transform.
template <int N, int V, int W>
__global__ __launch_bounds__(Rows1D<N>::LANES) void irfft1d_rows_kernel(const float2 *__restrict__ in,
                                                                        float *__restrict__ out, long rows, int n,
                                                                        int pad_l)
{
    using G = Rows1D<N>;
    constexpr int M = G::M;
    __shared__ __attribute__((aligned(16))) float smem[G::LANES * G::S];
    const int tid = threadIdx.x;
    const long row0 = (long)blockIdx.x * G::LANES;
    const long left = rows - row0;
    const int nr = left < G::LANES ? (int)left : G::LANES;
    stage_spectra_in<N, W>(smem, in + row0 * G::NH, nr, tid);
    __syncthreads();

    // Z[k] = Ee[k] + i Oo[k],  Ee[k] = X[k] + conj X[M-k],  Oo[k] = exp(+2 pi i k / N) (X[k] - conj X[M-k])
    float zr[M], zi[M];
    float *mine = smem + tid * G::S;
    static_for<M / 2>([&](auto jj) {
        constexpr int j = decltype(jj)::value;
        const float4 p = reinterpret_cast<const float4 *>(mine)[j];
        zr[2 * j] = p.x;
        zi[2 * j] = p.y;
        zr[2 * j + 1] = p.z;
        zi[2 * j + 1] = p.w;
    });
    {
        const float x0 = zr[0], xm = reinterpret_cast<const float2 *>(mine)[M].x;
        zr[0] = x0 + xm;
        zi[0] = x0 - xm;
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
    // y[2m] = Re z[m], y[2m+1] = Im z[m], over the lane's own canvas row
    static_for<N / 4>([&](auto jj) {
        constexpr int j = decltype(jj)::value;
        reinterpret_cast<float4 *>(mine)[j] = make_float4(zr[brev<M>(2 * j)], zi[brev<M>(2 * j)],
                                                          zr[brev<M>(2 * j + 1)], zi[brev<M>(2 * j + 1)]);
    });
    __syncthreads();
    stage_rows_out<N, V>(smem, out + row0 * n, nr, n, pad_l, tid);
}

// ---------------------------------------------------------------------------------
// 1-D, N = 64 and 128: a row over L = N / 16 lanes of one wavefront
//
// One lane per row means 64 complex values (N = 128) in the registers of a lane and one wavefront per
// SIMD.  Here a row's half-length complex sequence z (M = N / 2 values) is split over L lanes of 8 values
// each, so a lane needs some 50 registers and the wavefronts of a CU cover each other's memory latency.
// With n = s + L m and k = q + 8 p (lane s, m, q < 8, p < L) and w = exp(-2 pi i / M):
//   Z[q + 8 p] = sum_s w_L^(s p) [ w^(s q) sum_m z[s + L m] w_8^(m q) ]
// i.e. an 8-point transform inside the lane, one twiddle per value, then an L-point transform ACROSS the
// lanes: log2 L butterfly stages whose partner lanes differ in one bit of the lane number and exchange
// their values through DPP moves (row_shl / row_shr by four lanes under bank masks, quad_perm for two and
// one): no LDS traffic and no barrier.  Lane s ends up with the outputs k = 8 p .. 8 p + 7, p = the bit
// reversal of s.  The split into the real row's spectrum (forward) or its reverse (inverse) needs Z[k]
// together with Z[M - k], which belongs to another lane of the row: it goes through the row's own canvas
// line in LDS.  Staging in and out is that of the one-lane-per-row kernels.
// ---------------------------------------------------------------------------------
template <int N>
struct Split1D {
    static constexpr int M = N / 2;
    static constexpr int R = 8;              // values per lane
    static constexpr int L = M / R;          // lanes per row: 4 (N = 64), 8 (N = 128)
    static constexpr int ROWS = 64;          // rows per workgroup
    static constexpr int NT = ROWS * L;
    static_assert(L == 2 || L == 4 || L == 8, "N = 32, 64 or 128");
};

template <int CTRL, int BANK>
__device__ __forceinline__ float dpp_move(float old, float v)
{
    return __int_as_float(__builtin_amdgcn_update_dpp(__float_as_int(old), __float_as_int(v), CTRL, 0xf, BANK, false));
}
// the value lane (l ^ H) holds, H = 4, 2 or 1 (lanes of one row of 16)
template <int H>
__device__ __forceinline__ float lane_xor(float v)
{
    if constexpr (H == 4) {
        // lanes 0-3 and 8-11 of a row (banks 0, 2) take from four lanes up, the others from four lanes down
        return dpp_move<0x114, 0xa>(dpp_move<0x104, 0x5>(v, v), v);
    } else if constexpr (H == 2) {
        return dpp_move<0x4e, 0xf>(v, v);   // quad_perm [2, 3, 0, 1]
    } else {
        return dpp_move<0xb1, 0xf>(v, v);   // quad_perm [1, 0, 3, 2]
    }
}

// One decimation-in-frequency stage across lanes: lanes with bit H clear get a + b, the others
// (a - b) w, a from the lower lane.  sg = -1 / +1 and (wr, wi) = w / 1 for upper / lower lanes.
template <int H, bool TW>
__device__ __forceinline__ void cross_stage(float (&re)[8], float (&im)[8], float sg, float wr, float wi)
{
    static_for<8>([&](auto qq) {
        constexpr int q = decltype(qq)::value;
        const float ar = re[q], ai = im[q];
        const float br = lane_xor<H>(ar), bi = lane_xor<H>(ai);
        const float dr = __builtin_fmaf(sg, ar, br), di = __builtin_fmaf(sg, ai, bi);
        if constexpr (TW) {
            re[q] = __builtin_fmaf(dr, wr, -(di * wi));
            im[q] = __builtin_fmaf(dr, wi, di * wr);
        } else {
            re[q] = dr;
            im[q] = di;
        }
    });
}

// L-point transform over the lanes s = 0 .. L-1 of a row, for each of the 8 register positions; the
// result of index p is left in lane brev_L(p).
template <int L, bool INV>
__device__ __forceinline__ void cross_transform(float (&re)[8], float (&im)[8], int s)
{
    constexpr float C = 0.70710678118654752f;
    constexpr float SGN = INV ? 1.0f : -1.0f;   // sign of the twiddles' imaginary parts
    if constexpr (L == 8) {
        const bool up = (s & 4) != 0;
        const int j = s & 3;   // w_8^j
        const float wr = !up ? 1.0f : (j == 0 ? 1.0f : j == 1 ? C : j == 2 ? 0.0f : -C);
        const float wi = !up ? 0.0f : SGN * (j == 0 ? 0.0f : j == 2 ? 1.0f : C);
        cross_stage<4, true>(re, im, up ? -1.0f : 1.0f, wr, wi);
    }
    if constexpr (L >= 4) {
        const bool up = (s & 2) != 0;
        const bool odd = (s & 1) != 0;   // w_4^1 = -i (forward)
        const float wr = (up && odd) ? 0.0f : 1.0f;
        const float wi = (up && odd) ? SGN : 0.0f;
        cross_stage<2, true>(re, im, up ? -1.0f : 1.0f, wr, wi);
    }
    cross_stage<1, false>(re, im, (s & 1) ? -1.0f : 1.0f, 1.0f, 0.0f);
}

template <int L>
__device__ __forceinline__ int brev_lanes(int s)
{
    if constexpr (L == 8) return ((s & 1) << 2) | (s & 2) | ((s >> 2) & 1);
    else if constexpr (L == 4) return ((s & 1) << 1) | ((s >> 1) & 1);
    else return s;
}

// exp(-2 pi i j / M), j < M, as (cos, -sin) pairs behind the canvas
template <int M>
__device__ __forceinline__ void fill_twiddles(float *tw, int tid)
{
    if (tid < M) {
        float sn, cs;
        sincospif(-2.0f * (float)tid / (float)M, &sn, &cs);
        tw[2 * tid] = cs;
        tw[2 * tid + 1] = sn;
    }
}

template <int N, int V>
__global__ __launch_bounds__(Split1D<N>::NT) void rfft1d_split_kernel(const float *__restrict__ in,
                                                                      float2 *__restrict__ out, long rows, int n,
                                                                      int pad_l)
{
    using G = Split1D<N>;
    using C = Rows1D<N>;
    constexpr int M = G::M, R = G::R, L = G::L;
    __shared__ __attribute__((aligned(16))) float smem[G::ROWS * C::S + 2 * M];
    float *tw = smem + G::ROWS * C::S;
    const int tid = threadIdx.x;
    const long row0 = (long)blockIdx.x * G::ROWS;
    const long left = rows - row0;
    const int nr = left < G::ROWS ? (int)left : G::ROWS;
    fill_twiddles<M>(tw, tid);
    stage_rows_in<N, V, G::ROWS, G::NT>(smem, in + row0 * n, nr, n, pad_l, tid);
    __syncthreads();

    const int s = tid % L;
    float *mine = smem + (tid / L) * C::S;
    float re[R], im[R];
    static_for<R>([&](auto mm) {   // z[s + L m] = x[2 (s + L m)] + i x[2 (s + L m) + 1]
        constexpr int m = decltype(mm)::value;
        const float2 v = *reinterpret_cast<const float2 *>(mine + 2 * (s + L * m));
        re[m] = v.x;
        im[m] = v.y;
    });
    fft_inplace<R, false>(re, im);
    static_for<R - 1>([&](auto qq) {   // times w^(s q)
        constexpr int q = decltype(qq)::value + 1;
        constexpr int pos = brev<R>(q);
        const float2 t = *reinterpret_cast<const float2 *>(tw + 2 * (s * q));
        const float xr = re[pos], xi = im[pos];
        re[pos] = __builtin_fmaf(xr, t.x, -(xi * t.y));
        im[pos] = __builtin_fmaf(xr, t.y, xi * t.x);
    });
    cross_transform<L, false>(re, im, s);

    // Z[8 p + q] over the row's canvas line, complex k at floats 2k, 2k + 1
    const int p = brev_lanes<L>(s);
    float *blk = mine + 2 * R * p;
    __syncthreads();
    static_for<R / 2>([&](auto jj) {
        constexpr int j = decltype(jj)::value;
        reinterpret_cast<float4 *>(blk)[j] = make_float4(re[brev<R>(2 * j)], im[brev<R>(2 * j)],
                                                         re[brev<R>(2 * j + 1)], im[brev<R>(2 * j + 1)]);
    });
    __syncthreads();
    // X[k] = E + W^k O,  E = (Z[k] + conj Z[M-k]) / 2,  O = -i (Z[k] - conj Z[M-k]) / 2,  W = exp(-2 pi i / N),
    // Z[M] = Z[0]; W^(8 p + q) = exp(-pi i p / L) W^q, the first factor from the table (entry 4 p)
    const float2 up = *reinterpret_cast<const float2 *>(tw + 2 * (4 * p));
    float xr[R], xi[R];
    static_for<R>([&](auto qq) {
        constexpr int q = decltype(qq)::value;
        const int kp = (M - (R * p + q)) & (M - 1);
        const float2 cd = *reinterpret_cast<const float2 *>(mine + 2 * kp);
        const float a = re[brev<R>(q)], b = im[brev<R>(q)];
        const float t1 = a + cd.x, t2 = b - cd.y, t3 = b + cd.y, t4 = cd.x - a;
        constexpr float cr = (float)(0.5 * cos2pi(q, N)), ci = (float)(-0.5 * sin2pi(q, N));
        const float wr = __builtin_fmaf(up.x, cr, -(up.y * ci)), wi = __builtin_fmaf(up.x, ci, up.y * cr);
        const float pr = __builtin_fmaf(wr, t3, -(wi * t4)), pi_ = __builtin_fmaf(wr, t4, wi * t3);
        xr[q] = __builtin_fmaf(0.5f, t1, pr);
        xi[q] = __builtin_fmaf(0.5f, t2, pi_);
    });
    const float xm = re[0] - im[0];   // X[M] = Re Z[0] - Im Z[0] (lane p = 0)
    __syncthreads();
    static_for<R / 2>([&](auto jj) {
        constexpr int j = decltype(jj)::value;
        reinterpret_cast<float4 *>(blk)[j] = make_float4(xr[2 * j], xi[2 * j], xr[2 * j + 1], xi[2 * j + 1]);
    });
    if (p == 0) {
        mine[1] = 0.0f;   // bin 0 is real
        *reinterpret_cast<float2 *>(mine + 2 * M) = make_float2(xm, 0.0f);
    }
    __syncthreads();

    float2 *dst = out + row0 * C::NH;
    const int total = nr * C::NH;
    static_for<(G::ROWS * C::NH + G::NT - 1) / G::NT>([&](auto ii) {
        constexpr int i = decltype(ii)::value;
        const int idx = i * G::NT + tid;
        const int row = idx / C::NH, k = idx - row * C::NH;
        if (idx < total) dst[idx] = *reinterpret_cast<const float2 *>(smem + row * C::S + 2 * k);
    });
}

template <int N, int V, int W>
__global__ __launch_bounds__(Split1D<N>::NT) void irfft1d_split_kernel(const float2 *__restrict__ in,
                                                                       float *__restrict__ out, long rows, int n,
                                                                       int pad_l)
{
    using G = Split1D<N>;
    using C = Rows1D<N>;
    constexpr int M = G::M, R = G::R, L = G::L;
    __shared__ __attribute__((aligned(16))) float smem[G::ROWS * C::S + 2 * M];
    float *tw = smem + G::ROWS * C::S;
    const int tid = threadIdx.x;
    const long row0 = (long)blockIdx.x * G::ROWS;
    const long left = rows - row0;
    const int nr = left < G::ROWS ? (int)left : G::ROWS;
    fill_twiddles<M>(tw, tid);
    stage_spectra_in<N, W, G::ROWS, G::NT>(smem, in + row0 * C::NH, nr, tid);
    __syncthreads();

    const int s = tid % L;
    float *mine = smem + (tid / L) * C::S;
    // Z[k] = Ee[k] + i Oo[k],  Ee = X[k] + conj X[M-k],  Oo = V^k (X[k] - conj X[M-k]),  V = exp(+2 pi i / N);
    // the lane takes k = s + L m: V^k = exp(2 pi i s / N) V^(L m).  The imaginary parts of X[0] and X[M] are not used.
    float vsr, vsi;
    sincospif(2.0f * (float)s / (float)N, &vsi, &vsr);
    float zr[R], zi[R];
    static_for<R>([&](auto mm) {
        constexpr int m = decltype(mm)::value;
        const int k = s + L * m;
        const float2 x = *reinterpret_cast<const float2 *>(mine + 2 * k);
        const float2 y = *reinterpret_cast<const float2 *>(mine + 2 * (M - k));
        const bool dc = (m == 0) && (s == 0);
        const float a = x.x, b = dc ? 0.0f : x.y, c = y.x, d = dc ? 0.0f : y.y;
        const float sr = a + c, si = b - d, dr = a - c, di = b + d;
        constexpr float cr = (float)cos2pi(L * m, N), ci = (float)sin2pi(L * m, N);
        const float vr = __builtin_fmaf(vsr, cr, -(vsi * ci)), vi = __builtin_fmaf(vsr, ci, vsi * cr);
        const float pp = __builtin_fmaf(vr, dr, -(vi * di)), qq = __builtin_fmaf(vr, di, vi * dr);
        zr[m] = sr - qq;
        zi[m] = si + pp;
    });
    fft_inplace<R, true>(zr, zi);
    static_for<R - 1>([&](auto qq) {   // times conj w^(s q)
        constexpr int q = decltype(qq)::value + 1;
        constexpr int pos = brev<R>(q);
        const float2 t = *reinterpret_cast<const float2 *>(tw + 2 * (s * q));
        const float xr = zr[pos], xi = zi[pos];
        zr[pos] = __builtin_fmaf(xr, t.x, xi * t.y);
        zi[pos] = __builtin_fmaf(xi, t.x, -(xr * t.y));
    });
    cross_transform<L, true>(zr, zi, s);

    // z[8 p + q] = y[2 (8 p + q)] + i y[2 (8 p + q) + 1] over the row's canvas line
    const int p = brev_lanes<L>(s);
    float *blk = mine + 2 * R * p;
    __syncthreads();
    static_for<R / 2>([&](auto jj) {
        constexpr int j = decltype(jj)::value;
        reinterpret_cast<float4 *>(blk)[j] = make_float4(zr[brev<R>(2 * j)], zi[brev<R>(2 * j)],
                                                         zr[brev<R>(2 * j + 1)], zi[brev<R>(2 * j + 1)]);
    });
    __syncthreads();
    stage_rows_out<N, V, G::ROWS, G::NT>(smem, out + row0 * n, nr, n, pad_l, tid);
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
static hipError_t launch1d_tiny(bool inverse, const float *in, float *out, long rows, int n, int pad_l, hipStream_t s)
{
    const long pairs = (rows + 1) / 2;
    const long blocks = (pairs + 255) / 256;
    if (blocks > 0x7fffffffL) return hipErrorInvalidValue;
    if (!inverse) {
        FBFC_LAUNCH(rfft1d_kernel<N>, dim3((unsigned)blocks), dim3(256), 0, s, in,
                           reinterpret_cast<float2 *>(out), rows, n, pad_l);
        kernel_log_add("rfft1d_kernel", blocks * 256);
    } else {
        FBFC_LAUNCH(irfft1d_kernel<N>, dim3((unsigned)blocks), dim3(256), 0, s,
                           reinterpret_cast<const float2 *>(in), out, rows, n, pad_l);
        kernel_log_add("irfft1d_kernel", blocks * 256);
    }
    return hipGetLastError();
}

// 16-byte pieces need rows, padding and the real tensor itself to sit on 16-byte boundaries
static bool rows_vec4(const float *real, int n, int pad_l)
{
    return n % 4 == 0 && pad_l % 4 == 0 && (reinterpret_cast<uintptr_t>(real) & 15) == 0;
}

// N = 64 and 128: a row over four or eight lanes
template <int N>
static hipError_t launch1d_split(bool inverse, const float *in, float *out, long rows, int n, int pad_l, hipStream_t s)
{
    using G = Split1D<N>;
    const long blocks = (rows + G::ROWS - 1) / G::ROWS;
    if (blocks > 0x7fffffffL) return hipErrorInvalidValue;
    const dim3 grid((unsigned)blocks), block(G::NT);
    if (!inverse) {
        float2 *freq = reinterpret_cast<float2 *>(out);
        if (rows_vec4(in, n, pad_l))
            FBFC_LAUNCH((rfft1d_split_kernel<N, 4>), grid, block, 0, s, in, freq, rows, n, pad_l);
        else
            FBFC_LAUNCH((rfft1d_split_kernel<N, 1>), grid, block, 0, s, in, freq, rows, n, pad_l);
        kernel_log_add("rfft1d_split_kernel", blocks * G::NT);
    } else {
        const float2 *freq = reinterpret_cast<const float2 *>(in);
        const bool wide = (reinterpret_cast<uintptr_t>(in) & 15) == 0;  // chunks start on even complex counts
        const bool vec = rows_vec4(out, n, pad_l);
        if (vec && wide)
            FBFC_LAUNCH((irfft1d_split_kernel<N, 4, 2>), grid, block, 0, s, freq, out, rows, n, pad_l);
        else if (vec)
            FBFC_LAUNCH((irfft1d_split_kernel<N, 4, 1>), grid, block, 0, s, freq, out, rows, n, pad_l);
        else if (wide)
            FBFC_LAUNCH((irfft1d_split_kernel<N, 1, 2>), grid, block, 0, s, freq, out, rows, n, pad_l);
        else
            FBFC_LAUNCH((irfft1d_split_kernel<N, 1, 1>), grid, block, 0, s, freq, out, rows, n, pad_l);
        kernel_log_add("irfft1d_split_kernel", blocks * G::NT);
    }
    return hipGetLastError();
}

template <int N>
static hipError_t launch1d(bool inverse, const float *in, float *out, long rows, int n, int pad_l, hipStream_t s)
{
    using G = Rows1D<N>;
    const long blocks = (rows + G::LANES - 1) / G::LANES;
    if (blocks > 0x7fffffffL) return hipErrorInvalidValue;
    const dim3 grid((unsigned)blocks), block(G::LANES);
    if (!inverse) {
        float2 *freq = reinterpret_cast<float2 *>(out);
        if (rows_vec4(in, n, pad_l))
            FBFC_LAUNCH((rfft1d_rows_kernel<N, 4>), grid, block, 0, s, in, freq, rows, n, pad_l);
        else
            FBFC_LAUNCH((rfft1d_rows_kernel<N, 1>), grid, block, 0, s, in, freq, rows, n, pad_l);
        kernel_log_add("rfft1d_rows_kernel", blocks * G::LANES);
    } else {
        const float2 *freq = reinterpret_cast<const float2 *>(in);
        const bool wide = (reinterpret_cast<uintptr_t>(in) & 15) == 0;  // chunks start on even complex counts
        const bool vec = rows_vec4(out, n, pad_l);
        if (vec && wide)
            FBFC_LAUNCH((irfft1d_rows_kernel<N, 4, 2>), grid, block, 0, s, freq, out, rows, n, pad_l);
        else if (vec)
            FBFC_LAUNCH((irfft1d_rows_kernel<N, 4, 1>), grid, block, 0, s, freq, out, rows, n, pad_l);
        else if (wide)
            FBFC_LAUNCH((irfft1d_rows_kernel<N, 1, 2>), grid, block, 0, s, freq, out, rows, n, pad_l);
        else
            FBFC_LAUNCH((irfft1d_rows_kernel<N, 1, 1>), grid, block, 0, s, freq, out, rows, n, pad_l);
        kernel_log_add("irfft1d_rows_kernel", blocks * G::LANES);
    }
    return hipGetLastError();
}

static hipError_t dispatch1d(bool inverse, int N, const float *in, float *out, long rows, int n, int pad_l,
                             hipStream_t s)
{
    switch (N) {
        case 2: return launch1d_tiny<2>(inverse, in, out, rows, n, pad_l, s);
        case 4: return launch1d_tiny<4>(inverse, in, out, rows, n, pad_l, s);
        case 8: return launch1d<8>(inverse, in, out, rows, n, pad_l, s);
        case 16: return launch1d<16>(inverse, in, out, rows, n, pad_l, s);
        case 32: return launch1d_split<32>(inverse, in, out, rows, n, pad_l, s);
        case 64: return launch1d_split<64>(inverse, in, out, rows, n, pad_l, s);
        case 128: return launch1d_split<128>(inverse, in, out, rows, n, pad_l, s);
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
    if (blocks > 0x7fffffffL || (N != 2 && N != 4)) return hipErrorInvalidValue;
    kernel_log_add(N == 2 ? "rfft2d_tiny_kernel<2>" : "rfft2d_tiny_kernel<4>", blocks * 256);
    if (N == 2)
        FBFC_LAUNCH(rfft2d_tiny_kernel<2>, dim3((unsigned)blocks), dim3(256), 0, s, in,
                           reinterpret_cast<float2 *>(out), planes, h, w, pad_u, pad_l);
    else if (N == 4)
        FBFC_LAUNCH(rfft2d_tiny_kernel<4>, dim3((unsigned)blocks), dim3(256), 0, s, in,
                           reinterpret_cast<float2 *>(out), planes, h, w, pad_u, pad_l);
    else
        return hipErrorInvalidValue;
    return hipGetLastError();
}

hipError_t launch_irfft2d_tiny(int N, const float *in, float *out, long planes, int h, int w, int pad_u,
                               int pad_l, const float *bias, int bias_period, hipStream_t s)
{
    const long blocks = (planes + 255) / 256;
    if (blocks > 0x7fffffffL || (N != 2 && N != 4)) return hipErrorInvalidValue;
    kernel_log_add(N == 2 ? "irfft2d_tiny_kernel<2>" : "irfft2d_tiny_kernel<4>", blocks * 256);
    const int period = bias_period > 0 ? bias_period : 1;
    if (N == 2)
        FBFC_LAUNCH(irfft2d_tiny_kernel<2>, dim3((unsigned)blocks), dim3(256), 0, s,
                           reinterpret_cast<const float2 *>(in), out, planes, h, w, pad_u, pad_l, bias, period);
    else if (N == 4)
        FBFC_LAUNCH(irfft2d_tiny_kernel<4>, dim3((unsigned)blocks), dim3(256), 0, s,
                           reinterpret_cast<const float2 *>(in), out, planes, h, w, pad_u, pad_l, bias, period);
    else
        return hipErrorInvalidValue;
    return hipGetLastError();
}

}  // namespace fbfc
