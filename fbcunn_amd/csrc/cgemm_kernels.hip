// Per-frequency complex contraction over planes as an fp32 MFMA GEMM (gfx950).
//
// Replaces transposeMMFFI -> fbcuda transposeMM (src/MM.cu:14-73) and the
// cublasCgeam + cublasCgemmBatched pair of the Gemm module
// (src/CuBLASWrapper.cpp:113-125, 437-452).  The three call sites
// (fbcunn/SpatialConvolutionFBFFT.lua:157-164, 244-251, 337-344) map to modes
// 0, 1, 2 below.  Operands are frequency-major, so each frequency is a dense
// row-major complex matrix and no transpose kernel exists.
//
// v_mfma_f32_32x32x2_f32 takes the two k of a step from the two half-waves; because a
// sum may run over k in any order, each half-wave is given the k that are contiguous for
// it in memory.  A complex product is formed from three real ones (cmac3 below).
//
// Workgroup of the general kernel: 256 lanes = 4 waves in 2x2, each wave a 32x32 complex
// block; tile 64 x 64 x 16 complex per step with register-prefetch double buffering through LDS.
#include <hip/hip_runtime.h>

#include <atomic>
#include <cstdio>

#include "kernels.h"
#include "store_nt.h"

namespace fbfc {

typedef float floatx16 __attribute__((ext_vector_type(16)));

__device__ __forceinline__ int map_freq(int i, const FreqMap &fm)
{
    if (fm.split == 0 || i < fm.split) return i;
    const int j = i - fm.split;
    const int row = j / fm.rowlen;
    return fm.split + row * fm.nh + (j - row * fm.rowlen) + 1;
}

// The kernels' `accumulate` argument carries two flags.  A result the caches can keep until the inverse
// transform reads it is written through to the memory side; a larger one is streamed with non-temporal
// stores (same rule and numbers as the spectra of the forward transforms, fft_stage.h).
constexpr int RESULT_ACCUMULATE = 1, RESULT_STREAM = 2;
__device__ __forceinline__ void store_result(float2 *p, const float2 &v, int flags)
{
    if (flags & RESULT_STREAM) store_nt(p, v);
    else store_wt(p, v);
}

constexpr int BM = 64, BN = 64, KT = 16;
constexpr int LDK = 2 * KT + 4;  // floats per row of a K-contiguous tile [64][KT] (+16 B pad)
constexpr int LDM = 2 * 64;      // floats per row of a row-contiguous tile [KT][64]
constexpr int TILE_FLOATS_KC = 64 * LDK;
constexpr int TILE_FLOATS_MC = KT * LDM;
constexpr int TILE_FLOATS = TILE_FLOATS_KC > TILE_FLOATS_MC ? TILE_FLOATS_KC : TILE_FLOATS_MC;

// Loads one operand tile (1024 complex = 4 per lane) into registers.
//   KC == true : matrix is [rows][K], tile covers rows r0.. (64) x k0.. (KT)
//   KC == false: matrix is [K][cols], tile covers k0.. (KT) x c0.. (64)
template <bool KC>
__device__ __forceinline__ void load_tile(const float2 *__restrict__ M, int ld, int nrows_total,
                                          int ncols_total, int r0, int c0, int tid, float2 (&v)[4])
{
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const int e = tid + 256 * i;
        int r, c;
        if (KC) { r = e / KT; c = e % KT; } else { r = e / 64; c = e % 64; }
        const int gr = r0 + r, gc = c0 + c;
        v[i] = (gr < nrows_total && gc < ncols_total) ? M[(long)gr * ld + gc] : make_float2(0.f, 0.f);
    }
}

template <bool KC>
__device__ __forceinline__ void store_tile(float *lds, int tid, const float2 (&v)[4])
{
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const int e = tid + 256 * i;
        int r, c;
        if (KC) { r = e / KT; c = e % KT; } else { r = e / 64; c = e % 64; }
        float2 *p = reinterpret_cast<float2 *>(lds + r * (KC ? LDK : LDM) + 2 * c);
        *p = v[i];
    }
}

// ---------------------------------------------------------------------------------------
// Complex products with three real MFMAs instead of four.  With
//   P1 = sum ar br,  P2 = sum ai bi,  P3 = sum (ar +- ai)(br +- bi)
// the three modes are
//   A conj(B):     Re = P1 + P2,  Im = P3 - P1 + P2,  P3 from (ar + ai)(br - bi)
//   A B:           Re = P1 - P2,  Im = P3 - P1 - P2,  P3 from (ar + ai)(br + bi)
//   conj(A)^T B:   Re = P1 + P2,  Im = P3 - P1 + P2,  P3 from (ar - ai)(br + bi)
// i.e. 6 instead of 8 flops per complex multiply-add on the matrix cores, paid for with two
// vector adds per operand element and a third accumulator (16 registers per 32x32 block).
// ---------------------------------------------------------------------------------------
template <int MODE>
__device__ __forceinline__ void cmac3(float ar, float ai, float br, float bi, floatx16 &p1, floatx16 &p2,
                                      floatx16 &p3)
{
    const float sa = (MODE == 2) ? ar - ai : ar + ai;
    const float sb = (MODE == 0) ? br - bi : br + bi;
    p1 = __builtin_amdgcn_mfma_f32_32x32x2f32(ar, br, p1, 0, 0, 0);
    p2 = __builtin_amdgcn_mfma_f32_32x32x2f32(ai, bi, p2, 0, 0, 0);
    p3 = __builtin_amdgcn_mfma_f32_32x32x2f32(sa, sb, p3, 0, 0, 0);
}

template <int MODE>
__device__ __forceinline__ void combine3(const floatx16 &p1, const floatx16 &p2, const floatx16 &p3,
                                         floatx16 &cre, floatx16 &cim)
{
#pragma unroll
    for (int r = 0; r < 16; ++r) {
        const float s2 = (MODE == 1) ? -p2[r] : p2[r];
        cre[r] = p1[r] + s2;
        cim[r] = (p3[r] - p1[r]) + s2;
    }
}

template <int MODE>
__global__ __launch_bounds__(256) void cgemm_freq_kernel(const float2 *__restrict__ A,
                                                         const float2 *__restrict__ B,
                                                         float2 *__restrict__ C, int M, int N, int K,
                                                         float alpha, int accumulate, int tilesM,
                                                         int tilesN, int total_wgs, int chunk, FreqMap fm)
{
    constexpr bool A_KC = (MODE != 2);
    constexpr bool B_KC = (MODE == 0);
    __shared__ __align__(16) float As[2][TILE_FLOATS];
    __shared__ __align__(16) float Bs[2][TILE_FLOATS];

    // Workgroups are handed to the 8 XCDs round-robin; remap so that each XCD
    // works on a contiguous range of (frequency, tile) and the tiles of one
    // frequency share that XCD's L2.
    const int wg = (int)(blockIdx.x % 8) * chunk + (int)(blockIdx.x / 8);
    if (wg >= total_wgs) return;
    const int tiles = tilesM * tilesN;
    const int qi = wg / tiles;
    const int tile = wg - qi * tiles;
    const int q = map_freq(qi, fm);
    const int m0 = (tile / tilesN) * BM;
    const int n0 = (tile % tilesN) * BN;

    const float2 *Aq = A + (long)q * M * K;
    const float2 *Bq = B + (long)q * N * K;
    float2 *Cq = C + (long)q * M * N;

    const int tid = threadIdx.x;
    const int lane = tid & 63, wave = tid >> 6;
    const int wm = wave >> 1, wn = wave & 1;
    const int li = lane & 31, h = lane >> 5;

    floatx16 p1, p2, p3;
#pragma unroll
    for (int r = 0; r < 16; ++r) { p1[r] = 0.f; p2[r] = 0.f; p3[r] = 0.f; }

    float2 pa[4], pb[4];
    const int nk = (K + KT - 1) / KT;

    auto gload = [&](int kt) {
        const int k0 = kt * KT;
        if (A_KC) load_tile<true>(Aq, K, M, K, m0, k0, tid, pa);   // A[m][k]
        else      load_tile<false>(Aq, M, K, M, k0, m0, tid, pa);  // A[k][m]
        if (B_KC) load_tile<true>(Bq, K, N, K, n0, k0, tid, pb);   // B[n][k]
        else      load_tile<false>(Bq, N, K, N, k0, n0, tid, pb);  // B[k][n]
    };
    auto sstore = [&](int buf) {
        store_tile<A_KC>(As[buf], tid, pa);
        store_tile<B_KC>(Bs[buf], tid, pb);
    };

    gload(0);
    sstore(0);
    __syncthreads();

    for (int kt = 0; kt < nk; ++kt) {
        const int buf = kt & 1;
        if (kt + 1 < nk) gload(kt + 1);

        const float *as = As[buf];
        const float *bs = Bs[buf];
        const int arow = 32 * wm + li;  // row of the A' operand this lane feeds
        const int bcol = 32 * wn + li;  // column of the B' operand this lane feeds

        if (MODE == 0) {
            // both K-contiguous: half-wave h owns complex k in [8h, 8h+8) = 16 consecutive floats
            float a[16], b[16];
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const float4 va = *reinterpret_cast<const float4 *>(as + arow * LDK + 16 * h + 4 * j);
                const float4 vb = *reinterpret_cast<const float4 *>(bs + bcol * LDK + 16 * h + 4 * j);
                a[4 * j] = va.x; a[4 * j + 1] = va.y; a[4 * j + 2] = va.z; a[4 * j + 3] = va.w;
                b[4 * j] = vb.x; b[4 * j + 1] = vb.y; b[4 * j + 2] = vb.z; b[4 * j + 3] = vb.w;
            }
#pragma unroll
            for (int s = 0; s < 16; s += 2) cmac3<0>(a[s], a[s + 1], b[s], b[s + 1], p1, p2, p3);  // C = A conj(B)
        } else if (MODE == 1) {
            // A K-contiguous (as above); B row-contiguous [k][n]: one (re,im) pair per two steps
            float a[16];
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const float4 va = *reinterpret_cast<const float4 *>(as + arow * LDK + 16 * h + 4 * j);
                a[4 * j] = va.x; a[4 * j + 1] = va.y; a[4 * j + 2] = va.z; a[4 * j + 3] = va.w;
            }
#pragma unroll
            for (int kk = 0; kk < 8; ++kk) {
                const float2 vb = *reinterpret_cast<const float2 *>(bs + (8 * h + kk) * LDM + 2 * bcol);
                cmac3<1>(a[2 * kk], a[2 * kk + 1], vb.x, vb.y, p1, p2, p3);  // C = A B
            }
        } else {
            // both row-contiguous [k][.]: half-wave h owns k = 8h + kk.   C = conj(A)^T B
#pragma unroll
            for (int kk = 0; kk < 8; ++kk) {
                const float2 va = *reinterpret_cast<const float2 *>(as + (8 * h + kk) * LDM + 2 * arow);
                const float2 vb = *reinterpret_cast<const float2 *>(bs + (8 * h + kk) * LDM + 2 * bcol);
                cmac3<2>(va.x, va.y, vb.x, vb.y, p1, p2, p3);
            }
        }

        if (kt + 1 < nk) {
            sstore(buf ^ 1);  // the other buffer was last read before the previous barrier
            __syncthreads();
        }
    }

    // epilogue: accumulator register r of lane (li, h) is C[8*(r/4) + 4*h + r%4][li] of the block
    floatx16 cre, cim;
    combine3<MODE>(p1, p2, p3, cre, cim);
#pragma unroll
    for (int r = 0; r < 16; ++r) {
        const int row = m0 + 32 * wm + 8 * (r / 4) + 4 * h + (r % 4);
        const int col = n0 + 32 * wn + li;
        if (row < M && col < N) {
            float2 v = make_float2(alpha * cre[r], alpha * cim[r]);
            float2 *dst = Cq + (long)row * N + col;
            if (accumulate & RESULT_ACCUMULATE) {
                const float2 o = *dst;
                v.x += o.x;
                v.y += o.y;
            }
            store_result(dst, v, accumulate);
        }
    }
}

// ---------------------------------------------------------------------------------------
// LDS-direct variant of the tiled kernel (M % 64 == N % 64 == 0, K % 16 == 0).
//
// Operand tiles go from global memory straight into LDS with global_load_lds_dwordx4: no
// staging registers, no ds_write, and the returning data does not compete with the MFMAs for
// the vector register file (measured on this chip: with the same bytes per flop a MFMA loop
// fed by register loads sustains about 100 TFLOP/s, fed by LDS-direct loads about 125).
// One such instruction writes 64 lanes x 16 bytes to 1 KB of consecutive LDS, lane l at
// base + 16 l, each lane from its own global address; the tile layout in LDS is therefore
// chosen through which 16-byte chunk each lane fetches:
//   K-contiguous tile [64 rows][8 chunks]: one instruction = 8 rows; lane (r, c') fetches chunk
//     c = c' ^ ((r >> 1) & 7) of tile row r.  A row is 32 floats, so rows r and r + 2 start on the same
//     bank and the 16 (row parity, position) slots of 16 bytes span the 64 banks once: with the key taken
//     from r >> 1 the 16-byte reads "chunk c of 16 consecutive rows" land on 16 different slots
//     (keyed by r & 7 alone, rows r and r + 8 shared a slot: a two-way conflict on every read);
//   row-contiguous tile [16 k][32 chunks]: one instruction = 2 rows, stored as they lie.
// ---------------------------------------------------------------------------------------
// ROWS = rows of a K-contiguous tile resp. columns of a row-contiguous one (64 or 32): ROWS / 8 blocks
// of 1 KB, dealt round-robin to the NW waves of the workgroup.
template <bool KC, int ROWS, int NW>
__device__ __forceinline__ void lds_direct_tile(const float2 *__restrict__ Mq, int ld, int r0, int c0,
                                                float *lds, int wave, int lane)
{
    constexpr int NBLK = ROWS / 8;
#pragma unroll
    for (int j = 0; j < (NBLK + NW - 1) / NW; ++j) {
        const int blk = j * NW + wave;  // 1 KB block of the tile
        if (blk < NBLK) {
            const float2 *g;
            if (KC) {  // rows r0 + 8 blk .. +7, complex k c0 .. c0+15
                const int rl = lane >> 3, cs = lane & 7;
                g = Mq + (long)(r0 + 8 * blk + rl) * ld + c0 + 2 * (cs ^ (((8 * blk + rl) >> 1) & 7));
            } else {   // 16-byte chunk c of the tile stored as it lies: k row c / (ROWS/2), complex columns 2 (c % (ROWS/2))
                const int c = blk * 64 + lane;
                const int kl = c / (ROWS / 2), cs = c % (ROWS / 2);
                g = Mq + (long)(r0 + kl) * ld + c0 + 2 * cs;
            }
            __builtin_amdgcn_global_load_lds(
                (const void __attribute__((address_space(1))) *)g,
                (void __attribute__((address_space(3))) *)(lds + blk * 256), 16, 0, 0);
        }
    }
}

// s_waitcnt vmcnt(n) alone (expcnt and lgkmcnt left at their maxima)
template <int n>
__device__ __forceinline__ void wait_vmcnt()
{
    static_assert(n >= 0 && n < 64, "vmcnt is a 6-bit field");
    __builtin_amdgcn_s_waitcnt(0x0f70 | (n & 15) | ((n >> 4) << 14));
}

// Workgroup barrier without the memory fence of __syncthreads().  The fence makes the compiler put a
// wait for every outstanding vector-memory operation in front of the barrier; the tile loop states its
// own, narrower, condition: this wave's loads of the next tile have landed (wait_vmcnt) and its LDS reads
// of the current tile have returned (lgkmcnt(0)).  The "memory" clobber keeps the compiler from moving LDS
// accesses across.  Measured: 130 x 128x1024x1024 916 -> 883 us, 130 x 128x1024x512 502 -> 473 us.
__device__ __forceinline__ void tile_barrier()
{
    asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
}

// One 64 x (32 WN) tile by 2 x WN waves, workgroup index wg = frequency * tiles + tile.
// lds: A tiles (8 KB) and B tiles (4 WN KB), double-buffered: the next tile lands while this one is
// multiplied.  Measured alternatives that did not pay: a ring of three or four tiles in flight (the
// loop never waits for a load: 0.03 us of 16.5 us at 144 x 128^3; 21.4 -> 21.7 / 24.1 us), and two
// wave groups per tile that each take half of K to double the waves per SIMD (21.2 -> 24.9 us).
template <int MODE, int WN>
__device__ __forceinline__ void ldsdirect_body(float *lds, const float2 *__restrict__ A,
                                               const float2 *__restrict__ B, float2 *__restrict__ C,
                                               int M, int N, int K, float alpha, int accumulate,
                                               int tilesM, int tilesN, int wg, int q_base, const FreqMap &fm)
{
    constexpr bool A_KC = (MODE != 2);
    constexpr bool B_KC = (MODE == 0);
    constexpr int BNW = 32 * WN;           // tile columns
    constexpr int NW = 2 * WN;             // waves
    constexpr int TILE = 64 * KT * 2;      // floats per A tile (8 KB)
    constexpr int TILEB = BNW * KT * 2;    // floats per B tile
    constexpr int LDB = 2 * BNW;           // floats per k row of a row-contiguous B tile
    // buffer b of A at lds + b * TILE, of B at lds + 2 * TILE + b * TILEB

    const int tiles = tilesM * tilesN;
    const int qi = wg / tiles;
    const int tile = wg - qi * tiles;
    const int q = map_freq(q_base + qi, fm);
    // Consecutive workgroups (dispatched together, in step through K) walk along the dimension with
    // fewer tiles, so that the few tiles which share the other operand's panel read it at the same time;
    // the panels they do not share are the small ones and stay in the L2 for the whole frequency.
    // Measured at 130 x 128x1024x1024: bytes fetched 1.44 -> 1.06 x the operands, 884 -> 880 us.
    int tm, tn;
    if (tilesM < tilesN) {
        tn = tile / tilesM;
        tm = tile - tn * tilesM;
    } else {
        tm = tile / tilesN;
        tn = tile - tm * tilesN;
    }
    const int m0 = tm * BM;
    const int n0 = tn * BNW;
    const float2 *Aq = A + (long)q * M * K;
    const float2 *Bq = B + (long)q * N * K;
    float2 *Cq = C + (long)q * M * N;

    const int tid = threadIdx.x;
    const int lane = tid & 63, wave = tid >> 6;
    const int wm = wave / WN, wn = wave % WN;
    const int li = lane & 31, h = lane >> 5;

    floatx16 p1, p2, p3;
#pragma unroll
    for (int r = 0; r < 16; ++r) { p1[r] = 0.f; p2[r] = 0.f; p3[r] = 0.f; }

    const int nk = K / KT;
    auto issue = [&](int kt, int buf) {
        const int k0 = kt * KT;
        float *ab = lds + buf * TILE, *bb = lds + 2 * TILE + buf * TILEB;
        if (A_KC) lds_direct_tile<true, 64, NW>(Aq, K, m0, k0, ab, wave, lane);    // A[m][k]
        else      lds_direct_tile<false, 64, NW>(Aq, M, k0, m0, ab, wave, lane);   // A[k][m]
        if (B_KC) lds_direct_tile<true, BNW, NW>(Bq, K, n0, k0, bb, wave, lane);   // B[n][k]
        else      lds_direct_tile<false, BNW, NW>(Bq, N, k0, n0, bb, wave, lane);  // B[k][n]
    };

    issue(0, 0);
    wait_vmcnt<0>();
    tile_barrier();

    const int arow = 32 * wm + li, bcol = 32 * wn + li;
    // swizzled position of 16-byte chunk c of a K-contiguous row: row * 32 floats + 4 * (c ^ key(row))
    const int a_blk = arow * 32, a_x = (arow >> 1) & 7;
    const int b_blk = bcol * 32, b_x = (bcol >> 1) & 7;

    for (int kt = 0; kt < nk; ++kt) {
        const int buf = kt & 1;
        if (kt + 1 < nk) issue(kt + 1, buf ^ 1);  // asynchronous: lands while this tile is multiplied

        const float *as = lds + buf * TILE;
        const float *bs = lds + 2 * TILE + buf * TILEB;
        // all LDS reads of the step first, then its 24 MFMAs: one exposed LDS latency per step instead of
        // one per pair of k (the compiler otherwise interleaves them to save registers)
        float a[16], b[16];  // (re, im) of the 8 k this half-wave feeds
        if (A_KC) {
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const float4 va = *reinterpret_cast<const float4 *>(as + a_blk + (((4 * h + j) ^ a_x) << 2));
                a[4 * j] = va.x; a[4 * j + 1] = va.y; a[4 * j + 2] = va.z; a[4 * j + 3] = va.w;
            }
        } else {
#pragma unroll
            for (int kk = 0; kk < 8; ++kk) {
                // half-wave h owns k = 8h + kk: both components of A[k][arow]
                const float2 va = *reinterpret_cast<const float2 *>(as + (8 * h + kk) * LDM + 2 * arow);
                a[2 * kk] = va.x; a[2 * kk + 1] = va.y;
            }
        }
        if (B_KC) {
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const float4 vb = *reinterpret_cast<const float4 *>(bs + b_blk + (((4 * h + j) ^ b_x) << 2));
                b[4 * j] = vb.x; b[4 * j + 1] = vb.y; b[4 * j + 2] = vb.z; b[4 * j + 3] = vb.w;
            }
        } else {
#pragma unroll
            for (int kk = 0; kk < 8; ++kk) {
                const float2 vb = *reinterpret_cast<const float2 *>(bs + (8 * h + kk) * LDB + 2 * bcol);
                b[2 * kk] = vb.x; b[2 * kk + 1] = vb.y;
            }
        }
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int kk = 0; kk < 8; ++kk) cmac3<MODE>(a[2 * kk], a[2 * kk + 1], b[2 * kk], b[2 * kk + 1], p1, p2, p3);
        if (kt + 1 < nk) {
            wait_vmcnt<0>();  // this lane's share of the next tile is in LDS
            tile_barrier();   // ... and everyone's; nobody still reads the other buffer
        }
    }

    floatx16 cre, cim;
    combine3<MODE>(p1, p2, p3, cre, cim);
#pragma unroll
    for (int r = 0; r < 16; ++r) {
        const int row = m0 + 32 * wm + 8 * (r / 4) + 4 * h + (r % 4);
        const int col = n0 + 32 * wn + li;
        float2 v = make_float2(alpha * cre[r], alpha * cim[r]);
        float2 *dst = Cq + (long)row * N + col;
        if (accumulate & RESULT_ACCUMULATE) {
            const float2 o = *dst;
            v.x += o.x;
            v.y += o.y;
        }
        store_result(dst, v, accumulate);
    }
}

constexpr int ldsdirect_floats(int wn) { return 2 * (64 * KT * 2 + 32 * wn * KT * 2); }
constexpr int LDSDIRECT_FLOATS = ldsdirect_floats(2);  // 32 KB

// WN = 2: 64x64 tiles, 256 lanes.  WN = 1: 64x32 tiles, 128 lanes (N a multiple of 96 but not of 64).
template <int MODE, int WN>
__global__ __launch_bounds__(128 * WN) void cgemm_ldsdirect_kernel(const float2 *__restrict__ A,
                                                                  const float2 *__restrict__ B,
                                                                  float2 *__restrict__ C, int M, int N,
                                                                  int K, float alpha, int accumulate,
                                                                  int tilesM, int tilesN, int total_wgs,
                                                                  int chunk, FreqMap fm)
{
    __shared__ __align__(16) float lds[ldsdirect_floats(WN)];
    const int wg = (int)(blockIdx.x % 8) * chunk + (int)(blockIdx.x / 8);
    if (wg >= total_wgs) return;
    ldsdirect_body<MODE, WN>(lds, A, B, C, M, N, K, alpha, accumulate, tilesM, tilesN, wg, 0, fm);
}

#ifdef FBFC_PROBES  // only in the measurement library (libfbfftconv_probe.so), never in the shipped one
// Measurement variant of the 64x64 tile kernel: each workgroup also adds the shader-clock ticks
// (s_memtime) and the 100 MHz ticks (s_memrealtime) it lived for to ticks[0] and ticks[1]; their ratio
// is the clock the kernel actually ran at.  Under sustained fp32 MFMA load the chip settles well below its
// 2.4 GHz peak clock, which is what the MFMA roofline is quoted at.
template <int MODE>
__global__ __launch_bounds__(256) void cgemm_ldsdirect_clock_kernel(const float2 *__restrict__ A,
                                                                    const float2 *__restrict__ B,
                                                                    float2 *__restrict__ C, int M, int N,
                                                                    int K, float alpha, int tilesM, int tilesN,
                                                                    int total_wgs, int chunk,
                                                                    unsigned long long *ticks)
{
    __shared__ __align__(16) float lds[ldsdirect_floats(2)];
    const int wg = (int)(blockIdx.x % 8) * chunk + (int)(blockIdx.x / 8);
    if (wg >= total_wgs) return;
    const long long c0 = clock64(), w0 = wall_clock64();
    ldsdirect_body<MODE, 2>(lds, A, B, C, M, N, K, alpha, 0, tilesM, tilesN, wg, 0, FreqMap{0, 1, 0});
    if (threadIdx.x == 0) {
        atomicAdd(ticks, (unsigned long long)(clock64() - c0));
        atomicAdd(ticks + 1, (unsigned long long)(wall_clock64() - w0));
    }
}
#endif  // FBFC_PROBES

// ---------------------------------------------------------------------------------------
// Split-K kernel for small problems (few 64x64 tiles per CU).
//
// With only a handful of output tiles per SIMD, whole tiles cannot be balanced over the 1024
// SIMDs (config 4 has 2.25 32x32-complex blocks per SIMD).  Here a workgroup owns ONE 32x32
// complex block and its four waves each contract a quarter of K, so the unit of scheduling
// is a quarter block (9 per SIMD for config 4).  Operands go straight from global memory into
// the MFMA operand registers (each lane loads exactly the k' it feeds: 64 contiguous bytes of
// a K-contiguous row, or one complex per row of a row-contiguous operand); LDS is used only
// to add the partial accumulators.  Preconditions: K % (16 * SK) == 0; M and N may be ragged (the lanes past
// an edge load the last row or column again and store nothing)
// (SK = waves that share one block: 4, 2 or 1; with SK = 1 a workgroup is four independent blocks).
// ---------------------------------------------------------------------------------------
template <int MODE>
__device__ __forceinline__ void splitk_load(const float2 *__restrict__ Aq, const float2 *__restrict__ Bq,
                                            int M, int N, int K, int arow, int bcol, int k0, int h,
                                            float (&a)[16], float (&b)[16])
{
    constexpr bool A_KC = (MODE != 2);
    constexpr bool B_KC = (MODE == 0);
    if (A_KC) {  // A[m][k]: 8 consecutive complex of row arow
        const float4 *p = reinterpret_cast<const float4 *>(Aq + (long)arow * K + k0 + 8 * h);
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const float4 v = p[j];
            a[4 * j] = v.x; a[4 * j + 1] = v.y; a[4 * j + 2] = v.z; a[4 * j + 3] = v.w;
        }
    } else {     // A[k][m]: column arow of 8 consecutive rows
        const float2 *p = Aq + (long)(k0 + 8 * h) * M + arow;
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            const float2 v = p[(long)j * M];
            a[2 * j] = v.x; a[2 * j + 1] = v.y;
        }
    }
    if (B_KC) {  // B[n][k]
        const float4 *p = reinterpret_cast<const float4 *>(Bq + (long)bcol * K + k0 + 8 * h);
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const float4 v = p[j];
            b[4 * j] = v.x; b[4 * j + 1] = v.y; b[4 * j + 2] = v.z; b[4 * j + 3] = v.w;
        }
    } else {     // B[k][n]
        const float2 *p = Bq + (long)(k0 + 8 * h) * N + bcol;
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            const float2 v = p[(long)j * N];
            b[2 * j] = v.x; b[2 * j + 1] = v.y;
        }
    }
}

template <int MODE>
__device__ __forceinline__ void splitk_mfma(const float (&a)[16], const float (&b)[16], floatx16 &p1,
                                            floatx16 &p2, floatx16 &p3)
{
#pragma unroll
    for (int j = 0; j < 8; ++j) cmac3<MODE>(a[2 * j], a[2 * j + 1], b[2 * j], b[2 * j + 1], p1, p2, p3);
}

// red: [wave][accumulator register][lane] partial sums (used when SK > 1)
// RAGGED: M, N need not be multiples of 32 (separate instantiations: the aligned code is the tail of the hybrid
// and grouped kernels and stays as it was)
template <int MODE, int SK, bool RAGGED = false>
__device__ __forceinline__ void splitk_body(float (*red)[32][64], const float2 *__restrict__ A,
                                            const float2 *__restrict__ B, float2 *__restrict__ C, int M,
                                            int N, int K, float alpha, int accumulate, int tilesM,
                                            int tilesN, int total_tiles, int wg, int q_base, const FreqMap &fm)
{
    constexpr int TPW = 4 / SK;  // 32x32 blocks per workgroup; SK waves share one block's K range
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int li = lane & 31, h = lane >> 5;
    const int ks = wave % SK;  // which share of K
    const int gtile = wg * TPW + wave / SK;
    // consecutive blocks run along N: the waves of a workgroup share rows of A (through L1)
    const bool live = gtile < total_tiles;
    const int tiles = tilesM * tilesN;
    const int qi = live ? gtile / tiles : 0;
    const int tile = live ? gtile - qi * tiles : 0;
    const int q = map_freq(q_base + qi, fm);
    const int m0 = (tile / tilesN) * 32;
    const int n0 = (tile % tilesN) * 32;
    const float2 *Aq = A + (long)q * M * K;
    const float2 *Bq = B + (long)q * N * K;
    float2 *Cq = C + (long)q * M * N;

    // ragged M, N: the lanes past the edge load the last row / column again and store nothing
    const int arow = (!RAGGED || m0 + li < M) ? m0 + li : M - 1, bcol = (!RAGGED || n0 + li < N) ? n0 + li : N - 1;
    const int kq = K / SK;                    // this wave's share of K (a multiple of 16)
    const int kbeg = ks * kq, nkt = kq >> 4;  // K-tiles of 16 complex

    floatx16 p1, p2, p3;
#pragma unroll
    for (int r = 0; r < 16; ++r) { p1[r] = 0.f; p2[r] = 0.f; p3[r] = 0.f; }

    if (live) {
        if constexpr (SK == 1) {
            // long K loop per wave: explicit register double buffering, loads pinned ahead of the MFMAs
            float a0[16], b0[16], a1[16], b1[16];
            splitk_load<MODE>(Aq, Bq, M, N, K, arow, bcol, kbeg, h, a0, b0);
            int kt = 0;
            for (; kt + 1 < nkt; kt += 2) {
                splitk_load<MODE>(Aq, Bq, M, N, K, arow, bcol, kbeg + 16 * (kt + 1), h, a1, b1);
                __builtin_amdgcn_sched_barrier(0);
                splitk_mfma<MODE>(a0, b0, p1, p2, p3);
                __builtin_amdgcn_sched_barrier(0);
                // the last prefetch of an even count re-reads the final tile and is not used
                const int knext = (kt + 2 < nkt) ? kt + 2 : kt + 1;
                splitk_load<MODE>(Aq, Bq, M, N, K, arow, bcol, kbeg + 16 * knext, h, a0, b0);
                __builtin_amdgcn_sched_barrier(0);
                splitk_mfma<MODE>(a1, b1, p1, p2, p3);
                __builtin_amdgcn_sched_barrier(0);
            }
            if (kt < nkt) splitk_mfma<MODE>(a0, b0, p1, p2, p3);
        } else {
            // one to four K-tiles per wave: the compiler interleaves each tile's loads with the
            // previous tile's MFMAs, and at about 64 registers per lane five workgroups share a CU
            float a[16], b[16];
            for (int kt = 0; kt < nkt; ++kt) {
                splitk_load<MODE>(Aq, Bq, M, N, K, arow, bcol, kbeg + 16 * kt, h, a, b);
                splitk_mfma<MODE>(a, b, p1, p2, p3);
            }
        }
    }

    floatx16 cre, cim;
    combine3<MODE>(p1, p2, p3, cre, cim);  // linear: partial sums combine like whole ones

    if constexpr (SK == 1) {
        if (!live) return;
#pragma unroll
        for (int r = 0; r < 16; ++r) {
            // accumulator register r of lane (li, h) is C[8*(r/4) + 4*h + r%4][li] of the block
            const int row = m0 + 8 * (r / 4) + 4 * h + (r % 4);
            if (RAGGED && (row >= M || n0 + li >= N)) continue;
            float2 v = make_float2(alpha * cre[r], alpha * cim[r]);
            float2 *dst = Cq + (long)row * N + n0 + li;
            if (accumulate & RESULT_ACCUMULATE) {
                const float2 o = *dst;
                v.x += o.x;
                v.y += o.y;
            }
            store_result(dst, v, accumulate);
        }
    } else {
        // add the SK partial accumulators of a block: each of its waves finalises 16/SK registers
#pragma unroll
        for (int r = 0; r < 16; ++r) {
            red[wave][r][lane] = cre[r];
            red[wave][16 + r][lane] = cim[r];
        }
        __syncthreads();
        if (!live) return;
        const int w0 = wave - ks;  // first wave of this block
        constexpr int RPW = 16 / SK;
#pragma unroll
        for (int rr = 0; rr < RPW; ++rr) {
            const int r = RPW * ks + rr;
            float sre = 0.f, sim = 0.f;
#pragma unroll
            for (int v = 0; v < SK; ++v) {
                sre += red[w0 + v][r][lane];
                sim += red[w0 + v][16 + r][lane];
            }
            const int row = m0 + 8 * (r / 4) + 4 * h + (r % 4);
            if (RAGGED && (row >= M || n0 + li >= N)) continue;
            float2 v = make_float2(alpha * sre, alpha * sim);
            float2 *dst = Cq + (long)row * N + n0 + li;
            if (accumulate & RESULT_ACCUMULATE) {
                const float2 o = *dst;
                v.x += o.x;
                v.y += o.y;
            }
            store_result(dst, v, accumulate);
        }
    }
}

template <int MODE, int SK, bool RAGGED>
__global__ __launch_bounds__(256) void cgemm_splitk_kernel(const float2 *__restrict__ A,
                                                           const float2 *__restrict__ B,
                                                           float2 *__restrict__ C, int M, int N, int K,
                                                           float alpha, int accumulate, int tilesM,
                                                           int tilesN, int total_tiles, int total_wgs,
                                                           int chunk, FreqMap fm)
{
    __shared__ float red[SK > 1 ? 4 : 1][32][64];
    const int wg = (int)(blockIdx.x % 8) * chunk + (int)(blockIdx.x / 8);
    if (wg >= total_wgs) return;
    splitk_body<MODE, SK, RAGGED>(red, A, B, C, M, N, K, alpha, accumulate, tilesM, tilesN, total_tiles, wg, 0, fm);
}

// ---------------------------------------------------------------------------------------
// Hybrid launch for problems of a few 64x64 tiles per CU.  Whole rounds of tiles (a multiple of
// the 256 CUs) run as LDS-direct tiles; the frequencies left over, which would make a last round
// that fills only part of the chip, run as 32x32 blocks whose K range is split over the four
// waves of a workgroup, so that every CU gets the same share of them.  Workgroups of the first
// kind come first in dispatch order.  Both bodies use the same 32 KB of LDS.
// ---------------------------------------------------------------------------------------
template <int MODE>
__global__ __launch_bounds__(256) void cgemm_hybrid_kernel(const float2 *__restrict__ A,
                                                           const float2 *__restrict__ B,
                                                           float2 *__restrict__ C, int M, int N, int K,
                                                           float alpha, int accumulate, int q_direct,
                                                           int direct_wgs, int chunk_direct,
                                                           int split_tiles, int split_wgs, int chunk_split,
                                                           FreqMap fm)
{
    __shared__ __align__(16) float lds[LDSDIRECT_FLOATS];
    static_assert(LDSDIRECT_FLOATS == 4 * 32 * 64, "both bodies share one buffer");
    const int x = (int)(blockIdx.x % 8), j = (int)(blockIdx.x / 8);
    if (j < chunk_direct) {
        const int wg = x * chunk_direct + j;
        if (wg >= direct_wgs) return;
        ldsdirect_body<MODE, 2>(lds, A, B, C, M, N, K, alpha, accumulate, M / 64, N / 64, wg, 0, fm);
    } else {
        const int wg = x * chunk_split + (j - chunk_direct);
        if (wg >= split_wgs) return;
        // the split part starts at frequency q_direct
        splitk_body<MODE, 4>(reinterpret_cast<float (*)[32][64]>(lds), A, B, C, M, N, K, alpha, accumulate,
                             M / 32, N / 32, split_tiles, wg, q_direct, fm);
    }
}

static void note_kernel(const char *base, int mode, int variant, long grid_items)
{
    char name[64];
    if (variant >= 0) snprintf(name, sizeof name, "%s<%d, %d>", base, mode, variant);
    else snprintf(name, sizeof name, "%s<%d>", base, mode);
    kernel_log_add(name, grid_items);
}

template <int MODE, int SK>
static hipError_t launch_splitk(const float *A, const float *B, float *C, int n_freq, int m, int n,
                                int k, float alpha, int accumulate, FreqMap fm, hipStream_t s)
{
    const int tm = (m + 31) / 32, tn = (n + 31) / 32;
    const long tot32 = (long)n_freq * tm * tn;
    const long wgs = (tot32 * SK + 3) / 4;
    const int chunk = (int)((wgs + 7) / 8);
    note_kernel("cgemm_splitk_kernel", MODE, SK, (long)chunk * 8 * 256);
    const float2 *A2 = reinterpret_cast<const float2 *>(A), *B2 = reinterpret_cast<const float2 *>(B);
    float2 *C2 = reinterpret_cast<float2 *>(C);
    if ((m % 32) != 0 || (n % 32) != 0)
        FBFC_LAUNCH((cgemm_splitk_kernel<MODE, SK, true>), dim3((unsigned)(chunk * 8)), dim3(256), 0, s, A2, B2, C2,
                    m, n, k, alpha, accumulate, tm, tn, (int)tot32, (int)wgs, chunk, fm);
    else
        FBFC_LAUNCH((cgemm_splitk_kernel<MODE, SK, false>), dim3((unsigned)(chunk * 8)), dim3(256), 0, s, A2, B2, C2,
                    m, n, k, alpha, accumulate, tm, tn, (int)tot32, (int)wgs, chunk, fm);
    return hipGetLastError();
}

// A forced kernel variant (for measurements; see fbfc_debug_force_contraction_kernel): -1 = the
// shape rule below, 0 = register-staged LDS tiles, 8 = LDS-direct tiles, 9 = hybrid of LDS-direct
// tiles and split blocks, 1 / 2 / 4 = register-fed kernel with that many waves per block.
static std::atomic<int> g_force_variant{-1};
void cgemm_force_variant(int v) { g_force_variant.store(v); }
static int splitk_override() { return g_force_variant.load(std::memory_order_relaxed); }


// Which kernel a problem takes (measured on MI355X):
//  * a few rounds of 64x64 tiles whose last round would fill at most half the chip: whole rounds as
//    LDS-direct tiles, the rest as split blocks (25 vs 31 us at 144 x 128^3, 28.4 vs 30.5 at
//    544 x 128x64x64; with a fuller last round plain tiles are as fast);
//  * N a multiple of 96 but not of 64 (96 input planes): 64x32 tiles by two waves.  At 2112 frequencies
//    256x96x64 conj(A)^T B takes 268 us (284 with 64x96 tiles by six waves, 321 with the register-fed
//    kernel); 64x96x256 A B is as fast either way (251 us) and keeps the register-fed kernel;
//  * at least 4 full 64x64 tiles per CU, or at least one and K >= 32, and 64-aligned M, N: LDS-direct tiles;
//  * otherwise, if K is a multiple of 16 and M, N are multiples of 32 (or the problem is small, or a side is
//    under 32): the register-fed kernel, with more waves sharing one block's K range the fewer blocks there
//    are per SIMD;
//  * anything else: register-staged LDS tiles with bounds checks.
enum Variant { V_INVALID, V_HYBRID, V_TILES32, V_SPLIT4, V_SPLIT2, V_SPLIT1, V_TILES, V_STAGED };
struct Choice {
    Variant v;
    int q_direct;  // V_HYBRID: frequencies [0, q_direct) as tiles, the rest as split blocks
};

static Choice choose_variant(int mode, const float *A, const float *B, int n_freq, int m, int n, int k)
{
    const int tilesM = (m + BM - 1) / BM, tilesN = (n + BN - 1) / BN;
    const long total = (long)n_freq * tilesM * tilesN;
    if (total <= 0 || total > 0x7fffff00L) return {V_INVALID, 0};
    const bool aligned16 = ((reinterpret_cast<uintptr_t>(A) | reinterpret_cast<uintptr_t>(B)) & 15) == 0;
    const int force = splitk_override();
    const bool direct_ok = (m % 64) == 0 && (n % 64) == 0 && (k % 16) == 0 && aligned16;
    const long tot32 = (long)n_freq * ((m + 31) / 32) * ((n + 31) / 32);
    if (direct_ok && (k % 64) == 0 &&
        (force == 9 || (force < 0 && total >= 256 && total < 8 * 256 && total % 256 <= 128))) {
        const int t64 = tilesM * tilesN;
        const int q_direct = (int)((total / 256) * 256 / t64);
        if (n_freq - q_direct > 0 && q_direct > 0) return {V_HYBRID, q_direct};
    }
    if ((mode != 1 || force == 8) && (m % 64) == 0 && (n % 96) == 0 && (n % 64) != 0 && (k % 16) == 0 && aligned16 &&
        (force == 8 || (force < 0 && (long)n_freq * (m / 64) * (n / 96) >= 4 * 256)))
        return {V_TILES32, 0};
    // one to four rounds of tiles that the hybrid does not take (a last round more than half full, or none):
    // whole tiles still beat the register-fed kernel once K is 32 or more (128^3 per frequency: 480 tiles
    // 16.9 against 21.0 us, 512 tiles 17.3 against 21.6, 768 tiles 24.4 against 32.1, 256 tiles 11.1 against 11.9;
    // 130 x 128x128x32: 8.5 against 10.1)
    const bool prefer_direct = direct_ok && (force == 8 || (force < 0 && (total >= 4 * 256 || (total >= 256 && k >= 32))));
    // Ragged M or N (the lanes past the edge are masked): the register-fed kernel for small problems and for
    // sides under 32, where the staged kernel's 64 x 64 tiles are mostly empty (130 x 16x128x128: 9.6 against
    // 17.9 us, 128x3x128: 9.4 against 18.0, 100x128x128: 27.2 against 28.0); from about four blocks per SIMD on
    // the staged kernel's tiles win (528 x 100x64x64: 24.6 against 27.5 us, 2112 x 64x250x96: 239 against 276)
    const bool ragged = (m % 32) != 0 || (n % 32) != 0;
    const bool regs_ok = !ragged || force > 0 || tot32 < 4 * 1024 || m < 32 || n < 32;
    if (!prefer_direct && regs_ok && (k % 16) == 0 && aligned16 && tot32 * 4 < 0x7fffff00L && force != 0) {
        int sk = 0;
        if (force >= 0) sk = (force == 8) ? 0 : force;
        else if (tot32 < 4 * 1024 && (k % 64) == 0) sk = 4;
        else if (tot32 < 8 * 1024 && (k % 32) == 0) sk = 2;
        else sk = 1;
        if (sk == 4 && (k % 64) == 0) return {V_SPLIT4, 0};
        if (sk == 2 && (k % 32) == 0) return {V_SPLIT2, 0};
        if (sk == 1) return {V_SPLIT1, 0};
    }
    if (direct_ok && force != 0) return {V_TILES, 0};
    return {V_STAGED, 0};
}

static int result_flags(int accumulate, int n_freq, int m, int n)
{
    return (accumulate ? RESULT_ACCUMULATE : 0) | (stream_bytes((long)n_freq * m * n * 8) ? RESULT_STREAM : 0);
}

template <int MODE>
static hipError_t launch_mode(const float *A, const float *B, float *C, int n_freq, int m, int n,
                              int k, float alpha, int accumulate, FreqMap fm, hipStream_t s)
{
    const int tilesM = (m + BM - 1) / BM, tilesN = (n + BN - 1) / BN;
    const long total = (long)n_freq * tilesM * tilesN;
    const Choice ch = choose_variant(MODE, A, B, n_freq, m, n, k);
    accumulate = result_flags(accumulate, n_freq, m, n);
    const float2 *A2 = reinterpret_cast<const float2 *>(A), *B2 = reinterpret_cast<const float2 *>(B);
    float2 *C2 = reinterpret_cast<float2 *>(C);
    const int chunk = (int)((total + 7) / 8);
    switch (ch.v) {
        case V_HYBRID: {
            const int t64 = tilesM * tilesN;
            const int direct_wgs = ch.q_direct * t64;
            const int split_tiles = (n_freq - ch.q_direct) * (m / 32) * (n / 32);  // one workgroup per 32x32 block
            const int chunk_direct = (direct_wgs + 7) / 8, chunk_split = (split_tiles + 7) / 8;
            note_kernel("cgemm_hybrid_kernel", MODE, -1, (long)(chunk_direct + chunk_split) * 8 * 256);
            FBFC_LAUNCH(cgemm_hybrid_kernel<MODE>, dim3((unsigned)((chunk_direct + chunk_split) * 8)),
                               dim3(256), 0, s, A2, B2, C2, m, n, k, alpha, accumulate, ch.q_direct, direct_wgs,
                               chunk_direct, split_tiles, split_tiles, chunk_split, fm);
            return hipGetLastError();
        }
        case V_TILES32: {
            const int t32 = n / 32;
            const long tot = (long)n_freq * tilesM * t32;
            const int c32 = (int)((tot + 7) / 8);
            note_kernel("cgemm_ldsdirect_kernel", MODE, 1, (long)c32 * 8 * 128);
            FBFC_LAUNCH((cgemm_ldsdirect_kernel<MODE, 1>), dim3((unsigned)(c32 * 8)), dim3(128), 0, s, A2, B2,
                               C2, m, n, k, alpha, accumulate, tilesM, t32, (int)tot, c32, fm);
            return hipGetLastError();
        }
        case V_SPLIT4: return launch_splitk<MODE, 4>(A, B, C, n_freq, m, n, k, alpha, accumulate, fm, s);
        case V_SPLIT2: return launch_splitk<MODE, 2>(A, B, C, n_freq, m, n, k, alpha, accumulate, fm, s);
        case V_SPLIT1: return launch_splitk<MODE, 1>(A, B, C, n_freq, m, n, k, alpha, accumulate, fm, s);
        case V_TILES:
            note_kernel("cgemm_ldsdirect_kernel", MODE, 2, (long)chunk * 8 * 256);
            FBFC_LAUNCH((cgemm_ldsdirect_kernel<MODE, 2>), dim3((unsigned)(chunk * 8)), dim3(256), 0, s, A2,
                               B2, C2, m, n, k, alpha, accumulate, tilesM, tilesN, (int)total, chunk, fm);
            return hipGetLastError();
        case V_STAGED:
            note_kernel("cgemm_freq_kernel", MODE, -1, (long)chunk * 8 * 256);
            FBFC_LAUNCH(cgemm_freq_kernel<MODE>, dim3((unsigned)(chunk * 8)), dim3(256), 0, s, A2, B2, C2, m,
                               n, k, alpha, accumulate, tilesM, tilesN, (int)total, chunk, fm);
            return hipGetLastError();
        default: return hipErrorInvalidValue;
    }
}

// ---------------------------------------------------------------------------------------
// The two contractions of a backward pass (A B for gradInput, conj(A)^T B for gradWeight) as one
// grid: the tiles of both problems first, then the split blocks of both.  Each problem is cut into
// tiles and blocks exactly as its own launch would cut it and runs the same code, so the results are
// those of two launches; what is saved is one launch and one partly filled last round.
// ---------------------------------------------------------------------------------------
struct MmJob {
    const float2 *A, *B;
    float2 *C;
    int M, N, K;
    float alpha;
    int accumulate;
    int q_direct, direct_wgs, chunk_direct;  // frequencies [0, q_direct) as 64x64 tiles
    int split_tiles, chunk_split;            // the rest as 32x32 blocks, K split over four waves
};

__global__ __launch_bounds__(256) void cgemm_backward_kernel(MmJob j1, MmJob j2, FreqMap fm)
{
    __shared__ __align__(16) float lds[LDSDIRECT_FLOATS];
    const int x = (int)(blockIdx.x % 8);
    int j = (int)(blockIdx.x / 8);
    if (j < j1.chunk_direct) {
        const int wg = x * j1.chunk_direct + j;
        if (wg >= j1.direct_wgs) return;
        ldsdirect_body<1, 2>(lds, j1.A, j1.B, j1.C, j1.M, j1.N, j1.K, j1.alpha, j1.accumulate, j1.M / 64,
                             j1.N / 64, wg, 0, fm);
        return;
    }
    j -= j1.chunk_direct;
    if (j < j2.chunk_direct) {
        const int wg = x * j2.chunk_direct + j;
        if (wg >= j2.direct_wgs) return;
        ldsdirect_body<2, 2>(lds, j2.A, j2.B, j2.C, j2.M, j2.N, j2.K, j2.alpha, j2.accumulate, j2.M / 64,
                             j2.N / 64, wg, 0, fm);
        return;
    }
    j -= j2.chunk_direct;
    if (j < j1.chunk_split) {
        const int wg = x * j1.chunk_split + j;
        if (wg >= j1.split_tiles) return;
        splitk_body<1, 4>(reinterpret_cast<float (*)[32][64]>(lds), j1.A, j1.B, j1.C, j1.M, j1.N, j1.K, j1.alpha,
                          j1.accumulate, j1.M / 32, j1.N / 32, j1.split_tiles, wg, j1.q_direct, fm);
        return;
    }
    j -= j1.chunk_split;
    const int wg = x * j2.chunk_split + j;
    if (wg >= j2.split_tiles) return;
    splitk_body<2, 4>(reinterpret_cast<float (*)[32][64]>(lds), j2.A, j2.B, j2.C, j2.M, j2.N, j2.K, j2.alpha,
                      j2.accumulate, j2.M / 32, j2.N / 32, j2.split_tiles, wg, j2.q_direct, fm);
}

// false: this problem's kernel is not one the grouped grid runs
static bool make_mm_job(int mode, const MmArgs &a, int n_freq, MmJob &j)
{
    const Choice ch = choose_variant(mode, a.A, a.B, n_freq, a.m, a.n, a.k);
    int q_direct;
    if (ch.v == V_HYBRID) q_direct = ch.q_direct;
    else if (ch.v == V_TILES) q_direct = n_freq;
    else if (ch.v == V_SPLIT4 && (a.m % 32) == 0 && (a.n % 32) == 0) q_direct = 0;
    else return false;
    j.A = reinterpret_cast<const float2 *>(a.A);
    j.B = reinterpret_cast<const float2 *>(a.B);
    j.C = reinterpret_cast<float2 *>(a.C);
    j.M = a.m; j.N = a.n; j.K = a.k;
    j.alpha = a.alpha;
    j.accumulate = result_flags(a.accumulate, n_freq, a.m, a.n);
    j.q_direct = q_direct;
    j.direct_wgs = q_direct * (a.m / 64) * (a.n / 64);
    j.chunk_direct = (j.direct_wgs + 7) / 8;
    j.split_tiles = (n_freq - q_direct) * (a.m / 32) * (a.n / 32);
    j.chunk_split = (j.split_tiles + 7) / 8;
    return true;
}

hipError_t launch_cgemm_backward(const MmArgs &gi, const MmArgs &gw, int n_freq, FreqMap fm, hipStream_t s)
{
    MmJob j1, j2;
    if (make_mm_job(1, gi, n_freq, j1) && make_mm_job(2, gw, n_freq, j2)) {
        const long chunks = (long)j1.chunk_direct + j2.chunk_direct + j1.chunk_split + j2.chunk_split;
        if (chunks * 8 < 0x7fffff00L) {
            kernel_log_add("cgemm_backward_kernel", chunks * 8 * 256);
            FBFC_LAUNCH(cgemm_backward_kernel, dim3((unsigned)(chunks * 8)), dim3(256), 0, s, j1, j2, fm);
            return hipGetLastError();
        }
    }
    const hipError_t e = launch_mode<1>(gi.A, gi.B, gi.C, n_freq, gi.m, gi.n, gi.k, gi.alpha, gi.accumulate, fm, s);
    if (e != hipSuccess) return e;
    return launch_mode<2>(gw.A, gw.B, gw.C, n_freq, gw.m, gw.n, gw.k, gw.alpha, gw.accumulate, fm, s);
}

#ifdef FBFC_PROBES
hipError_t launch_cgemm_clock_probe(int mode, const float *A, const float *B, float *C, int n_freq, int m, int n,
                                    int k, unsigned long long *ticks, hipStream_t s)
{
    if (mode < 0 || mode > 2 || (m % 64) != 0 || (n % 64) != 0 || (k % 16) != 0 || m <= 0 || n <= 0 || k <= 0)
        return hipErrorInvalidValue;
    if (((reinterpret_cast<uintptr_t>(A) | reinterpret_cast<uintptr_t>(B)) & 15) != 0) return hipErrorInvalidValue;
    const int tilesM = m / 64, tilesN = n / 64;
    const long total = (long)n_freq * tilesM * tilesN;
    if (total <= 0 || total > 0x7fffff00L) return hipErrorInvalidValue;
    const int chunk = (int)((total + 7) / 8);
    const float2 *A2 = reinterpret_cast<const float2 *>(A), *B2 = reinterpret_cast<const float2 *>(B);
    float2 *C2 = reinterpret_cast<float2 *>(C);
    const dim3 grid((unsigned)(chunk * 8)), block(256);
    switch (mode) {
        case 0: FBFC_LAUNCH(cgemm_ldsdirect_clock_kernel<0>, grid, block, 0, s, A2, B2, C2, m, n, k, 1.0f, tilesM, tilesN, (int)total, chunk, ticks); break;
        case 1: FBFC_LAUNCH(cgemm_ldsdirect_clock_kernel<1>, grid, block, 0, s, A2, B2, C2, m, n, k, 1.0f, tilesM, tilesN, (int)total, chunk, ticks); break;
        default: FBFC_LAUNCH(cgemm_ldsdirect_clock_kernel<2>, grid, block, 0, s, A2, B2, C2, m, n, k, 1.0f, tilesM, tilesN, (int)total, chunk, ticks); break;
    }
    return hipGetLastError();
}
#endif  // FBFC_PROBES

hipError_t launch_cgemm_freq_map(int mode, const float *A, const float *B, float *C, int n_freq, FreqMap fm,
                                 int m, int n, int k, float alpha, int accumulate, hipStream_t s)
{
    switch (mode) {
        case 0: return launch_mode<0>(A, B, C, n_freq, m, n, k, alpha, accumulate, fm, s);
        case 1: return launch_mode<1>(A, B, C, n_freq, m, n, k, alpha, accumulate, fm, s);
        case 2: return launch_mode<2>(A, B, C, n_freq, m, n, k, alpha, accumulate, fm, s);
        default: return hipErrorInvalidValue;
    }
}

hipError_t launch_cgemm_freq(int mode, const float *A, const float *B, float *C, int n_freq, int m,
                             int n, int k, float alpha, int accumulate, hipStream_t s)
{
    return launch_cgemm_freq_map(mode, A, B, C, n_freq, FreqMap{0, 1, 0}, m, n, k, alpha, accumulate, s);
}

}  // namespace fbfc
