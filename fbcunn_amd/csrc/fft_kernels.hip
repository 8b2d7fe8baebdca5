// Batched 2-D real<->complex FFT kernels for gfx950 (power-of-two N, 8..128).
//
// Replaces what the reference asks of fbcuda's fbfft2D / fbifft2D through
// src/fft/FBFFTHost.cpp:39-116 (call sites :86-88, :93, :101-111): implicit zero
// padding at (padU, padL) on the way in, crop at (padU, padL) on the way out,
// Hermitian half spectrum, unnormalised inverse.
//
// Design (one workgroup = T consecutive planes, T*N/2 lanes: 256, or 512 for N = 64):
//   * the T planes are one contiguous chunk of the real tensor: it is copied to
//     LDS with fully coalesced loads;
//   * row pass: one lane transforms TWO real rows at once as one complex
//     length-N FFT held entirely in registers (z = rowA + i rowB) and untangles
//     the two Hermitian spectra; columns 0 and N/2 of a real row spectrum are
//     real, so they share one complex slot and the tile is exactly N/2 wide;
//   * the tile R[y][kx][t] (plane index t fastest) lives in LDS, aliasing the
//     staging chunk; every canvas row has its fixed place in it;
//   * column pass: one lane transforms one column (N complex points) in
//     registers; the lane owning slot 0 untangles columns 0 and N/2;
//   * results go straight from registers to the frequency-major buffer
//     freq[(ky*(N/2+1)+kx)*planes + plane]: the T lanes that share a frequency
//     write T consecutive complex numbers (T*8 bytes, 128 B for N=32).
// The inverse kernel is the mirror image and adds the bias while cropping.
#include <hip/hip_runtime.h>

#include <atomic>
#include <cstdio>
#include <mutex>

#include "bias_dc.h"
#include "fft_regs.h"
#include "fft_stage.h"
#include "fft_windows.h"
#include "kernels.h"
#include "store_nt.h"

namespace fbfc {

// SMALL: the forward variant for planes of at most 16 x 16 at N = 64: its tile has so few rows that
// all columns fit at once, so it runs in one phase (144 -> 137 us for 24576 planes of 9 x 9).
template <int N, bool INVERSE = false, bool SMALL = false, int PHASES = 0>
struct FftShape {
    // planes per workgroup: 256 lanes' worth, except N = 64, which takes 16 planes (512 lanes) so
    // that its runs per frequency are whole 128-byte lines -- measured with the bare
    // access pattern (contiguous reads, frequency-major writes, no arithmetic) at 16384 planes of
    // 47 x 47: 123 us with 64-byte runs from two 256-lane workgroups per CU, 89 us with 128-byte runs
    // from one 512-lane workgroup; at 24576 planes of 9 x 9: 128 against 90 us
    static constexpr int T = (N == 64) ? 16 : 512 / N;
    static constexpr int THREADS = T * N / 2;
    static constexpr int NH2 = N / 2;       // complex slots per tile row
    static constexpr int NH = N / 2 + 1;    // stored column frequencies
    // Phases: the LDS tile holds NH2/PH of the tile columns at a time (the others wait in registers)
    // and the input / output staging area T/PH planes at a time.  N >= 64: two phases, a whole tile
    // would not fit the 160 KB of LDS (N = 128 ran in four until the waiting columns made it spill).
    // N = 32 forward: two phases halve the LDS footprint and a third workgroup fits a CU, measured
    // 19.6 -> 17.4 us for config 3's pair of transforms; the inverse keeps one unless the launch is large.
    // PHASES > 0 overrides the choice (the N = 32 inverse of many planes, see launch_inv)
    static constexpr int PH = PHASES > 0 ? PHASES : SMALL ? 1 : (N >= 64) ? 2 : (N == 32 && !INVERSE) ? 2 : 1;
    static constexpr int KXP = NH2 / PH;    // tile columns per phase
    static constexpr int TP = T / PH;       // planes per staging round
    // waves per SIMD the register budget is sized for (N = 128 keeps 256 values per lane)
    static constexpr int MIN_WAVES = SMALL ? 2 : (N >= 128) ? 1 : (N == 32 && !INVERSE) ? 3 : PH;
    // padding (in complex elements) between tile rows.  A wave of the row pass holds TP planes
    // (2 TP dwords side by side) of 64 / TP row pairs, two tile rows apart; a row stride of
    // TP / 2 (mod 16) complex elements puts consecutive row pairs 2 TP banks apart, so the wave's
    // 128 dwords tile the 64 banks exactly twice.
    static constexpr int ROWPAD = (TP >= 32) ? 0 : (TP >= 2) ? TP / 2 : 1;
    static constexpr int ROWSTRIDE = KXP * T + ROWPAD;  // complex elements
    // lanes of one staging round (the row pass of round r runs on waves [r LPR/64, (r+1) LPR/64))
    static constexpr int LPR = THREADS / PH;
};

static std::atomic<int> g_stream_override{-1};
int spectrum_stream_override() { return g_stream_override.load(std::memory_order_relaxed); }
void spectrum_stream_force(int v) { g_stream_override.store(v); }

// whether this kernel's runs per frequency are whole 128-byte lines
template <int N>
constexpr bool whole_lines() { return FftShape<N, false>::T * 8 >= 128; }

// Windowed operands: virtual plane v = (b * nt + tile) * d1 + c, so the workgroups of one tile (d1 / T of
// them) are followed by those of the next tile -- on other XCDs, although neighbouring windows of one
// image plane share cache lines (a 128-byte window row at an arbitrary offset touches two lines).  With
// remap set, launch index j = 8 r + x is given group u = 8 (r / nt) + x of the d0 * d1 / T (batch, plane
// group) pairs and tile r % nt: XCD x walks through the tiles of its groups one after the other, and the
// shared lines are still in its L2.  Needs d1 % T == 0 and (d0 * d1 / T) % 8 == 0.
template <int T>
__device__ __forceinline__ long window_block(unsigned j, const Window &w)
{
    const unsigned G = (unsigned)w.d1 / T, nt = (unsigned)w.nt;
    const unsigned x = j & 7u, r = j >> 3;
    const unsigned tile = r % nt, u = (r / nt) * 8u + x;
    const unsigned b = u / G, cg = u - b * G;
    return (long)(b * nt + tile) * G + cg;
}

template <int T>
static int window_remap_ok(const Window &w, long planes)
{
    if (!w.on || w.d1 % T != 0) return 0;
    const long groups = planes / ((long)w.nt * w.d1) * (w.d1 / T);
    return groups % 8 == 0 && planes / T < (1L << 31);
}

// ---------------------------------------------------------------------------------
// Windows (tiled convolution).  A windowed operand is a (d0, d1, img_h, img_w) tensor seen as
// d0 * nt * d1 "virtual planes" of h x w: virtual plane v = (b * nt + tile) * d1 + c is the window
// of plane (b, c) whose corner is (ty * step_y + off_y, tx * step_x + off_x), tile = ty * ntx + tx.
// Reads outside the image give zero, writes outside it are dropped.  The staging area keeps the
// same canvas-row layout (padL = 0 on the way in), so the transforms themselves do not change.
// ---------------------------------------------------------------------------------
// per virtual plane of the workgroup: element offset of its image plane (lo, hi) and window corner
template <int N>
__device__ __forceinline__ void build_window_table(int4 *tbl, const Window &win, long x0, long planes, int tid)
{
    if (tid < FftShape<N>::T) {
        long v = x0 + tid;
        if (v >= planes) v = planes - 1;
        const long vb = v / win.d1;
        const int c = (int)(v - vb * win.d1);
        const long b = vb / win.nt;
        const int tile = (int)(vb - b * win.nt);
        const int ty = tile / win.ntx, tx = tile - ty * win.ntx;
        const long off = (b * win.d1 + c) * ((long)win.img_h * win.img_w);
        tbl[tid] = make_int4((int)(unsigned)(off & 0xffffffffL), (int)(off >> 32),
                             ty * win.step_y + win.off_y, tx * win.step_x + win.off_x);
    }
}

// ---------------------------------------------------------------------------------
// forward: real (planes,h,w) -> freq [N*(N/2+1)][planes] complex
// ---------------------------------------------------------------------------------
// NZ < N: planes of at most NZ x NZ at the canvas origin (convolution kernels): the transforms skip
// the inputs that are known to be zero.
template <int N, bool WIN, int NZ, bool RAW>
__global__ __launch_bounds__((FftShape<N, false, (NZ < N)>::THREADS), (FftShape<N, false, (NZ < N)>::MIN_WAVES)) void rfft2d_kernel(FwdJob job0, FwdJob job1,
                                                                      FwdJob job2, unsigned blocks0,
                                                                      unsigned blocks01)
{
    using S = FftShape<N, false, (NZ < N)>;
    constexpr int T = S::T;
    extern __shared__ __align__(16) float smem[];
    const int tid = threadIdx.x;
    const unsigned v = blockIdx.x;
    // up to three tensors per launch: workgroups [0, blocks0) work on job 0, [blocks0, blocks01) on
    // job 1, the rest on job 2
    const bool second = v >= blocks0, third = v >= blocks01;
    const FwdJob &job = third ? job2 : (second ? job1 : job0);
    const unsigned vfirst = third ? blocks01 : (second ? blocks0 : 0u);
    const float *__restrict__ in = job.in;
    float2 *__restrict__ out = job.out;
    const long planes = job.planes;
    const int h = job.h, w = job.w;
    const int padU = job.padU, padL = job.padL;
    const int vec4 = job.vec4;
    const int herm = job.herm;
    [[maybe_unused]] const Window &win = job.win;
    const int job_tbl_off = job.tbl_off;
    long x0 = plane_group<T>(v - vfirst) * T;
    if constexpr (WIN) {
        if (win.remap) x0 = window_block<T>(v - vfirst, win) * T;
    }
    if (x0 >= planes) return;
    const int np = (int)((planes - x0 < (long)T) ? (planes - x0) : (long)T);
    const int hw = h * w;
    [[maybe_unused]] int4 *tbl = reinterpret_cast<int4 *>(smem + job_tbl_off);
    if constexpr (WIN) {
        if (win.on) build_window_table<N>(tbl, win, x0, planes, tid);
    }
    float re[N], im[N];

    // ---- row pass: lane (t, rp) owns canvas rows 2rp and 2rp+1 of plane t.  The planes are staged
    // TP at a time; the lanes of round r are LPR consecutive ones (whole waves), so a wave runs the
    // row reads of its own round only ----
    const int round_of_lane = tid / S::LPR, rl = tid % S::LPR;
    const int t = round_of_lane * S::TP + rl % S::TP;
    const int rp = rl / S::TP;
    const int ya = 2 * rp, yb = ya + 1;
    const int ia = ya - padU, ib = yb - padU;
    const bool va = (ia >= 0) && (ia < h);
    const bool vb = (ib >= 0) && (ib < h);
    const bool row_active = (t < np) && (va || vb);

    // ---- stage the contiguous chunk of planes in LDS, TP planes per round ----
    constexpr int LDR = Canvas<N>::LDR;
    // Planes of odd height and width are staged raw, by asynchronous LDS-direct loads (their rows fall on
    // different LDS banks by themselves); windowed operands, even sizes (a 32 x 32 plane staged raw puts
    // every row on the same banks) and N = 128 are staged as zero-padded canvas rows.
    static_assert(!RAW || (!WIN && N <= 64), "raw staging: plain operands, N <= 64");
    // raw staging: bit x of colmask = canvas column x lies inside the plane
    [[maybe_unused]] const unsigned long long colmask = ((w >= 64) ? ~0ull : ((1ull << w) - 1ull)) << padL;
    static_for<S::PH>([&](auto hh) {
        constexpr int hs = decltype(hh)::value;
        int nph = np - hs * S::TP;
        nph = nph < 0 ? 0 : (nph > S::TP ? S::TP : nph);
        if (hs > 0) __syncthreads();  // previous round fully read
        if constexpr (RAW) {
            // N floats of slack on either side of the chunk (the first row is read from -padL on, the last
            // one up to N - 1 - padL), then N zeros for the canvas rows outside the plane
            float *raw = smem + N;
            float *zeros = raw + S::TP * hw + N;
            if (hs == 0 && tid < N) zeros[tid] = 0.0f;
            // N >= 64: planes of this size add up to tensors no cache holds until their next use, so
            // they are streamed (non-temporal hint)
            stage_raw<(N >= 64) ? 2 : 0, S::THREADS>(raw, in + (x0 + hs * S::TP) * hw, nph * hw, vec4 != 0, tid);
            __builtin_amdgcn_s_waitcnt(0x0f70);  // vmcnt(0): this wave's pieces have landed
            __syncthreads();
            if (row_active && round_of_lane == hs) {
                const int tl = t - hs * S::TP;
                const float *pa = va ? raw + (tl * h + ia) * w - padL : zeros;
                const float *pb = vb ? raw + (tl * h + ib) * w - padL : zeros;
                static_for<N>([&](auto xx) {
                    constexpr int x = decltype(xx)::value;
                    if constexpr (x < NZ) {
                        // what lies left and right of the row in LDS is masked off bit-wise
                        const unsigned m = ((colmask >> x) & 1ull) ? 0xffffffffu : 0u;
                        re[x] = __uint_as_float(__float_as_uint(pa[x]) & m);
                        im[x] = __uint_as_float(__float_as_uint(pb[x]) & m);
                    } else {
                        re[x] = 0.0f;
                        im[x] = 0.0f;
                    }
                });
            }
        } else {
            bool windowed = false;
            if constexpr (WIN) windowed = win.on != 0;
            // floats between the canvases of two planes, and where the all-zero row lies
            const int pstride = windowed ? window_plane_stride<N>(h) : h * LDR;
            const int zoff = S::TP * pstride;
            if (windowed) {
                if (hs == 0) __syncthreads();  // window table complete
                if (tid < N) smem[zoff + tid] = 0.0f;
                copy_windows<N, true>(smem, const_cast<float *>(in), tbl, hs * S::TP, nph, h, w, 0, win, tid, pstride);
            } else {
                zero_canvas_margins<N, S::THREADS>(smem, nph * h, w, padL, zoff, tid);
                copy_canvas<N, true, S::THREADS>(smem, const_cast<float *>(in) + (x0 + hs * S::TP) * hw, nph * h, w, padL, vec4, tid);
            }
            __syncthreads();
            if (row_active && round_of_lane == hs) {
                const int tl = t - hs * S::TP;
                const float4 *pa = reinterpret_cast<const float4 *>(smem + (va ? tl * pstride + ia * LDR : zoff));
                const float4 *pb = reinterpret_cast<const float4 *>(smem + (vb ? tl * pstride + ib * LDR : zoff));
                static_for<N / 4>([&](auto jj) {
                    constexpr int j = decltype(jj)::value;
                    if constexpr (4 * j < NZ) {
                        const float4 a = pa[j], b = pb[j];
                        re[4 * j] = a.x; re[4 * j + 1] = a.y; re[4 * j + 2] = a.z; re[4 * j + 3] = a.w;
                        im[4 * j] = b.x; im[4 * j + 1] = b.y; im[4 * j + 2] = b.z; im[4 * j + 3] = b.w;
                    } else {
                        re[4 * j] = re[4 * j + 1] = re[4 * j + 2] = re[4 * j + 3] = 0.0f;
                        im[4 * j] = im[4 * j + 1] = im[4 * j + 2] = im[4 * j + 3] = 0.0f;
                    }
                });
            }
        }
    });

    // ---- row FFT and untangling ----
    // A[k] / B[k]: spectra of rows ya / yb; slot 0 carries the real-valued columns 0 and N/2.
    // The first phase's columns go straight to the LDS tile, later ones wait in registers.
    // The tile R[y][kx][t] holds every canvas row the column pass reads (all N, or NZ for small
    // planes) at a fixed place, so the column pass addresses it with compile-time offsets; the lanes
    // whose two rows lie outside the plane write the zeros.
    constexpr int NLATE = S::NH2 - S::KXP;  // 0 when there is a single phase
    constexpr int TROWS = (NZ < N) ? NZ : N;
    float ar[NLATE > 0 ? NLATE : 1], ai[NLATE > 0 ? NLATE : 1], br[NLATE > 0 ? NLATE : 1], bi[NLATE > 0 ? NLATE : 1];
    float2 *R = reinterpret_cast<float2 *>(smem);
    __syncthreads();  // staging area fully consumed; the tile may overwrite it
    if (row_active) {
        fft_inplace_nz<N, NZ, false>(re, im);
        float2 *Ra = R + ya * S::ROWSTRIDE + t;
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
    } else if (t < np && ya < TROWS) {
        // both rows are zero in every phase: written once, the refills below leave them alone
        float2 *Ra = R + ya * S::ROWSTRIDE + t;
        float2 *Rb = Ra + S::ROWSTRIDE;
        static_for<S::KXP>([&](auto kk) {
            constexpr int k = decltype(kk)::value;
            Ra[k * T] = make_float2(0.0f, 0.0f);
            Rb[k * T] = make_float2(0.0f, 0.0f);
        });
    }

    // Each phase: (later phases first refill the tile from registers) then the lanes whose
    // column belongs to the phase pull it into registers, which frees the tile again.
    // Column pass: lane (tc, kx) owns tile column kx of plane tc.
    const int tc = tid % T;
    const int kx = tid / T;
    static_for<S::PH>([&](auto pp) {
        constexpr int ph = decltype(pp)::value;
        if constexpr (ph > 0) {
            __syncthreads();  // previous phase's columns are in registers
            if (row_active) {
                float2 *Ra = R + ya * S::ROWSTRIDE + t;
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
        if ((tc < np) && (kx / S::KXP) == ph) {
            const int kl = kx - ph * S::KXP;
            const float2 *col = R + kl * T + tc;
            static_for<N>([&](auto yy) {
                constexpr int y = decltype(yy)::value;
                if constexpr (y < NZ) {
                    const float2 v = col[y * S::ROWSTRIDE];
                    re[y] = v.x;
                    im[y] = v.y;
                } else {
                    re[y] = 0.0f;
                    im[y] = 0.0f;
                }
            });
        }
    });

    // ---- column FFT and frequency-major store, all lanes at once ----
    if (tc < np) {
        fft_inplace_nz<N, NZ, false>(re, im);
        // address = uniform base (frequency row ky, first plane of the group) + 32-bit lane offset
        const unsigned voff = (unsigned)(((long)kx * planes + tc) * (long)sizeof(float2));
        const unsigned vnyq = (unsigned)(((long)(N / 2) * planes + tc) * (long)sizeof(float2));
        char *obase = reinterpret_cast<char *>(out + x0);
        const long rowbytes = (long)S::NH * planes * (long)sizeof(float2);
        auto store_all = [&](auto mode_tag) {
            constexpr int STREAM = decltype(mode_tag)::value;
            if (kx != 0) {
                static_for<N>([&](auto kk) {
                    constexpr int ky = decltype(kk)::value;
                    store_freq_run<STREAM>(reinterpret_cast<float2 *>(obase + ky * rowbytes + voff),
                                           make_float2(re[brev<N>(ky)], im[brev<N>(ky)]));
                });
            } else {
                // C = FFT(col0 + i colNyq), both real sequences: untangle
                static_for<N>([&](auto kk) {
                    constexpr int ky = decltype(kk)::value;
                    constexpr int kn = (N - ky) % N;
                    const float zr = re[brev<N>(ky)], zi = im[brev<N>(ky)];
                    const float nr = re[brev<N>(kn)], ni = im[brev<N>(kn)];
                    // both columns are spectra of real sequences: rows above N/2 repeat rows below it
                    if (ky <= N / 2 || !herm) {
                        store_freq_run<STREAM>(reinterpret_cast<float2 *>(obase + ky * rowbytes + voff),
                                               make_float2(0.5f * (zr + nr), 0.5f * (zi - ni)));
                        store_freq_run<STREAM>(reinterpret_cast<float2 *>(obase + ky * rowbytes + vnyq),
                                               make_float2(0.5f * (zi + ni), 0.5f * (nr - zr)));
                    }
                });
            }
        };
        with_store_mode<whole_lines<N>()>(job.stream, store_all);
    }
}

// ---------------------------------------------------------------------------------
// inverse: freq [N*(N/2+1)][planes] complex -> real (planes,h,w), unnormalised,
// real[r][s] = y[r+padU][s+padL] (+ bias[plane % bias_period])
// ---------------------------------------------------------------------------------
template <int N, bool WIN, int PHASES = 0>
__global__ __launch_bounds__((FftShape<N, true, false, PHASES>::THREADS), (FftShape<N, true, false, PHASES>::MIN_WAVES)) void irfft2d_kernel(InvJob job0, InvJob job1,
                                                      unsigned blocks0, BiasGradJob bgrad,
                                                      unsigned bgrad_blocks)
{
    using S = FftShape<N, true, false, PHASES>;
    constexpr int T = S::T;
    extern __shared__ __align__(16) float smem[];
    if (blockIdx.x < bgrad_blocks) {
        // an independent small job riding on this launch: the bias gradient of the same pass
        // (1 KB of the dynamic LDS, which is never smaller than one tile row pair)
        bias_grad_dc_body(bgrad, blockIdx.x, reinterpret_cast<float (*)[64]>(smem));
        return;
    }
    const int tid = threadIdx.x;
    const unsigned v = blockIdx.x - bgrad_blocks;
    const bool second = v >= blocks0;
    const InvJob &job = second ? job1 : job0;
    const float2 *__restrict__ in = job.in;
    float *__restrict__ out = job.out;
    const long planes = job.planes;
    const int h = job.h, w = job.w, padU = job.padU, padL = job.padL;
    const float *__restrict__ bias = job.bias;
    const int bias_period = job.bias_period, vec4 = job.vec4, tbl_off = job.tbl_off;
    [[maybe_unused]] const Window &win = job.win;
    long x0 = plane_group<T>(v - (second ? blocks0 : 0u)) * T;
    if constexpr (WIN) {
        if (win.remap) x0 = window_block<T>(v - (second ? blocks0 : 0u), win) * T;
    }
    if (x0 >= planes) return;
    const int np = (int)((planes - x0 < (long)T) ? (planes - x0) : (long)T);
    const int hw = h * w;
    [[maybe_unused]] int4 *tbl = reinterpret_cast<int4 *>(smem + tbl_off);
    if constexpr (WIN) {
        // read again only after the barriers of the passes below
        if (win.on) build_window_table<N>(tbl, win, x0, planes, tid);
    }
    const int t = tid % T;
    float re[N], im[N];
    float2 *R = reinterpret_cast<float2 *>(smem);

    // ---- column pass: lane (t, kx) fetches its whole column and transforms it, all lanes at once ----
    const int kx = tid / T;
    if (t < np) {
        // address = uniform base (frequency row ky, first plane of the group) + 32-bit lane offset
        const unsigned voff = (unsigned)(((long)kx * planes + t) * (long)sizeof(float2));
        const unsigned vnyq = (unsigned)(((long)(N / 2) * planes + t) * (long)sizeof(float2));
        const char *ibase = reinterpret_cast<const char *>(in + x0);
        const long rowbytes = (long)S::NH * planes * (long)sizeof(float2);
        if (kx != 0) {
            static_for<N>([&](auto kk) {
                constexpr int ky = decltype(kk)::value;
                const float2 v = *reinterpret_cast<const float2 *>(ibase + ky * rowbytes + voff);
                re[ky] = v.x;
                im[ky] = v.y;
            });
        } else {
            // pack columns 0 and N/2 (each the spectrum of a real sequence): C = X0 + i XN.  Rows
            // above N/2 are the conjugates of the rows below it and are not read.
            static_for<N / 2 + 1>([&](auto kk) {
                constexpr int ky = decltype(kk)::value;
                const float2 a = *reinterpret_cast<const float2 *>(ibase + ky * rowbytes + voff);
                const float2 b = *reinterpret_cast<const float2 *>(ibase + ky * rowbytes + vnyq);
                re[ky] = a.x - b.y;
                im[ky] = a.y + b.x;
                if constexpr (ky > 0 && ky < N / 2) {
                    re[N - ky] = a.x + b.y;
                    im[N - ky] = b.x - a.y;
                }
            });
        }
        fft_inplace<N, true>(re, im);
    }

    // ---- row pass bookkeeping: lane (tr, rp) rebuilds canvas rows 2rp, 2rp+1 of plane tr.  The
    // planes leave TP at a time; the lanes of round r are LPR consecutive ones (whole waves), so a wave
    // runs the staging writes of its own round only ----
    const int round_of_lane = tid / S::LPR, rl = tid % S::LPR;
    const int tr = round_of_lane * S::TP + rl % S::TP;
    const int rp = rl / S::TP;
    const int ya = 2 * rp, yb = ya + 1;
    const int ia = ya - padU, ib = yb - padU;
    const bool va = (ia >= 0) && (ia < h);
    const bool vb = (ib >= 0) && (ib < h);
    const bool row_active = (tr < np) && (va || vb);
    // Z[k] = Ya[k] + i Yb[k], k = 0..N-1, with Y[N-k] = conj Y[k]
    float zr[N], zi[N];

    static_for<S::PH>([&](auto pp) {
        constexpr int ph = decltype(pp)::value;
        if (ph > 0) __syncthreads();  // previous phase's tile fully read
        if ((t < np) && (kx / S::KXP) == ph) {
            const int kl = kx - ph * S::KXP;
            float2 *col = R + kl * T + t;
            // every canvas row has its fixed place in the tile R[y][kx][t]: compile-time offsets
            static_for<N>([&](auto yy) {
                constexpr int y = decltype(yy)::value;
                col[y * S::ROWSTRIDE] = make_float2(re[brev<N>(y)], im[brev<N>(y)]);
            });
        }
        __syncthreads();
        if (row_active) {
            const float2 *Ra = R + ya * S::ROWSTRIDE + tr;
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
        if (bias != nullptr) bv = bias[(x0 + tr) % bias_period];
    }
    // ---- canvas rows (+bias) into the staging area, cropped coalesced copy-out, TP planes per round ----
    constexpr int LDR = Canvas<N>::LDR;
    static_for<S::PH>([&](auto hh) {
        constexpr int hs = decltype(hh)::value;
        int nph = np - hs * S::TP;
        nph = nph < 0 ? 0 : (nph > S::TP ? S::TP : nph);
        if (hs > 0) __syncthreads();  // previous round copied out
        bool windowed = false;
        if constexpr (WIN) windowed = win.on != 0;
        const int pstride = windowed ? window_plane_stride<N>(h) : h * LDR + job.ppad;
        if (row_active && round_of_lane == hs) {
            const int tl = tr - hs * S::TP;
            if (va) {
                float4 *pa = reinterpret_cast<float4 *>(smem + tl * pstride + ia * LDR);
                static_for<N / 4>([&](auto jj) {
                    constexpr int j = decltype(jj)::value;
                    pa[j] = make_float4(zr[brev<N>(4 * j)] + bv, zr[brev<N>(4 * j + 1)] + bv,
                                        zr[brev<N>(4 * j + 2)] + bv, zr[brev<N>(4 * j + 3)] + bv);
                });
            }
            if (vb) {
                float4 *pb = reinterpret_cast<float4 *>(smem + tl * pstride + ib * LDR);
                static_for<N / 4>([&](auto jj) {
                    constexpr int j = decltype(jj)::value;
                    pb[j] = make_float4(zi[brev<N>(4 * j)] + bv, zi[brev<N>(4 * j + 1)] + bv,
                                        zi[brev<N>(4 * j + 2)] + bv, zi[brev<N>(4 * j + 3)] + bv);
                });
            }
        }
        __syncthreads();
        if (windowed)
            copy_windows<N, false>(smem, out, tbl, hs * S::TP, nph, h, w, padL, win, tid, pstride);
        else
            copy_canvas<N, false, S::THREADS>(smem, out + (x0 + hs * S::TP) * hw, nph * h, w, padL, vec4, tid, h, job.ppad);
    });
}

// ---------------------------------------------------------------------------------
// host launchers
// ---------------------------------------------------------------------------------
template <int N, bool INVERSE, bool SMALL = false, int PHASES = 0>
static size_t fft_lds_bytes(int h, int w, int padU, bool windowed = false)
{
    using S = FftShape<N, INVERSE, SMALL, PHASES>;
    (void)padU;
    // the tile holds every canvas row at a fixed place (the rows the small-plane forward variant reads)
    const size_t tile = (size_t)(SMALL ? 16 : N) * S::ROWSTRIDE * sizeof(float2);
    // canvas-row staging (the inverse, windowed operands, N = 128) or, smaller, the raw chunk with N
    // floats of slack on either side and N zeros behind
    // (+ 4 floats per plane: the most canvas_plane_pad asks for with these kernels' lane order)
    const size_t canvas = ((size_t)S::TP * (h * Canvas<N>::LDR + 4) + Canvas<N>::LDR) * sizeof(float);
    (void)windowed;
    const size_t raw = ((size_t)S::TP * h * w + 3 * N) * sizeof(float);
    const size_t stage = canvas > raw ? canvas : raw;
    return ((tile > stage ? tile : stage) + 15) & ~(size_t)15;
}

template <int N>
static long fwd_blocks(long planes)
{
    using S = FftShape<N, false>;
    long blocks = (planes + S::T - 1) / S::T;
    if (S::T * 8 < 128) blocks = (blocks + 15) / 16 * 16;  // whole cycles of the paired mapping
    return blocks;
}

template <int N, bool SMALL = false>
static FwdJob make_job(const FwdArgs &a)
{
    using S = FftShape<N, false, SMALL>;
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
    j.win.remap = window_remap_ok<S::T>(a.win, a.planes);
    return j;
}

static bool window_ok(const Window &w, long planes, int h, int ww)
{
    if (!w.on) return true;
    return w.d1 > 0 && w.nt > 0 && w.ntx > 0 && w.nt % w.ntx == 0 && w.step_y > 0 && w.step_x > 0 &&
           w.img_h > 0 && w.img_w > 0 && h > 0 && ww > 0 && planes % ((long)w.nt * w.d1) == 0;
}

// second == nullptr: one tensor only; third only with second
// raw staging needs odd plane sizes (see the kernel) in every operand of the launch
static bool raw_ok(const FwdArgs &a) { return (a.h & 1) && (a.w & 1) && !a.win.on; }

template <int N, bool WIN, int NZ, bool RAW>
static hipError_t launch_fwd_impl(const FwdArgs &a, const FwdArgs *second, hipStream_t s,
                                  const FwdArgs *third = nullptr)
{
    size_t lds = fft_lds_bytes<N, false, (NZ < N)>(a.h, a.w, a.padU, a.win.on != 0);
    const long blocks0 = fwd_blocks<N>(a.planes);
    long blocks01 = blocks0, blocks = blocks0;
    FwdJob j0 = make_job<N, (NZ < N)>(a);
    FwdJob j1 = j0, j2 = j0;
    if (second != nullptr) {
        const size_t lds1 = fft_lds_bytes<N, false, (NZ < N)>(second->h, second->w, second->padU, second->win.on != 0);
        if (lds1 > lds) lds = lds1;
        blocks01 += fwd_blocks<N>(second->planes);
        blocks = blocks01;
        j1 = make_job<N, (NZ < N)>(*second);
        if (third != nullptr) {
            const size_t lds2 = fft_lds_bytes<N, false, (NZ < N)>(third->h, third->w, third->padU, third->win.on != 0);
            if (lds2 > lds) lds = lds2;
            blocks += fwd_blocks<N>(third->planes);
            j2 = make_job<N, (NZ < N)>(*third);
        }
    }
    if (WIN) {  // the window table sits behind the tile / staging area
        j0.tbl_off = j1.tbl_off = j2.tbl_off = (int)(lds / sizeof(float));
        lds += FftShape<N>::T * sizeof(int4);
    }
    if (blocks > 0x7fffffffL) return hipErrorInvalidValue;
    {
        char name[64];
        snprintf(name, sizeof name, "rfft2d_kernel<%d, %s, %d, %s>", N, WIN ? "true" : "false", NZ, RAW ? "true" : "false");
        kernel_log_add(name, blocks * FftShape<N, false, (NZ < N)>::THREADS);
    }
    FBFC_LAUNCH((rfft2d_kernel<N, WIN, NZ, RAW>), dim3((unsigned)blocks), dim3(FftShape<N, false, (NZ < N)>::THREADS), lds, s, j0, j1,
                       j2, (unsigned)blocks0, (unsigned)blocks01);
    return hipGetLastError();
}

template <int N, bool WIN, int NZ = N>
static hipError_t launch_fwd(const FwdArgs &a, const FwdArgs *second, hipStream_t s, const FwdArgs *third = nullptr)
{
    if constexpr (!WIN && N <= 64) {
        if (raw_ok(a) && (second == nullptr || raw_ok(*second)) && (third == nullptr || raw_ok(*third)))
            return launch_fwd_impl<N, WIN, NZ, true>(a, second, s, third);
    }
    return launch_fwd_impl<N, WIN, NZ, false>(a, second, s, third);
}

template <int N, bool WIN, int PHASES>
static InvJob make_inv_job(const InvArgs &a)
{
    using S = FftShape<N, true, false, PHASES>;
    InvJob j;
    j.in = reinterpret_cast<const float2 *>(a.in);
    j.out = a.out;
    j.planes = a.planes;
    j.h = a.h; j.w = a.w; j.padU = a.padU; j.padL = a.padL;
    j.bias = a.bias;
    j.bias_period = a.bias_period > 0 ? a.bias_period : 1;
    // every copy-out round starts TP planes after the previous one: all of them 16-byte aligned
    j.vec4 = ((reinterpret_cast<uintptr_t>(a.out) & 15) == 0) && (((long)S::TP * a.h * a.w) % 4 == 0);
    j.ppad = a.win.on ? 0 : canvas_plane_pad(Canvas<N>::LDR, a.h, a.w, j.vec4, 2, 1);
    j.tbl_off = 0;
    j.win = a.win;
    j.win.remap = window_remap_ok<S::T>(a.win, a.planes);
    return j;
}

// second == nullptr: one tensor only.  The bias-gradient job, if any, is taken from `a` or `second`.
template <int N, bool WIN, int PHASES>
static hipError_t launch_inv_impl(const InvArgs &a, hipStream_t s, const InvArgs *second = nullptr)
{
    using S = FftShape<N, true, false, PHASES>;
    size_t lds = fft_lds_bytes<N, true, false, PHASES>(a.h, a.w, a.padU, a.win.on != 0);
    auto nblocks = [](long planes) {
        long b = (planes + S::T - 1) / S::T;
        if (S::T * 8 < 128) b = (b + 15) / 16 * 16;  // whole cycles of the paired mapping
        return b;
    };
    const long blocks0 = nblocks(a.planes);
    long blocks = blocks0;
    InvJob j0 = make_inv_job<N, WIN, PHASES>(a);
    InvJob j1 = j0;
    const InvArgs *bg = (a.go_freq != nullptr) ? &a : nullptr;
    if (second != nullptr) {
        const size_t lds1 = fft_lds_bytes<N, true, false, PHASES>(second->h, second->w, second->padU, second->win.on != 0);
        if (lds1 > lds) lds = lds1;
        blocks += nblocks(second->planes);
        j1 = make_inv_job<N, WIN, PHASES>(*second);
        if (bg == nullptr && second->go_freq != nullptr) bg = second;
    }
    if (WIN) {
        j0.tbl_off = j1.tbl_off = (int)(lds / sizeof(float));
        lds += S::T * sizeof(int4);
    }
    BiasGradJob bgrad = {nullptr, nullptr, 0.0f, 0, 0};
    if (bg != nullptr)
        bgrad = BiasGradJob{reinterpret_cast<const float2 *>(bg->go_freq), bg->grad_bias, bg->scale, bg->batch,
                            bg->out_planes};
    const unsigned bblocks = (bgrad.dc != nullptr) ? bias_grad_dc_blocks(bgrad.planes) : 0u;
    if (blocks + bblocks > 0x7fffffffL) return hipErrorInvalidValue;
    {
        char name[64];
        snprintf(name, sizeof name, "irfft2d_kernel<%d, %s, %d>", N, WIN ? "true" : "false", PHASES);
        kernel_log_add(name, (blocks + bblocks) * S::THREADS);
    }
    FBFC_LAUNCH((irfft2d_kernel<N, WIN, PHASES>), dim3((unsigned)blocks + bblocks), dim3(S::THREADS), lds, s,
                       j0, j1, (unsigned)blocks0, bgrad, bblocks);
    return hipGetLastError();
}

static bool inv32_in_phases(long planes) { return planes > 512L * FftShape<32, true>::T; }

template <int N, bool WIN>
static hipError_t launch_inv(const InvArgs &a, hipStream_t s)
{
    // N = 32: with the whole tile in LDS two workgroups share a CU, in two phases four do.  A launch
    // of more than one round of two workgroups per CU is faster with the four (12288 planes of
    // 27 x 27: 20.9 -> 16.9 us, 65536 planes: 95 -> 84 us); up to one round the two are level
    // (8192 planes: 10.9 and 11.0 us) and the whole tile stays.
    if constexpr (N == 32) {
        if (inv32_in_phases(a.planes)) return launch_inv_impl<N, WIN, 2>(a, s);
    }
    return launch_inv_impl<N, WIN, 0>(a, s);
}

// the kernels address a frequency row with 32-bit lane offsets
long fft_max_planes(int N) { return ((1L << 31) - 1) / ((long)(N / 2 + 1) * 8); }
static bool planes_ok(int N, long planes) { return planes > 0 && planes <= fft_max_planes(N); }

// Raises the dynamic-LDS limit of every kernel instantiation on the current device.  Called once per
// device (plan creation, first stand-alone transform), so that no launch makes an attribute call:
// launches may then be captured into a graph whatever shape comes first.
template <class K>
static hipError_t raise_lds_limit(K *kernel)
{
    return hipFuncSetAttribute(reinterpret_cast<const void *>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize,
                               160 * 1024);
}

template <int N>
static hipError_t raise_lds_limits_windowed()
{
    hipError_t e = raise_lds_limit(&rfft2d_kernel<N, true, N, false>);
    if (e == hipSuccess) e = raise_lds_limit(&irfft2d_kernel<N, true, 0>);
    if (e == hipSuccess && N == 32) e = raise_lds_limit(&irfft2d_kernel<N, true, (N == 32 ? 2 : 0)>);
    return e;
}

template <int N>
static hipError_t raise_lds_limits_plain()
{
    hipError_t e = raise_lds_limit(&rfft2d_kernel<N, false, N, false>);
    if constexpr (N <= 64) {
        if (e == hipSuccess) e = raise_lds_limit(&rfft2d_kernel<N, false, N, true>);
    }
    if (e == hipSuccess) e = raise_lds_limit(&irfft2d_kernel<N, false, 0>);
    if (e == hipSuccess && N == 32) e = raise_lds_limit(&irfft2d_kernel<N, false, (N == 32 ? 2 : 0)>);
    return e;
}

hipError_t fft_prepare_device()
{
    static std::mutex mu;
    static bool done[64] = {};
    int dev = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return e;
    if (dev < 0 || dev >= 64) return hipErrorInvalidDevice;
    std::lock_guard<std::mutex> lock(mu);
    if (done[dev]) return hipSuccess;
    e = raise_lds_limits_plain<8>();
    if (e == hipSuccess) e = raise_lds_limits_plain<16>();
    if (e == hipSuccess) e = raise_lds_limits_plain<32>();
    if (e == hipSuccess) e = fft_large_prepare_device();
    if (e == hipSuccess) e = raise_lds_limit(&irfft2d_kernel<64, false, 0>);
    if (e == hipSuccess) e = raise_lds_limit(&rfft2d_kernel<64, false, 64, false>);
    if (e == hipSuccess) e = raise_lds_limit(&rfft2d_kernel<64, false, 64, true>);
    if (e == hipSuccess) e = raise_lds_limits_windowed<8>();
    if (e == hipSuccess) e = raise_lds_limits_windowed<16>();
    if (e == hipSuccess) e = raise_lds_limits_windowed<32>();
    if (e == hipSuccess) done[dev] = true;
    return e;
}

// N = 64: the operand sizes that take the 8-plane kernels of fft_large.hip (two workgroups per CU, half-line
// runs).  Both forward kernels run 4096 planes per round of workgroups; the 8-plane one fills a last round
// that is at most half full better (2048 planes of 55 x 55: 19.3 -> 18.7 us, 6144: 44.2 -> 42.0 us) and loses
// on full rounds (4096: 25.6 -> 27.7 us, 8192: 49.4 -> 59.0 us, 12288: 81.6 -> 87.6 us).
static bool fwd64_rows(long planes) { return planes <= 2048 || (planes > 4096 && planes <= 6144); }
// The 8-plane inverse wins up to three rounds (2048 planes: 18.9 -> 15.4 us, 6144: 42.8 -> 37.1 us, 12288:
// 72.1 -> 69.5 us) and loses from 16384 planes on (96.6 -> 103.4 us).
static bool inv64_rows(long planes) { return planes <= 12288; }

// N = 32 forward: the operand sizes that take the one-row-per-lane kernel (see dispatch_fwd)
static bool fwd32_rows(long planes)
{
    const long k = (planes + 4095) / 4096;
    return k <= 2 || k == 4;
}

static hipError_t dispatch_fwd(int N, const FwdArgs &a, const FwdArgs *b, hipStream_t s)
{
    if (!planes_ok(N, a.planes) || (b != nullptr && !planes_ok(N, b->planes))) return hipErrorInvalidValue;
    if (!window_ok(a.win, a.planes, a.h, a.w) || (b != nullptr && !window_ok(b->win, b->planes, b->h, b->w)))
        return hipErrorInvalidValue;
    if (a.win.on || (b != nullptr && b->win.on)) {
        switch (N) {
            case 8: return launch_fwd<8, true>(a, b, s);
            case 16: return launch_fwd<16, true>(a, b, s);
            case 32: return launch_fwd<32, true>(a, b, s);
            default: return hipErrorInvalidValue;
        }
    }
    switch (N) {
        case 8: return launch_fwd<8, false>(a, b, s);
        case 16: return launch_fwd<16, false>(a, b, s);
        case 32: {
            // Per operand, as at N = 64 below.  The one-row-per-lane kernel of fft_large.hip (512 lanes, four
            // workgroups per CU) against the two-rows-per-lane one (256 lanes, three per CU), both 16 planes
            // per workgroup: what decides is how the workgroups of an operand divide over the CUs.  With
            // k = ceil(planes / 4096) workgroups per CU: 8192 planes of 27 x 27 (k = 2) 11.3 -> 10.2 us,
            // 16384 planes (k = 4) 23.3 -> 20.8 us, but 12288 planes (k = 3) 15.6 -> 16.6 us and 24576 planes
            // (k = 6) 29.8 -> 32.1 us; beyond that the two are within a few per cent either way, and one kernel
            // for all large operands keeps the operands of a pass in one launch.
            auto rows = [](const FwdArgs &x) { return fwd32_rows(x.planes); };
            if (b != nullptr && rows(a) != rows(*b)) {
                const hipError_t e = dispatch_fwd(N, a, nullptr, s);
                return e != hipSuccess ? e : dispatch_fwd(N, *b, nullptr, s);
            }
            if (rows(a)) return launch_rfft2d_large(N, a, b, s);
            return launch_fwd<32, false>(a, b, s);
        }
        case 64: {
            // Every operand gets the kernel its own size asks for, whatever it is launched with (results must
            // not depend on how transforms are grouped into launches):
            //  * planes of at most 16 x 16 at the origin (convolution kernels): the variant that skips the zero
            //    inputs, launched on its own;
            //  * plane counts that leave the last round of 16-plane workgroups at most half full (fwd64_rows):
            //    the 8-plane kernel of fft_large.hip;
            //  * all others: whole-line runs (16384 planes of 47 x 47: 107 against 112 us).
            auto small = [](const FwdArgs &x) { return x.h <= 16 && x.w <= 16 && x.padU == 0 && x.padL == 0; };
            auto rows = [&](const FwdArgs &x) { return small(x) || fwd64_rows(x.planes); };
            if (b != nullptr && (small(a) || small(*b) || rows(a) != rows(*b))) {
                const hipError_t e = dispatch_fwd(N, a, nullptr, s);
                return e != hipSuccess ? e : dispatch_fwd(N, *b, nullptr, s);
            }
            if (rows(a)) return launch_rfft2d_large(N, a, b, s);
            return launch_fwd<64, false>(a, b, s);
        }
        case 128: return launch_rfft2d_large(N, a, b, s);
        default: return hipErrorInvalidValue;
    }
}

hipError_t launch_rfft2d(int N, const float *in, float *out, long planes, int h, int w, int padU,
                         int padL, hipStream_t s)
{
    const FwdArgs a = {in, out, planes, h, w, padU, padL, {}, 0};
    return dispatch_fwd(N, a, nullptr, s);
}

hipError_t launch_rfft2d_one(int N, const FwdArgs &a, hipStream_t s) { return dispatch_fwd(N, a, nullptr, s); }

hipError_t launch_rfft2d_pair(int N, const FwdArgs &a, const FwdArgs &b, hipStream_t s)
{
    return dispatch_fwd(N, a, &b, s);
}

// Three forward transforms of one size: one launch where one kernel takes all three operands
// (N <= 32, no windows), otherwise a pair and a single one.
hipError_t launch_rfft2d_triple(int N, const FwdArgs &a, const FwdArgs &b, const FwdArgs &c, hipStream_t s)
{
    // every operand keeps the staging variant it gets in a pair or alone: all three agree on it
    const bool plain = !a.win.on && !b.win.on && !c.win.on && raw_ok(a) == raw_ok(b) && raw_ok(b) == raw_ok(c);
    if (plain && planes_ok(N, a.planes) && planes_ok(N, b.planes) && planes_ok(N, c.planes)) {
        switch (N) {
            case 8: return launch_fwd<8, false>(a, &b, s, &c);
            case 16: return launch_fwd<16, false>(a, &b, s, &c);
            case 32: {
                const bool ra = fwd32_rows(a.planes), rb = fwd32_rows(b.planes), rc = fwd32_rows(c.planes);
                if (ra && rb && rc) return launch_rfft2d_large(N, a, &b, s, &c);
                if (ra || rb || rc) break;
                return launch_fwd<32, false>(a, &b, s, &c);
            }
            default: break;
        }
    }
    const hipError_t e = dispatch_fwd(N, a, &b, s);
    return e != hipSuccess ? e : dispatch_fwd(N, c, nullptr, s);
}

// Two forward transforms that two different passes would each launch on its own: one grid where that runs
// every plane through the kernel it would get alone (N <= 32, no windows, the same staging variant; dispatch_fwd
// splits a pair whose operands take different kernels), two launches otherwise.
hipError_t launch_rfft2d_each(int N, const FwdArgs &a, const FwdArgs &b, hipStream_t s)
{
    if (N <= 32 && !a.win.on && !b.win.on && raw_ok(a) == raw_ok(b)) return dispatch_fwd(N, a, &b, s);
    const hipError_t e = dispatch_fwd(N, a, nullptr, s);
    return e != hipSuccess ? e : dispatch_fwd(N, b, nullptr, s);
}

hipError_t launch_irfft2d_args(int N, const InvArgs &a, hipStream_t s)
{
    if (!planes_ok(N, a.planes) || !window_ok(a.win, a.planes, a.h, a.w)) return hipErrorInvalidValue;
    if (a.win.on) {
        switch (N) {
            case 8: return launch_inv<8, true>(a, s);
            case 16: return launch_inv<16, true>(a, s);
            case 32: return launch_inv<32, true>(a, s);
            default: return hipErrorInvalidValue;
        }
    }
    switch (N) {
        case 8: return launch_inv<8, false>(a, s);
        case 16: return launch_inv<16, false>(a, s);
        case 32: return launch_inv<32, false>(a, s);
        case 64:
            return (inv64_rows(a.planes) || (a.h <= 16 && a.w <= 16)) ? launch_irfft2d_large(N, a, s)
                                                                             : launch_inv<64, false>(a, s);
        case 128: return launch_irfft2d_large(N, a, s);
        default: return hipErrorInvalidValue;
    }
}

// Two inverse transforms of one size: one launch for N <= 32 without windows, two otherwise.
hipError_t launch_irfft2d_two(int N, const InvArgs &a, const InvArgs &b, hipStream_t s)
{
    if (!a.win.on && !b.win.on && planes_ok(N, a.planes) && planes_ok(N, b.planes)) {
        switch (N) {
            case 8: return launch_inv_impl<8, false, 0>(a, s, &b);
            case 16: return launch_inv_impl<16, false, 0>(a, s, &b);
            case 32: {
                // each tensor keeps the kernel it would get alone; one launch if that is the same kernel
                const bool pa = inv32_in_phases(a.planes), pb = inv32_in_phases(b.planes);
                if (pa != pb) break;
                return pa ? launch_inv_impl<32, false, 2>(a, s, &b) : launch_inv_impl<32, false, 0>(a, s, &b);
            }
            default: break;
        }
    }
    const hipError_t e = launch_irfft2d_args(N, a, s);
    return e != hipSuccess ? e : launch_irfft2d_args(N, b, s);
}

hipError_t launch_irfft2d(int N, const float *in, float *out, long planes, int h, int w, int padU,
                          int padL, const float *bias, int bias_period, hipStream_t s)
{
    const InvArgs a = {in, out, planes, h, w, padU, padL, bias, bias_period, {}, nullptr, nullptr, 0.0f, 0, 0};
    return launch_irfft2d_args(N, a, s);
}

hipError_t launch_irfft2d_bias_grad(int N, const float *in, float *out, long planes, int h, int w,
                                    const float *go_freq, float *grad_bias, float scale, int batch,
                                    int out_planes, hipStream_t s)
{
    const InvArgs a = {in, out, planes, h, w, 0, 0, nullptr, 1, {}, go_freq, grad_bias, scale, batch, out_planes};
    return launch_irfft2d_args(N, a, s);
}

}  // namespace fbfc
