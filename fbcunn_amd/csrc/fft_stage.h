// Pieces shared by the 2-D transform kernels: the LDS staging of real planes (canvas rows or the raw
// chunk), the workgroup -> plane-group mapping and the spectrum stores.
#pragma once
#include <hip/hip_runtime.h>

#include "kernels.h"
#include "store_nt.h"

namespace fbfc {

// LDS staging area in canvas-row layout.  Row (p*h + r) of the staged planes starts at
// (p*h + r) * LDR floats and holds the N canvas columns of that row: input column x sits
// at padL + x, the margins are zero.  LDR = N + 4 floats keeps rows 16-byte aligned (the
// row pass reads and writes them with 16-byte LDS accesses) while rotating them over the
// banks.  The global side is the contiguous chunk of nrows * w floats.
template <int N>
struct Canvas {
    static constexpr int LDR = N + 4;
};

// Workgroup -> plane-group mapping.  Workgroups are handed to the 8 XCDs round-robin.  When a
// group's run per frequency is only part of a 128-byte line (T*8 = 64 or 32 bytes), the G = 16 / T
// groups that share each line are given to workgroups b, b+8, ... b+8(G-1): same XCD, dispatched back
// to back, so the parts meet in that XCD's L2 (one line fetched once / written back whole).
// GROUPS_PER_LINE < 0: derived from T.
template <int T, int GROUPS_PER_LINE = -1>
__device__ __forceinline__ long plane_group(unsigned bid)
{
    constexpr int G = GROUPS_PER_LINE > 0 ? GROUPS_PER_LINE : (T * 8 >= 128 ? 1 : 2);
    if constexpr (G == 1) {
        return (long)bid;
    } else {
        const unsigned cyc = bid / (8u * G), r = bid % (8u * G);
        return (long)((unsigned)G * (cyc * 8u + (r & 7u)) + (r >> 3));
    }
}
// the launch must cover whole cycles of that mapping
template <int T, int GROUPS_PER_LINE = -1>
inline long plane_group_blocks(long planes)
{
    constexpr int G = GROUPS_PER_LINE > 0 ? GROUPS_PER_LINE : (T * 8 >= 128 ? 1 : 2);
    long blocks = (planes + T - 1) / T;
    if (G > 1) blocks = (blocks + 8 * G - 1) / (8 * G) * (8 * G);
    return blocks;
}

// Global -> canvas rows (forward transforms): nrows rows of w floats, contiguous in memory, to rows of LDR floats.
// Canvas rows -> global (inverse transforms): the reverse.  ppad > 0 (inverse only): the canvases of consecutive
// planes (h rows each) lie ppad floats further apart than their rows alone (canvas_plane_pad); only with 16-byte
// pieces and planes of a multiple of four floats, so that a piece never straddles two planes.
template <int N, bool TO_LDS, int NT = 256>
__device__ __forceinline__ void copy_canvas(float *smem, float *g, int nrows, int w, int padL,
                                            int vec4, int tid, int h = 1, int ppad = 0)
{
    constexpr int LDR = Canvas<N>::LDR;
    const int total = nrows * w;
    int done = 0;
    if (vec4) {
        const int n4 = total >> 2;
        float4 *g4 = reinterpret_cast<float4 *>(g);
        int row = (tid * 4) / w, x = tid * 4 - row * w;
        const int drow = (4 * NT) / w, dx = 4 * NT - drow * w;
        if constexpr (TO_LDS) {
            // U loads in flight per lane before the first one is waited for: one load per round trip
            // would leave the memory system idle for most of the copy
            constexpr int U = (N >= 64) ? 12 : 8;
            for (int i0 = tid; i0 < n4; i0 += NT * U) {
                float4 q[U];
#pragma unroll
                for (int u = 0; u < U; ++u) {
                    const int i = i0 + NT * u;
                    if (i < n4) {
                        if constexpr (N >= 64) {
                            // planes of this size add up to tensors no cache holds until their next use:
                            // stream them (measured at 16384 planes of 55 x 55: 160 -> 136 us; smaller
                            // sizes got slower)
                            const floatx4_nt t = __builtin_nontemporal_load(reinterpret_cast<const floatx4_nt *>(g4 + i));
                            q[u] = make_float4(t.x, t.y, t.z, t.w);
                        } else {
                            q[u] = g4[i];
                        }
                    }
                }
                if ((w & 1) == 0) {
                    // even width: each half of a piece lies in one canvas row
#pragma unroll
                    for (int u = 0; u < U; ++u) {
                        const int i = i0 + NT * u;
                        if (i < n4) {
                            float *a0 = smem + row * LDR + padL + x;
                            float *a1 = (x + 2 >= w) ? smem + (row + 1) * LDR + padL + (x + 2 - w) : a0 + 2;
                            if ((padL & 1) == 0) {
                                *reinterpret_cast<float2 *>(a0) = make_float2(q[u].x, q[u].y);
                                *reinterpret_cast<float2 *>(a1) = make_float2(q[u].z, q[u].w);
                            } else {
                                a0[0] = q[u].x; a0[1] = q[u].y; a1[0] = q[u].z; a1[1] = q[u].w;
                            }
                        }
                        row += drow;
                        x += dx;
                        if (x >= w) { x -= w; ++row; }
                    }
                } else {
#pragma unroll
                    for (int u = 0; u < U; ++u) {
                        const int i = i0 + NT * u;
                        if (i < n4) {
                            const float v[4] = {q[u].x, q[u].y, q[u].z, q[u].w};
                            int r_ = row, x_ = x;
#pragma unroll
                            for (int c = 0; c < 4; ++c) {
                                smem[r_ * LDR + padL + x_] = v[c];
                                if (++x_ == w) { x_ = 0; ++r_; }
                            }
                        }
                        row += drow;
                        x += dx;
                        if (x >= w) { x -= w; ++row; }
                    }
                }
            }
        } else {
            if ((w & 1) == 0) {
                // Even widths: the two halves of a 16-byte piece lie in one canvas row each, so a piece costs two
                // addresses instead of four with a wrap test per element, and 8-byte LDS reads when the padding
                // is even too.  pl, pe: plane of the lane's piece and the piece's first element within it.
                const int hw = h * w;
                int pl = 0, pe = 0, dpl = 0, dpe = 0;
                if (ppad) {
                    pl = (tid * 4) / hw;
                    pe = tid * 4 - pl * hw;
                    dpl = (4 * NT) / hw;
                    dpe = 4 * NT - dpl * hw;
                }
                const bool even_pad = (padL & 1) == 0;
                for (int i = tid; i < n4; i += NT) {
                    const float *sp = smem + pl * ppad + padL;
                    const int a0 = row * LDR + x;
                    const int a1 = (x + 2 >= w) ? (row + 1) * LDR + (x + 2 - w) : a0 + 2;
                    float4 q;
                    if (even_pad) {
                        const float2 lo = *reinterpret_cast<const float2 *>(sp + a0);
                        const float2 hi = *reinterpret_cast<const float2 *>(sp + a1);
                        q = make_float4(lo.x, lo.y, hi.x, hi.y);
                    } else {
                        q = make_float4(sp[a0], sp[a0 + 1], sp[a1], sp[a1 + 1]);
                    }
                    store_nt(g4 + i, q);
                    row += drow;
                    x += dx;
                    if (x >= w) { x -= w; ++row; }
                    if (ppad) {
                        pl += dpl;
                        pe += dpe;
                        if (pe >= hw) { pe -= hw; ++pl; }
                    }
                }
            } else {
                for (int i = tid; i < n4; i += NT) {
                    float v[4];
                    int r_ = row, x_ = x;
#pragma unroll
                    for (int c = 0; c < 4; ++c) {
                        v[c] = smem[r_ * LDR + padL + x_];
                        if (++x_ == w) { x_ = 0; ++r_; }
                    }
                    store_nt(g4 + i, make_float4(v[0], v[1], v[2], v[3]));
                    row += drow;
                    x += dx;
                    if (x >= w) { x -= w; ++row; }
                }
            }
        }
        done = n4 << 2;
    }
    {
        const int first = done + tid;
        int row = first / w, x = first - row * w;
        const int drow = NT / w, dx = NT - drow * w;
        for (int i = first; i < total; i += NT) {
            float *sp = smem + row * LDR + padL + x;
            if (TO_LDS) *sp = g[i]; else g[i] = *sp;
            row += drow;
            x += dx;
            if (x >= w) { x -= w; ++row; }
        }
    }
}

// Spectrum stores.  Kernels whose runs per frequency are whole 128-byte lines write them through
// (store_nt.h), or non-temporally when the spectrum outgrows the caches (kernels.h) or the measurement knob says so; part-line runs rely on the L2 to join
// the workgroups that share a line and stay ordinary stores (written through, 6144 planes of 55 x 55 at
// N = 64 with 64-byte runs take 45.2 instead of 43.2 us, 4096 planes at N = 128 with 32-byte runs 216
// instead of 187 us).
enum SpectrumStore { STORE_WT = 0, STORE_NT = 1, STORE_ORDINARY = 2 };
template <int MODE>
__device__ __forceinline__ void store_freq_run(float2 *p, const float2 &v)
{
    if constexpr (MODE == STORE_NT) store_nt(p, v);
    else if constexpr (MODE == STORE_WT) store_wt(p, v);
    else *p = v;
}
// One complex value to byte offset voff of a frequency row.  The row's address is uniform: it goes into a
// buffer resource (scalar registers, two scalar additions per row) and the lane offset is the store's 32-bit
// vector offset, so a store costs no vector address arithmetic (as a global store to row + voff every one
// of the N stores of a lane carried a 64-bit vector addition).  The cache policy bits are those of
// store_freq_run: sc1 (write-through) = 16, nt = 2.
template <int MODE>
__device__ __forceinline__ void store_freq_at(char *rowbase, unsigned voff, const float2 &v)
{
    if constexpr (MODE == STORE_ORDINARY) {
        // part-line runs: the plain global store (as buffer stores the same runs were 8 % slower)
        *reinterpret_cast<float2 *>(rowbase + voff) = v;
        return;
    }
    typedef float fx2 __attribute__((ext_vector_type(2)));
    const __amdgpu_buffer_rsrc_t rsrc = __builtin_amdgcn_make_buffer_rsrc(rowbase, 0, -1, 0x00020000);
    const fx2 t = {v.x, v.y};
    constexpr int aux = (MODE == STORE_NT) ? 2 : (MODE == STORE_WT) ? 16 : 0;
    __builtin_amdgcn_raw_buffer_store_b64(t, rsrc, (int)voff, 0, aux);
}
// calls body(integral_constant<int, mode>) with the run-time mode as a compile-time one
template <bool WHOLE_LINES, class F>
__device__ __forceinline__ void with_store_mode(int mode, F &&body)
{
    if constexpr (!WHOLE_LINES) {
        body(std::integral_constant<int, STORE_ORDINARY>{});
    } else {
        if (mode == STORE_NT) body(std::integral_constant<int, STORE_NT>{});
        else body(std::integral_constant<int, STORE_WT>{});
    }
}

int spectrum_stream_override();  // 1: non-temporal spectrum stores always (a measurement knob)
inline int spectrum_store_mode(long planes, int n)
{
    if (spectrum_stream_override() == 1) return STORE_NT;
    return stream_bytes(planes * (long)n * (n / 2 + 1) * 8) ? STORE_NT : STORE_WT;
}

// Raw staging for the forward transform: the chunk of nfloats contiguous floats at g goes to LDS as it
// lies, by LDS-direct loads (global_load_lds): no staging registers, no LDS store instructions and no
// index arithmetic; the row pass then reads its rows at their (unaligned) places and masks the padding.
// 16-byte pieces where the chunk allows (aligned16), 4-byte pieces for the rest.  The destination of a
// wave instruction is wave-uniform; lane l lands at + l * size.  AUX: cache policy bits (2 = non-temporal).
template <int AUX, int NT = 256>
__device__ __forceinline__ void stage_raw(float *raw, const float *g, int nfloats, bool aligned16, int tid)
{
    const int wave = tid >> 6, lane = tid & 63;
    int done = 0;
    if (aligned16) {
        const int n16 = nfloats >> 2;
        for (int p0 = wave * 64; p0 < n16; p0 += NT) {
            if (p0 + lane < n16)
                __builtin_amdgcn_global_load_lds(
                    (const void __attribute__((address_space(1))) *)(g + 4 * (p0 + lane)),
                    (void __attribute__((address_space(3))) *)(raw + 4 * p0), 16, 0, AUX);
        }
        done = n16 << 2;
    }
    for (int e0 = done + wave * 64; e0 < nfloats; e0 += NT) {
        if (e0 + lane < nfloats)
            __builtin_amdgcn_global_load_lds((const void __attribute__((address_space(1))) *)(g + e0 + lane),
                                             (void __attribute__((address_space(3))) *)(raw + e0), 4, 0, AUX);
    }
}

// Zeroes the margins of nrows canvas rows and the all-zero row kept at float offset zoff.
template <int N, int NT = 256>
__device__ __forceinline__ void zero_canvas_margins(float *smem, int nrows, int w, int padL, int zoff,
                                                    int tid)
{
    constexpr int LDR = Canvas<N>::LDR;
    for (int row = tid; row < nrows; row += NT) {
        float *sp = smem + row * LDR;
        for (int c = 0; c < padL; ++c) sp[c] = 0.0f;
        for (int c = padL + w; c < N; ++c) sp[c] = 0.0f;
    }
    if (tid < N) smem[zoff + tid] = 0.0f;
}

// Inverse transforms: floats to add between the canvases of two planes so that the plane stride, counted in
// 16-byte slots, is `res` modulo `mod`.  The row pass writes canvas rows with 16-byte LDS accesses, 16 lanes per cycle; whether those 16
// lanes (so many planes times so many rows, by the kernel's lane order) cover all 64 banks depends on that stride:
//   * lanes that walk through 16 planes of one row (or 8 planes of two row pairs): an odd number of slots
//     (mod 2, res 1), which h * LDR / 4 is by itself for odd h only;
//   * one row per lane, TP planes fastest, then 16 / TP consecutive rows (a slot apart modulo 16 at N = 64 and 128,
//     nine at N = 32): 16 / TP slots modulo 32 / TP.
// 0 unless the copy runs in 16-byte pieces that cannot straddle two planes (even width, h * w a multiple of
// four floats).
inline int canvas_plane_pad(int ldr, int h, int w, int vec4, int mod, int res)
{
    if (!vec4 || (w & 1) != 0 || ((h * w) & 3) != 0) return 0;
    const int q = (h * ldr / 4) % mod;
    return 4 * ((res - q + mod) % mod);
}

// One launch can transform two tensors of the same FFT size (the two forward FFTs of a pass):
// workgroups [0, blocks0) work on job 0, the rest on job 1.
struct FwdJob {
    const float *in;
    float2 *out;
    long planes;
    int h, w, padU, padL, vec4;
    int tbl_off;  // windowed operand: float offset of the window table in LDS
    int herm;     // leave out the entries (ky > N/2, kx in {0, N/2}): conjugates of (N - ky, kx)
    int stream;   // SpectrumStore: how the spectrum is written
    Window win;
};

// One launch of the inverse kernel can produce two tensors of the same FFT size (the two inverse
// transforms of backward()): workgroups [0, blocks0) work on job 0, the rest on job 1.
struct InvJob {
    const float2 *in;
    float *out;
    long planes;
    int h, w, padU, padL;
    const float *bias;
    int bias_period, vec4;
    int ppad;     // floats between the canvases of two planes beyond their rows (canvas_plane_pad)
    int tbl_off;
    Window win;
};

}  // namespace fbfc
