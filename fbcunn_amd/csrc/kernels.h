// Internal launch interface between the C ABI (api.cpp) and the kernels.
#pragma once
#include <hip/hip_runtime.h>
#include <hip/hip_ext.h>
#include <stddef.h>

namespace fbfc {

// Per-launch timing.  While a pass runs with per-launch timing armed (api.cpp), every kernel launch of the
// calling thread takes the next pair of events from the armed list and is issued with them attached to
// the dispatch itself: their elapsed time is the kernel's own start-to-end time on the device, which is
// what a profiler's kernel trace reports, with no event or launch overhead in it.  Unarmed (the normal
// case) a launch is an ordinary launch.
bool launch_events_next(hipEvent_t *start, hipEvent_t *stop);
#define FBFC_LAUNCH(kernel, grid, block, lds, stream, ...)                                              \
    do {                                                                                                \
        hipEvent_t es_ = nullptr, ee_ = nullptr;                                                        \
        if (fbfc::launch_events_next(&es_, &ee_))                                                       \
            hipExtLaunchKernelGGL(kernel, grid, block, lds, stream, es_, ee_, 0, __VA_ARGS__);          \
        else                                                                                            \
            hipLaunchKernelGGL(kernel, grid, block, lds, stream, __VA_ARGS__);                          \
    } while (0)

// fft_kernels.hip ------------------------------------------------------------
// N in {8,16,32,64,128}; any other value returns hipErrorInvalidValue.
hipError_t launch_rfft2d(int N, const float *in, float *out, long planes, int h, int w, int padU,
                         int padL, hipStream_t s);
// A (d0, d1, img_h, img_w) tensor seen through windows (tiled convolution): virtual plane
// v = (b * nt + tile) * d1 + c is the h x w window of plane (b, c) with corner
// (ty * step_y + off_y, tx * step_x + off_x), tile = ty * ntx + tx.  Outside the image reads give
// zero and writes are dropped.  on = 0: ordinary contiguous planes.  Windows need N <= 32.
struct Window {
    int on;
    int d1, nt, ntx, step_y, step_x, off_y, off_x, img_h, img_w;
    int remap;  // set by the launchers: workgroups walk the tiles of one plane group on one XCD
};
// Two forward transforms of the same size in one launch (the two FFTs of a pass).
struct FwdArgs {
    const float *in;
    float *out;
    long planes;  // virtual planes when windowed
    int h, w, padU, padL;
    Window win;
    int herm;  // 1: do not write the entries (ky > N/2, kx in {0, N/2}), conjugates of (N - ky, kx)
};
hipError_t launch_rfft2d_pair(int N, const FwdArgs &a, const FwdArgs &b, hipStream_t s);
hipError_t launch_rfft2d_one(int N, const FwdArgs &a, hipStream_t s);
// The inverse never reads the entries (ky > N/2, kx in {0, N/2}): it takes them as the conjugates of
// (N - ky, kx), which they are for the spectrum of a real plane.
hipError_t launch_irfft2d(int N, const float *in, float *out, long planes, int h, int w, int padU,
                          int padL, const float *bias, int bias_period, hipStream_t s);

// Inverse transform (no padding offset, no bias add) that also carries the pass's bias gradient:
// grad_bias[f] = scale * sum_b Re go_freq[0][b][f] (go_freq = spectrum of gradOutput).
hipError_t launch_irfft2d_bias_grad(int N, const float *in, float *out, long planes, int h, int w,
                                    const float *go_freq, float *grad_bias, float scale, int batch,
                                    int out_planes, hipStream_t s);

// General form of the inverse: optional bias add, optional windowed store, optional bias-gradient job
// (go_freq != nullptr: grad_bias[f] = scale * sum_{b < batch} Re go_freq[0][b][f]).
struct InvArgs {
    const float *in;
    float *out;
    long planes;
    int h, w, padU, padL;
    const float *bias;
    int bias_period;
    Window win;
    const float *go_freq;
    float *grad_bias;
    float scale;
    int batch, out_planes;
};
hipError_t launch_irfft2d_args(int N, const InvArgs &a, hipStream_t s);
// backward(): its three forward transforms and its two inverse transforms as one launch each where one
// kernel takes them all (N <= 32, no windows), as several launches otherwise; same results either way
hipError_t launch_rfft2d_triple(int N, const FwdArgs &a, const FwdArgs &b, const FwdArgs &c, hipStream_t s);
// two transforms that would otherwise be two launches of launch_rfft2d_one, with the same results
hipError_t launch_rfft2d_each(int N, const FwdArgs &a, const FwdArgs &b, hipStream_t s);
hipError_t launch_irfft2d_two(int N, const InvArgs &a, const InvArgs &b, hipStream_t s);

// Largest number of planes one launch of an N x N transform takes (the kernels address a frequency
// row of the spectrum with 32-bit byte offsets): floor((2^31 - 1) / ((N/2 + 1) * 8)).
long fft_max_planes(int N);
// Raises the dynamic-LDS limit of every transform kernel on the current device, once per device.
// After it no launch makes an attribute call (launches may be captured whatever shape comes first).
hipError_t fft_prepare_device();

// fft_large.hip: the transforms of size 64 and 128 (plain operands; no windows)
hipError_t launch_rfft2d_large(int N, const FwdArgs &a, const FwdArgs *b, hipStream_t s, const FwdArgs *c = nullptr);
hipError_t launch_irfft2d_large(int N, const InvArgs &a, hipStream_t s);
hipError_t fft_large_prepare_device();

// fused_kernels.hip: the fused tiled convolution (tile FFT sizes 8, 16, 32) ---------------------------
// updateOutput / updateGradInput: result(vbatch tiles x n_big planes) = inverse transform of
// alpha * sum over the n_small contracted planes of FFT(window) x (conj) W, W = w_freq[q][f * P + p] with
// plane index small * w_stride_small + big * w_stride_big.
struct FusedConvArgs {
    const float *small;   // tensor of the contracted side (input resp. gradOutput)
    float *big;           // result tensor (output resp. gradInput)
    const float *w_freq;  // weight spectrum, frequency-major
    const float *bias;    // added per big plane; nullptr: none
    Window small_win, big_win;
    int small_h, small_w;                       // windows of the contracted side
    int big_h, big_w, big_pad_u, big_pad_l;     // result tiles and where they sit in the circular result
    int n_small, n_big, w_stride_small, w_stride_big, out_planes, in_planes;
    int vbatch;           // batch * tiles
    int conj_w;           // 1: multiply by conj(W) (updateOutput)
    float alpha;
};
hipError_t launch_fused_conv(int N, const FusedConvArgs &a, hipStream_t s);
// accGradParameters: grad_weight(F, P, kh, kw) = alpha * sum over tiles of the k x k crop of
// IFFT(conj(FFT(gradOutput tile)) FFT(input window)); `part` holds nranges partial results of
// out_planes * in_planes * kh * kw floats (nranges from fused_accgrad_ranges).
struct FusedAccArgs {
    const float *input, *grad_output;
    float *grad_weight, *part;
    Window in_win, go_win;
    int in_h, in_w, go_h, go_w, kh, kw;
    int out_planes, in_planes, vbatch, nranges;
    float alpha;
};
int fused_accgrad_ranges(int N, int vbatch, int out_planes, int in_planes);
hipError_t launch_fused_accgrad(int N, const FusedAccArgs &a, hipStream_t s);
// raises the dynamic-LDS limit of the fused kernels on the current device (plan creation calls it)
hipError_t fused_prepare_device();

// fft_small.hip ------------------------------------------------------------------
// 1-D batched transforms, N in {2,4,...,128}: rows of n reals at pad_l of the N-point canvas
// <-> (rows, N/2+1) complex, row-major; the inverse is unnormalised.
hipError_t launch_rfft1d(int N, const float *in, float *out, long rows, int n, int pad_l, hipStream_t s);
hipError_t launch_irfft1d(int N, const float *in, float *out, long rows, int n, int pad_l, hipStream_t s);
// 2-D transforms of size 2 and 4 (frequency-major spectrum, as for the larger sizes)
hipError_t launch_rfft2d_tiny(int N, const float *in, float *out, long planes, int h, int w, int pad_u,
                              int pad_l, hipStream_t s);
hipError_t launch_irfft2d_tiny(int N, const float *in, float *out, long planes, int h, int w, int pad_u,
                               int pad_l, const float *bias, int bias_period, hipStream_t s);

// cgemm_kernels.hip ------------------------------------------------------------
// mode 0: C[m][n] (+)= alpha * sum_k A[m][k] * conj(B[n][k])   A (m x k), B (n x k)
// mode 1: C[m][n] (+)= alpha * sum_k A[m][k] * B[k][n]         A (m x k), B (k x n)
// mode 2: C[m][n] (+)= alpha * sum_k conj(A[k][m]) * B[k][n]   A (k x m), B (k x n)
// for each of n_freq frequencies; operands frequency-major, complex interleaved.
hipError_t launch_cgemm_freq(int mode, const float *A, const float *B, float *C, int n_freq, int m,
                             int n, int k, float alpha, int accumulate, hipStream_t s);

// Which frequencies a contraction visits.  The spectrum of a real plane is Hermitian also along ky
// in the columns kx = 0 and kx = N/2: X[N-ky][kx] = conj X[ky][kx], so the entries (ky > N/2,
// kx in {0, N/2}) carry nothing new.  With a map, the i-th frequency contracted is
//   i < split: i;  else split + row * nh + col + 1  with (row, col) = divmod(i - split, rowlen),
// i.e. rows ky <= N/2 whole and rows ky > N/2 without their first and last column.
// split = 0: every frequency of the buffer in order.
struct FreqMap {
    int split, rowlen, nh;
};
inline FreqMap hermitian_map(int N) { return FreqMap{(N / 2 + 1) * (N / 2 + 1), N / 2 - 1, N / 2 + 1}; }
inline int hermitian_count(int N) { return (N / 2 + 1) * (N / 2 + 1) + (N / 2 - 1) * (N / 2 - 1); }
hipError_t launch_cgemm_freq_map(int mode, const float *A, const float *B, float *C, int n_freq, FreqMap fm,
                                 int m, int n, int k, float alpha, int accumulate, hipStream_t s);
// The two contractions of a backward pass, C1 = A1 B1 (mode 1) and C2 = conj(A2)^T B2 (mode 2), over the
// same frequencies: one launch where both problems take tile / split-block kernels, two otherwise; the
// results are those of two launch_cgemm_freq_map calls either way.
struct MmArgs {
    const float *A, *B;
    float *C;
    int m, n, k;
    float alpha;
    int accumulate;
};
hipError_t launch_cgemm_backward(const MmArgs &gi, const MmArgs &gw, int n_freq, FreqMap fm, hipStream_t s);

// Launch log of the calling thread: every kernel launcher appends "<kernel name> grid=<work-items>";
// the pass entry points clear it before a stage and keep what the stage logged.
void kernel_log_clear();
void kernel_log_add(const char *name, long grid_items);
const char *kernel_log_get();
// Measurement knob: -1 = choose by shape; 0 = register-staged LDS tiles, 8 = LDS-direct tiles,
// 9 = hybrid of LDS-direct tiles and split blocks, 1 / 2 / 4 = register-fed kernel with that many
// waves per block (falls back to the shape rule where the forced variant cannot run the shape).
void cgemm_force_variant(int v);
// What one kernel writes for the next to read once (a spectrum, a contraction result) is written through to
// the memory side, whose 256 MB cache keeps it, up to this size; beyond it, it would not survive until it is
// read and is streamed with non-temporal stores.  Per training step, non-temporal always / never / above the
// limit: 96 -> 256 planes, 24 x 24 (53 / 107 / 142 MB of spectra) 615 / 588 / 587 us; batch 64, 96 -> 256,
// 55 x 55 (104 / 415 / 277 MB) 1.381 / 1.407 / 1.375 ms.
constexpr long kStreamBytes = 144L << 20;
inline bool stream_bytes(long bytes) { return bytes > kStreamBytes; }
// -1: the rule above (default); 1: non-temporal spectrum stores always (where runs are whole lines)
void spectrum_stream_force(int v);
// Measurement library only (built with FBFC_PROBES): the 64x64 tile kernel with clock counters, which adds
// every workgroup's shader-clock and 100 MHz ticks to ticks[0] and ticks[1] (m, n multiples of 64, k of 16)
hipError_t launch_cgemm_clock_probe(int mode, const float *A, const float *B, float *C, int n_freq, int m, int n,
                                    int k, unsigned long long *ticks, hipStream_t s);

// layout_kernels.hip: frequency-major freq[q][plane] <-> the reference's plane-major buf[plane][q].
// mode 0: same frequency order; 1: buf[a][c] = X[ky = c][kx = a] (fbfft for N < 8 or N > 32);
// 2: buf[a][c] = X[ky = a][kx = c], a <= N/2 (fbfft for 8 <= N <= 32).  nq = entries per plane.
hipError_t launch_freq_to_planes(const float *freq, float *buf, long planes, int nq, int N, int mode,
                                 hipStream_t s);
hipError_t launch_planes_to_freq(const float *buf, float *freq, long planes, int nq, int N, int mode,
                                 hipStream_t s);

// direct_kernels.hip: spatial-domain convolution (any stride).  desc = the 11 ints of fbfc_conv_desc.
hipError_t launch_direct_fprop(const int *desc, const float *in, const float *w, const float *bias, float *out,
                               hipStream_t s);
hipError_t launch_direct_bprop(const int *desc, const float *go, const float *w, float *gi, hipStream_t s);
hipError_t launch_direct_accgrad(const int *desc, const float *in, const float *go, float *gw, float scale,
                                 hipStream_t s);

// bias_kernels.hip ---------------------------------------------------------------
hipError_t launch_bias_add(float *out, const float *bias, int batch, int planes, int hw,
                           hipStream_t s);
size_t bias_grad_scratch_bytes(int batch, int planes);
hipError_t launch_bias_grad(const float *grad_out, float *grad_bias, float scale, int batch,
                            int planes, int hw, float *scratch, hipStream_t s);

// Strided forms: element (b, f, r, c) at b * sb + f * sf + r * sh + c * sw floats, bias[f] at f * bias_stride.
hipError_t launch_bias_add_strided(float *out, const float *bias, int batch, int planes, int h, int w,
                                   long sb, long sf, long sh, long sw, long bias_stride, hipStream_t s);
hipError_t launch_bias_grad_strided(const float *grad_out, float *grad_bias, float scale, int batch,
                                    int planes, int h, int w, long sb, long sf, long sh, long sw,
                                    long bias_stride, float *scratch, hipStream_t s);
// bias_noalloc.hip: the bias gradient with its partial sums in a fixed device array (no allocation,
// no workspace argument); at most bias_grad_noalloc_max_planes() planes.  prepare() looks the array
// up on the current device (the first launch does so too).
int bias_grad_noalloc_max_planes();
hipError_t bias_grad_noalloc_prepare();
hipError_t launch_bias_grad_noalloc(const float *grad_out, float *grad_bias, float scale, int batch,
                                    int planes, int hw, hipStream_t s);

// freq = frequency-major spectrum of grad_out (its first frequency row holds the plane sums)
hipError_t launch_bias_grad_dc(const float *freq, float *grad_bias, float scale, int batch, int planes,
                               hipStream_t s);

}  // namespace fbfc
