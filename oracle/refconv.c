/*
 * CPU oracle for the FFT-convolution path.  TEST INFRASTRUCTURE ONLY.
 *
 * This file restates, in plain C, the CPU algorithms the reference uses to
 * judge its FFT convolution modules.  Only tests, the smoke check and the
 * bench's cpu_baseline leg may link or load it; the shipped library never
 * does.  Nothing here runs on a GPU.
 *
 * Functions and the reference code they follow:
 *   orc_cross_correlation_valid          test/ReferenceConvolutions.cpp:86-200
 *   orc_convolution_full                 test/ReferenceConvolutions.cpp:338-450
 *   orc_cross_correlation_reverse_valid  test/ReferenceConvolutions.cpp:452-554
 *   orc_valid_conv_size / rev / full     test/ReferenceConvolutions.h:17-34
 *   orc_bias_update_output               test/BiasTest.cpp:83-103
 *   orc_bias_acc_grad_parameters         test/BiasTest.cpp:107-130
 *   orc_is_within                        test/TestUtils.cpp:119-149
 *   orc_dft2d_r2c / orc_idft2d_c2r       the DFT definition; what
 *                                        src/fft/FFTWrapperLua.cpp:209-272
 *                                        asks of fbfft (unnormalised inverse,
 *                                        implicit zero padding at padU,padL)
 *   orc_freq_contract                    src/fft/CuFFTConvolution_UpdateOutput.cu:25-59,
 *                                        _AccGradParameters.cu:25-64,
 *                                        _UpdateGradInput.cu:24-59 and the
 *                                        transposeMMFFI call sites
 *                                        fbcunn/SpatialConvolutionFBFFT.lua:157-164,
 *                                        244-251, 337-344
 *
 * Summation order.  For every output element the float32 additions happen in
 * the same order as in the reference loops, so results are bit-identical to
 * the reference's on the same inputs.  OpenMP is applied only to loops the
 * reference marks "doall" (independent output elements), never to a
 * reduction, so threading does not change any result.
 *
 * Pinning (which checks keep this file honest) lives in tests/test_oracle_*.py:
 * the reference's own closed-form table (ones 7x7 (*) ones 3x3, full), its
 * cuFFT known-answer vectors, its padded-vs-unpadded self-consistency test,
 * scipy's correlate2d/convolve2d, inner-product adjoint identities and
 * brute-force loops on tiny shapes.
 */
#include <math.h>
#ifdef _OPENMP
#include <omp.h>
#endif
#include <stddef.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#define IDX4(a, b, c, d, B, C, D) ((((size_t)(a) * (B) + (b)) * (C) + (c)) * (D) + (d))

/* Threads the parallel loops use from now on (n < 1: leave as is); returns the count in effect.
 * Only the timing of the CPU baseline uses it. */
int orc_set_threads(int n)
{
#ifdef _OPENMP
    if (n >= 1) omp_set_num_threads(n);
    return omp_get_max_threads();
#else
    (void)n;
    return 1;
#endif
}

long orc_valid_conv_size(long in, long k, long stride) { return (in - k) / stride + 1; }
long orc_valid_rev_conv_size(long in, long k, long stride) { return in - (k - 1) * stride; }
long orc_full_conv_size(long in, long k, long stride) { return (in - 1) * stride + k; }

/* fprop: output (B,F,oR,oC) = input (B,P,H,W) valid-cross-correlated with
 * filters (F,P,kH,kW); zero padding is implied, never materialised.
 * Returns 0, or a negative code for the argument errors the reference throws. */
int orc_cross_correlation_valid(const float *input, long B, long P, long H, long W,
                                const float *filters, long F, long kH, long kW,
                                long strideR, long strideC,
                                long padT, long padB, long padL, long padR,
                                float *output)
{
    if (strideR < 1 || strideC < 1) return -3;
    if (kH > H || kW > W) return -4;
    if ((H - kH) % strideR != 0 || (W - kW) % strideC != 0) return -5;
    const long oR = orc_valid_conv_size(H + padT + padB, kH, strideR);
    const long oC = orc_valid_conv_size(W + padL + padR, kW, strideC);
    memset(output, 0, sizeof(float) * (size_t)B * F * oR * oC);

#pragma omp parallel for collapse(2) schedule(static)
    for (long b = 0; b < B; ++b) {
        for (long f = 0; f < F; ++f) {
            float *out = output + IDX4(b, f, 0, 0, F, oR, oC);
            for (long p = 0; p < P; ++p) { /* reduction: plane order kept */
                const float *in = input + IDX4(b, p, 0, 0, P, H, W);
                const float *flt = filters + IDX4(f, p, 0, 0, P, kH, kW);
                for (long r = 0; r < oR; ++r) {
                    const long r0 = r * strideR - padT;
                    for (long c = 0; c < oC; ++c) {
                        const long c0 = c * strideC - padL;
                        float val = 0.0f;
                        for (long fr = 0; fr < kH; ++fr) {
                            const long ir = r0 + fr;
                            if (ir < 0 || ir >= H) continue;
                            for (long fc = 0; fc < kW; ++fc) {
                                const long ic = c0 + fc;
                                if (ic < 0 || ic >= W) continue;
                                val += flt[fr * kW + fc] * in[ir * W + ic];
                            }
                        }
                        out[r * oC + c] += val;
                    }
                }
            }
        }
    }
    return 0;
}

/* bprop: gradInput (B,P,H,W) = gradOutput (B,F,oR,oC) fully convolved with
 * filters (F,P,kH,kW), keeping only the un-padded window of the result. */
int orc_convolution_full(const float *output, long B, long F, long oR, long oC,
                         const float *filters, long P, long kH, long kW,
                         long strideR, long strideC,
                         long padT, long padB, long padL, long padR,
                         float *input)
{
    if (strideR < 1 || strideC < 1) return -3;
    const long H = orc_full_conv_size(oR, kH, strideR) - padT - padB;
    const long W = orc_full_conv_size(oC, kW, strideC) - padL - padR;
    memset(input, 0, sizeof(float) * (size_t)B * P * H * W);

#pragma omp parallel for collapse(2) schedule(static)
    for (long b = 0; b < B; ++b) {
        for (long p = 0; p < P; ++p) {
            float *in = input + IDX4(b, p, 0, 0, P, H, W);
            for (long f = 0; f < F; ++f) { /* reduction */
                const float *out = output + IDX4(b, f, 0, 0, F, oR, oC);
                const float *flt = filters + IDX4(f, p, 0, 0, P, kH, kW);
                for (long ir = 0; ir < H; ++ir) {
                    const long irp = ir + padT;
                    for (long fr = irp % strideR; fr <= irp && fr < kH; fr += strideR) {
                        const long orow = (irp - fr) / strideR;
                        if (orow >= oR) continue;
                        for (long ic = 0; ic < W; ++ic) {
                            const long icp = ic + padL;
                            for (long fc = icp % strideC; fc <= icp && fc < kW; fc += strideC) {
                                const long ocol = (icp - fc) / strideC;
                                if (ocol >= oC) continue;
                                in[ir * W + ic] += flt[fr * kW + fc] * out[orow * oC + ocol];
                            }
                        }
                    }
                }
            }
        }
    }
    return 0;
}

/* accGrad: gradWeight (F,P,kH,kW) = scale * sum_b input(b,p) valid-cross-
 * correlated with gradOutput(b,f).  The result starts from zero (assignment,
 * not accumulation into a caller value). */
int orc_cross_correlation_reverse_valid(const float *input, long B, long P, long H, long W,
                                        const float *output, long F, long oR, long oC,
                                        long strideR, long strideC, float scale,
                                        long padT, long padB, long padL, long padR,
                                        float *filters)
{
    if (strideR < 1 || strideC < 1) return -3;
    if (oR > H + padT + padB || oC > W + padL + padR) return -4;
    const long kH = orc_valid_rev_conv_size(H + padT + padB, oR, strideR);
    const long kW = orc_valid_rev_conv_size(W + padL + padR, oC, strideC);
    memset(filters, 0, sizeof(float) * (size_t)F * P * kH * kW);

    /* The reference's outermost loop is the batch reduction; per (f,p) filter
     * element the additions happen in (batch, outRow, outCol) order.  Moving
     * the independent (f,p) loops outside keeps that order for every element. */
#pragma omp parallel for collapse(2) schedule(static)
    for (long f = 0; f < F; ++f) {
        for (long p = 0; p < P; ++p) {
            float *flt = filters + IDX4(f, p, 0, 0, P, kH, kW);
            for (long b = 0; b < B; ++b) {
                const float *in = input + IDX4(b, p, 0, 0, P, H, W);
                const float *out = output + IDX4(b, f, 0, 0, F, oR, oC);
                for (long r = 0; r < oR; ++r) {
                    for (long c = 0; c < oC; ++c) {
                        const float o = out[r * oC + c];
                        for (long fr = 0; fr < kH; ++fr) {
                            const long ir = r * strideR + fr - padT;
                            if (ir < 0 || ir >= H) continue;
                            for (long fc = 0; fc < kW; ++fc) {
                                const long ic = c * strideC + fc - padL;
                                if (ic < 0 || ic >= W) continue;
                                flt[fr * kW + fc] += scale * o * in[ir * W + ic];
                            }
                        }
                    }
                }
            }
        }
    }
    return 0;
}

/* out[b][f][r][c] += bias[f], in place. */
void orc_bias_update_output(float *output, long B, long F, long R, long C, const float *bias)
{
    for (long b = 0; b < B; ++b)
        for (long f = 0; f < F; ++f) {
            const float bv = bias[f];
            float *o = output + IDX4(b, f, 0, 0, F, R, C);
            for (long i = 0; i < R * C; ++i) o[i] += bv;
        }
}

/* gradBias[f] = scale * sum_{b,r,c} gradOutput[b][f][r][c]  (assignment). */
void orc_bias_acc_grad_parameters(const float *gradOutput, long B, long F, long R, long C,
                                  float scale, float *gradBias)
{
    for (long f = 0; f < F; ++f) {
        float sum = 0.0f;
        for (long b = 0; b < B; ++b) {
            const float *o = gradOutput + IDX4(b, f, 0, 0, F, R, C);
            for (long i = 0; i < R * C; ++i) sum += o[i];
        }
        gradBias[f] = sum * scale;
    }
}

/* The reference's element comparison: relative to |a|+|b|, absolute near 0. */
int orc_is_within(float a, float b, float rel)
{
    const float adj = 0.5f * rel;
    if (a == b || (isnan(a) && isnan(b))) return 1;
    if (!isfinite(a) && !isfinite(b)) return signbit(a) == signbit(b);
    if (fabsf(a) < rel || fabsf(b) < rel || !isnormal(a) || !isnormal(b))
        return !(fabsf(a - b) > adj);
    return !(fabsf(a - b) > adj * (fabsf(a) + fabsf(b)));
}

/* Naive 2-D real-to-complex DFT, double accumulation.
 * in  : planes x h x w real, placed at rows padU.., cols padL.. of an
 *       nR x nC zero canvas.
 * out : planes x nR x (nC/2+1) x 2  (row frequency full, column frequency
 *       halved), X[u][v] = sum_{y,x} canvas[y][x] exp(-2 pi i (u y/nR + v x/nC)).
 * Works for any nR, nC (not only powers of two). */
void orc_dft2d_r2c(const float *in, long planes, long h, long w, long padU, long padL,
                   long nR, long nC, float *out)
{
    const long nCh = nC / 2 + 1;
    const double PI2 = 6.283185307179586476925286766559;
#pragma omp parallel for schedule(static)
    for (long pl = 0; pl < planes; ++pl) {
        const float *x = in + (size_t)pl * h * w;
        float *o = out + (size_t)pl * nR * nCh * 2;
        for (long u = 0; u < nR; ++u)
            for (long v = 0; v < nCh; ++v) {
                double re = 0.0, im = 0.0;
                for (long y = 0; y < h; ++y)
                    for (long xx = 0; xx < w; ++xx) {
                        const long cy = y + padU, cx = xx + padL;
                        if (cy >= nR || cx >= nC) continue;
                        /* reduce the phase exactly in integers first */
                        const double ph = -PI2 * ((double)((u * cy) % nR) / (double)nR +
                                                  (double)((v * cx) % nC) / (double)nC);
                        re += x[y * w + xx] * cos(ph);
                        im += x[y * w + xx] * sin(ph);
                    }
                o[(u * nCh + v) * 2 + 0] = (float)re;
                o[(u * nCh + v) * 2 + 1] = (float)im;
            }
    }
}

/* Naive unnormalised inverse of the above from the half spectrum, with crop:
 * y[r][s] = sum_{u,v} X[u][v] exp(+2 pi i (u r/nR + v s/nC)) over the FULL
 * spectrum (missing half rebuilt by Hermitian symmetry), and
 * out[r][s] = y[r+padU][s+padL] for r<h, s<w.  No 1/(nR nC). */
void orc_idft2d_c2r(const float *freq, long planes, long h, long w, long padU, long padL,
                    long nR, long nC, float *out)
{
    const long nCh = nC / 2 + 1;
    const double PI2 = 6.283185307179586476925286766559;
#pragma omp parallel for schedule(static)
    for (long pl = 0; pl < planes; ++pl) {
        const float *X = freq + (size_t)pl * nR * nCh * 2;
        float *o = out + (size_t)pl * h * w;
        for (long r = 0; r < h; ++r)
            for (long s = 0; s < w; ++s) {
                const long rr = r + padU, ss = s + padL;
                double acc = 0.0;
                for (long u = 0; u < nR; ++u)
                    for (long v = 0; v < nC; ++v) {
                        double xr, xi;
                        if (v < nCh) {
                            xr = X[(u * nCh + v) * 2];
                            xi = X[(u * nCh + v) * 2 + 1];
                        } else { /* X[u][v] = conj X[-u][-v] */
                            const long uu = (nR - u) % nR, vv = nC - v;
                            xr = X[(uu * nCh + vv) * 2];
                            xi = -X[(uu * nCh + vv) * 2 + 1];
                        }
                        const double ph = PI2 * ((double)((u * rr) % nR) / (double)nR +
                                                 (double)((v * ss) % nC) / (double)nC);
                        acc += xr * cos(ph) - xi * sin(ph);
                    }
                o[r * w + s] = (float)acc;
            }
    }
}

/* Per-frequency complex contraction on plane-major spectra (d0,d1,Q,2).
 * pass 0 (updateOutput)      : O[b][f][q] = alpha sum_p I[b][p][q] conj(W[f][p][q])
 * pass 1 (updateGradInput)   : GI[b][p][q] = alpha sum_f GO[b][f][q] W[f][p][q]
 * pass 2 (accGradParameters) : GW[f][p][q] = alpha sum_b conj(GO[b][f][q]) I[b][p][q]
 * A, Bm, C are the first, second and third tensor of the transposeMMFFI call
 * of that pass.  Double accumulation. */
void orc_freq_contract(int pass, const float *A, const float *Bm, float *C,
                       long nB, long nP, long nF, long Q, float alpha)
{
    if (pass == 0) {
#pragma omp parallel for collapse(2) schedule(static)
        for (long b = 0; b < nB; ++b)
            for (long f = 0; f < nF; ++f)
                for (long q = 0; q < Q; ++q) {
                    double re = 0, im = 0;
                    for (long p = 0; p < nP; ++p) {
                        const float *a = A + ((b * nP + p) * Q + q) * 2;
                        const float *w = Bm + ((f * nP + p) * Q + q) * 2;
                        re += (double)a[0] * w[0] + (double)a[1] * w[1];
                        im += (double)a[1] * w[0] - (double)a[0] * w[1];
                    }
                    C[((b * nF + f) * Q + q) * 2 + 0] = (float)(alpha * re);
                    C[((b * nF + f) * Q + q) * 2 + 1] = (float)(alpha * im);
                }
    } else if (pass == 1) {
#pragma omp parallel for collapse(2) schedule(static)
        for (long b = 0; b < nB; ++b)
            for (long p = 0; p < nP; ++p)
                for (long q = 0; q < Q; ++q) {
                    double re = 0, im = 0;
                    for (long f = 0; f < nF; ++f) {
                        const float *a = A + ((b * nF + f) * Q + q) * 2;
                        const float *w = Bm + ((f * nP + p) * Q + q) * 2;
                        re += (double)a[0] * w[0] - (double)a[1] * w[1];
                        im += (double)a[0] * w[1] + (double)a[1] * w[0];
                    }
                    C[((b * nP + p) * Q + q) * 2 + 0] = (float)(alpha * re);
                    C[((b * nP + p) * Q + q) * 2 + 1] = (float)(alpha * im);
                }
    } else {
#pragma omp parallel for collapse(2) schedule(static)
        for (long f = 0; f < nF; ++f)
            for (long p = 0; p < nP; ++p)
                for (long q = 0; q < Q; ++q) {
                    double re = 0, im = 0;
                    for (long b = 0; b < nB; ++b) {
                        const float *a = A + ((b * nF + f) * Q + q) * 2;  /* GO, conjugated */
                        const float *x = Bm + ((b * nP + p) * Q + q) * 2; /* I */
                        re += (double)a[0] * x[0] + (double)a[1] * x[1];
                        im += (double)a[0] * x[1] - (double)a[1] * x[0];
                    }
                    C[((f * nP + p) * Q + q) * 2 + 0] = (float)(alpha * re);
                    C[((f * nP + p) * Q + q) * 2 + 1] = (float)(alpha * im);
                }
    }
}
