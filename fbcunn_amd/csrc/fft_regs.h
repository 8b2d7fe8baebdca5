// In-register complex FFT of a compile-time power-of-two length.
//
// One lane holds a whole length-N complex sequence in registers (re[N], im[N])
// and transforms it with fully unrolled radix-2 butterflies (input in natural order,
// one twiddle per block applied before the add/subtract, so that a butterfly is six
// multiply-adds).  Every array index and every twiddle factor is a compile-time
// constant, so the arrays never leave the register file.  The result is left in
// bit-reversed order: X[k] is found at position fbfc::brev<N>(k).
#pragma once
#include <hip/hip_runtime.h>
#include <utility>

namespace fbfc {

// ---- compile-time trigonometry -------------------------------------------------
constexpr double kPi = 3.14159265358979323846264338327950288;

constexpr double sin_taylor(double x) {  // |x| <= pi/4
    double x2 = x * x, term = x, sum = x;
    for (int i = 1; i <= 12; ++i) {
        term *= -x2 / double((2 * i) * (2 * i + 1));
        sum += term;
    }
    return sum;
}
constexpr double cos_taylor(double x) {  // |x| <= pi/4
    double x2 = x * x, term = 1.0, sum = 1.0;
    for (int i = 1; i <= 12; ++i) {
        term *= -x2 / double((2 * i - 1) * (2 * i));
        sum += term;
    }
    return sum;
}
// cos(2 pi k / n) and sin(2 pi k / n) for integers, octant-reduced exactly.
constexpr double cos2pi(int k, int n) {
    k %= n;
    if (k < 0) k += n;
    if (2 * k > n) k = n - k;                     // cos is even around pi
    if (4 * k > n) return -cos2pi(n - 2 * k, 2 * n);  // cos(pi - a) = -cos a, a = 2pi (n/2-k)/n
    if (8 * k > n) return sin_taylor(2.0 * kPi * double(n - 4 * k) / double(4 * n));  // cos a = sin(pi/2 - a)
    return cos_taylor(2.0 * kPi * double(k) / double(n));
}
constexpr double sin2pi(int k, int n) {
    // sin a = cos(a - pi/2) = cos(2 pi (4k - n) / (4n))
    return cos2pi(4 * k - n, 4 * n);
}

template <int N>
constexpr int brev(int k) {
    int r = 0;
    for (int b = 1; b < N; b <<= 1) {
        r = (r << 1) | (k & 1);
        k >>= 1;
    }
    return r;
}

// ---- compile-time loop ---------------------------------------------------------
template <int... Is, class F>
__host__ __device__ __forceinline__ void static_for_impl(std::integer_sequence<int, Is...>, F &&f) {
    (f(std::integral_constant<int, Is>{}), ...);
}
template <int N, class F>
__host__ __device__ __forceinline__ void static_for(F &&f) {
    static_for_impl(std::make_integer_sequence<int, N>{}, static_cast<F &&>(f));
}

// ---- butterflies ----------------------------------------------------------------
// The transform of a block x[0..LEN) at register offset OFF is the "twisted" DFT
//   X[k] = sum_n x[n] exp(-/+ 2 pi i n (k + theta) / LEN),   theta = TNUM / TDEN
// (- forward, + inverse; theta = 0 for the whole sequence).  Splitting k = 2 k' + b gives
//   y_b[n] = x[n] + (-1)^b T x[n + LEN/2],  T = exp(-/+ pi i theta),   n < LEN/2
//   X[2 k' + b] = twisted DFT of y_b with theta' = (b + theta) / 2:
// input in natural order, X[k] left at position brev(k), and ONE twiddle per block that multiplies
// the second operand BEFORE the add/subtract.  That form fuses into multiply-adds:
//   lo' = lo + T hi   (2 fma per component),   hi' = lo - T hi = 2 lo - lo'   (1 fma per component)
// 6 instructions for a butterfly with a non-trivial twiddle (a decimation-in-frequency butterfly,
// which multiplies after the subtraction, takes 8), 4 for T in {1, -/+ i}.
template <int TNUM, int TDEN, bool INV>
__host__ __device__ __forceinline__ void butterfly(float &ar, float &ai, float &br, float &bi) {
    if constexpr (TNUM == 0) {  // T = 1
        const float lr = ar + br, li = ai + bi;
        br = ar - br;
        bi = ai - bi;
        ar = lr;
        ai = li;
    } else if constexpr (2 * TNUM == TDEN) {  // T = -i (forward) / +i (inverse): T b = (bi, -br) / (-bi, br)
        const float pr = INV ? ar - bi : ar + bi, pi_ = INV ? ai + br : ai - br;
        const float qr = INV ? ar + bi : ar - bi, qi = INV ? ai - br : ai + br;
        ar = pr; ai = pi_;
        br = qr; bi = qi;
    } else {
        constexpr float tr = (float)cos2pi(TNUM, 2 * TDEN);
        constexpr float ti = (float)(INV ? sin2pi(TNUM, 2 * TDEN) : -sin2pi(TNUM, 2 * TDEN));
        // lo' = a + T b
        const float lr = __builtin_fmaf(tr, br, __builtin_fmaf(-ti, bi, ar));
        const float li = __builtin_fmaf(tr, bi, __builtin_fmaf(ti, br, ai));
        br = __builtin_fmaf(2.0f, ar, -lr);
        bi = __builtin_fmaf(2.0f, ai, -li);
        ar = lr;
        ai = li;
    }
}

template <int LEN, int OFF, int TNUM, int TDEN, bool INV>
__host__ __device__ __forceinline__ void fft_block(float *re, float *im) {
    if constexpr (LEN >= 2) {
        constexpr int H = LEN / 2;
        static_for<H>([&](auto kk) {
            constexpr int k = decltype(kk)::value;
            butterfly<TNUM, TDEN, INV>(re[OFF + k], im[OFF + k], re[OFF + k + H], im[OFF + k + H]);
        });
        fft_block<H, OFF, TNUM, 2 * TDEN, INV>(re, im);
        fft_block<H, OFF + H, TDEN + TNUM, 2 * TDEN, INV>(re, im);
    }
}

// Input-pruned variant: only the first NZ inputs of the block are non-zero (the caller leaves
// literal zeros in the others).  While half the block length is at least NZ every butterfly has
// hi = 0, so lo' = hi' = lo: the second half is a copy of the first, whatever the twiddle.
template <int LEN, int OFF, int TNUM, int TDEN, bool INV, int NZ>
__host__ __device__ __forceinline__ void fft_block_nz(float *re, float *im) {
    if constexpr (LEN / 2 >= NZ && LEN >= 2) {
        constexpr int H = LEN / 2;
        static_for<NZ>([&](auto kk) {
            constexpr int k = decltype(kk)::value;
            re[OFF + k + H] = re[OFF + k];
            im[OFF + k + H] = im[OFF + k];
        });
        fft_block_nz<H, OFF, TNUM, 2 * TDEN, INV, NZ>(re, im);
        fft_block_nz<H, OFF + H, TDEN + TNUM, 2 * TDEN, INV, NZ>(re, im);
    } else {
        fft_block<LEN, OFF, TNUM, TDEN, INV>(re, im);
    }
}

// Unnormalised length-N transform of a sequence whose inputs from NZ on are literal zeros.
template <int N, int NZ, bool INV>
__host__ __device__ __forceinline__ void fft_inplace_nz(float (&re)[N], float (&im)[N]) {
    static_assert(NZ >= 1 && NZ <= N, "NZ leading non-zero inputs");
    fft_block_nz<N, 0, 0, 1, INV, NZ>(re, im);
}

// Unnormalised length-N transform in place; output index k lives at brev<N>(k).
template <int N, bool INV>
__host__ __device__ __forceinline__ void fft_inplace(float (&re)[N], float (&im)[N]) {
    fft_block<N, 0, 0, 1, INV>(re, im);
}

}  // namespace fbfc
