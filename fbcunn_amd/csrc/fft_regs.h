// In-register complex FFT of a compile-time power-of-two length.
//
// One lane holds a whole length-N complex sequence in registers (re[N], im[N])
// and transforms it with fully unrolled radix-2 decimation-in-frequency
// butterflies.  Every array index and every twiddle factor is a compile-time
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
// One DIF butterfly of a length-LEN sub-transform starting at OFF:
//   a' = a + b ;  b' = (a - b) * W,  W = exp(-/+ 2 pi i K / LEN)  (- forward, + inverse)
template <int LEN, int OFF, int K, bool INV>
__host__ __device__ __forceinline__ void butterfly(float *re, float *im) {
    constexpr int H = LEN / 2;
    const float ar = re[OFF + K], ai = im[OFF + K];
    const float br = re[OFF + K + H], bi = im[OFF + K + H];
    re[OFF + K] = ar + br;
    im[OFF + K] = ai + bi;
    const float dr = ar - br, di = ai - bi;
    if constexpr (K == 0) {
        re[OFF + K + H] = dr;
        im[OFF + K + H] = di;
    } else if constexpr (4 * K == LEN) {  // W = -i (forward) / +i (inverse)
        re[OFF + K + H] = INV ? -di : di;
        im[OFF + K + H] = INV ? dr : -dr;
    } else if constexpr (8 * K == LEN) {  // W = (1 -/+ i) / sqrt2
        constexpr float s = 0.70710678118654752440f;
        re[OFF + K + H] = INV ? (dr - di) * s : (dr + di) * s;
        im[OFF + K + H] = INV ? (dr + di) * s : (di - dr) * s;
    } else if constexpr (8 * K == 3 * LEN) {  // W = (-1 -/+ i) / sqrt2
        constexpr float s = 0.70710678118654752440f;
        re[OFF + K + H] = INV ? (-dr - di) * s : (di - dr) * s;
        im[OFF + K + H] = INV ? (dr - di) * s : (-dr - di) * s;
    } else {
        constexpr float wr = (float)cos2pi(K, LEN);
        constexpr float wi = (float)(INV ? sin2pi(K, LEN) : -sin2pi(K, LEN));
        re[OFF + K + H] = dr * wr - di * wi;
        im[OFF + K + H] = dr * wi + di * wr;
    }
}

template <int LEN, int OFF, bool INV>
__host__ __device__ __forceinline__ void fft_dif(float *re, float *im) {
    if constexpr (LEN >= 2) {
        static_for<LEN / 2>([&](auto k) { butterfly<LEN, OFF, decltype(k)::value, INV>(re, im); });
        fft_dif<LEN / 2, OFF, INV>(re, im);
        fft_dif<LEN / 2, OFF + LEN / 2, INV>(re, im);
    }
}

// Input-pruned variant: only the first NZ inputs of the length-LEN sequence at OFF are non-zero (the
// caller leaves literal zeros in the others).  While half the length is at least NZ a butterfly has
// b = 0, so a' = a and b' = a * W for the NZ leading positions and nothing at all for the others;
// both halves then again have NZ leading non-zeros.
template <int LEN, int OFF, int K, bool INV>
__host__ __device__ __forceinline__ void butterfly_b0(float *re, float *im) {
    constexpr int H = LEN / 2;
    const float ar = re[OFF + K], ai = im[OFF + K];
    if constexpr (K == 0) {
        re[OFF + H] = ar;
        im[OFF + H] = ai;
    } else {
        constexpr float wr = (float)cos2pi(K, LEN);
        constexpr float wi = (float)(INV ? sin2pi(K, LEN) : -sin2pi(K, LEN));
        re[OFF + K + H] = ar * wr - ai * wi;
        im[OFF + K + H] = ar * wi + ai * wr;
    }
}

template <int LEN, int OFF, bool INV, int NZ>
__host__ __device__ __forceinline__ void fft_dif_nz(float *re, float *im) {
    if constexpr (LEN / 2 >= NZ && LEN >= 2) {
        static_for<NZ>([&](auto k) { butterfly_b0<LEN, OFF, decltype(k)::value, INV>(re, im); });
        fft_dif_nz<LEN / 2, OFF, INV, NZ>(re, im);
        fft_dif_nz<LEN / 2, OFF + LEN / 2, INV, NZ>(re, im);
    } else {
        fft_dif<LEN, OFF, INV>(re, im);
    }
}

// Unnormalised length-N transform of a sequence whose inputs from NZ on are literal zeros.
template <int N, int NZ, bool INV>
__host__ __device__ __forceinline__ void fft_inplace_nz(float (&re)[N], float (&im)[N]) {
    static_assert(NZ >= 1 && NZ <= N, "NZ leading non-zero inputs");
    fft_dif_nz<N, 0, INV, NZ>(re, im);
}

// Unnormalised length-N transform in place; output index k lives at brev<N>(k).
template <int N, bool INV>
__host__ __device__ __forceinline__ void fft_inplace(float (&re)[N], float (&im)[N]) {
    fft_dif<N, 0, INV>(re, im);
}

}  // namespace fbfc
