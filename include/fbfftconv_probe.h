/*
 * fbfftconv_probe — the one entry point of the MEASUREMENT library libfbfftconv_probe.so.
 * It has no counterpart in the reference and is not part of the product: the shipped
 * libfbfftconv.so contains neither this symbol nor the instrumented kernel behind it.
 */
#ifndef FBFFTCONV_PROBE_H
#define FBFFTCONV_PROBE_H

#ifdef __cplusplus
extern "C" {
#endif

/* The shader clock the 64x64 tile contraction kernel actually runs at.  Issues `launches`
 * back-to-back launches of the per-frequency product with clock counters in the kernel and returns,
 * for the last launch, shader-clock ticks per microsecond of workgroup lifetime in *mhz.
 * mode 0: C = A conj(B)^T with A (Q, m, k), B (Q, n, k) (updateOutput); mode 1: C = A B with
 * B (Q, k, n) (updateGradInput); mode 2: C = conj(A)^T B with A (Q, k, m), B (Q, k, n)
 * (accGradParameters); C (Q, m, n) is written unscaled.  m, n multiples of 64, k of 16, 16-byte
 * aligned operands.  ticks: four 64-bit counters in device memory, zeroed by the caller (the call
 * allocates nothing).  The MFMA peak is quoted at the 2.4 GHz peak clock; under sustained fp32 MFMA
 * load the chip runs lower, and this is the number that says how much lower.  Synchronises the
 * stream.  Returns 0, 1 (invalid argument) or 5 (HIP error). */
int fbfc_probe_contraction_clock(int mode, const float *A, const float *B, float *C, int n_freq, int m,
                                 int n, int k, int launches, unsigned long long *ticks, float *mhz,
                                 void *stream);

#ifdef __cplusplus
}
#endif
#endif /* FBFFTCONV_PROBE_H */
