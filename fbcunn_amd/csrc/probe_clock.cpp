// Measurement library (libfbfftconv_probe.so): the shader clock the 64x64 tile contraction kernel
// runs at.  Built from cgemm_kernels.hip with FBFC_PROBES defined plus this file; the shipped library
// contains none of it.  Nothing here allocates: the caller brings the tick counters.
#include <hip/hip_runtime.h>

#include "../../include/fbfftconv_probe.h"
#include "kernels.h"

namespace fbfc {
// the contraction launchers log what they launch; the probe library keeps no log
void kernel_log_clear() {}
void kernel_log_add(const char *, long) {}
const char *kernel_log_get() { return ""; }
bool launch_events_next(hipEvent_t *, hipEvent_t *) { return false; }
}  // namespace fbfc

extern "C" int fbfc_probe_contraction_clock(int mode, const float *A, const float *B, float *C, int n_freq, int m,
                                            int n, int k, int launches, unsigned long long *ticks, float *mhz,
                                            void *stream)
{
    if (A == nullptr || B == nullptr || C == nullptr || ticks == nullptr || mhz == nullptr || launches < 1) return 1;
    hipStream_t s = static_cast<hipStream_t>(stream);
    hipError_t e = hipSuccess;
    // the clock settles over the run of launches: the last one counts into ticks[0..1], the others
    // into ticks[2..3]
    for (int i = 0; i < launches && e == hipSuccess; ++i)
        e = fbfc::launch_cgemm_clock_probe(mode, A, B, C, n_freq, m, n, k, ticks + (i == launches - 1 ? 0 : 2), s);
    unsigned long long h[2] = {0, 0};
    if (e == hipSuccess) e = hipMemcpyAsync(h, ticks, sizeof h, hipMemcpyDeviceToHost, s);
    if (e == hipSuccess) e = hipStreamSynchronize(s);
    if (e == hipErrorInvalidValue) return 1;
    if (e != hipSuccess) return 5;
    *mhz = h[1] ? (float)((double)h[0] / ((double)h[1] / 100.0)) : 0.0f;
    return 0;
}
