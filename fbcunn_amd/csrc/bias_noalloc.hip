// The bias gradient for callers that cannot allocate device memory (code under HIP graph
// capture, tight serving loops, harnesses that forbid hipMalloc).
//
// fbfc_acc_grad_parameters_bias takes its partial sums' workspace from the caller; the entry
// point built on this file keeps them in a fixed array in device memory instead.  Every GPU the
// library runs on holds its own copy of the array, at its own address, until the process ends.
// In host code the array's name is only a stand-in for the symbol: it is never passed to a kernel,
// a memset or a copy.  The address on a device comes from hipGetSymbolAddress, looked up once per
// device with that device current, and that pointer is what the kernels get.
#include <hip/hip_runtime.h>

#include <atomic>
#include <mutex>

#include "kernels.h"

namespace fbfc {

// kNoAllocMaxPlanes planes x 16 batch slices (the most bias_grad_scratch_bytes ever asks for per
// plane) of one float: 256 KB.
constexpr int kNoAllocMaxPlanes = 4096;
constexpr int kNoAllocSlices = 16;
static __device__ __align__(256) float scratch[kNoAllocMaxPlanes * kNoAllocSlices];

int bias_grad_noalloc_max_planes() { return kNoAllocMaxPlanes; }

// Device address of the current GPU's copy of the array; nullptr and *err set on failure.
static float *scratch_on_current_device(hipError_t *err)
{
    static std::mutex mu;
    static std::atomic<float *> ptr[64] = {};
    int dev = 0;
    *err = hipGetDevice(&dev);
    if (*err != hipSuccess) return nullptr;
    if (dev < 0 || dev >= 64) {
        *err = hipErrorInvalidDevice;
        return nullptr;
    }
    // after the first call on a device the pointer is read without the lock
    float *known = ptr[dev].load(std::memory_order_acquire);
    if (known != nullptr) return known;
    std::lock_guard<std::mutex> lock(mu);
    known = ptr[dev].load(std::memory_order_relaxed);
    if (known == nullptr) {
        void *p = nullptr;
        *err = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
        if (*err != hipSuccess) return nullptr;
        known = static_cast<float *>(p);
        ptr[dev].store(known, std::memory_order_release);
    }
    return known;
}

hipError_t bias_grad_noalloc_prepare()
{
    hipError_t e = hipSuccess;
    (void)scratch_on_current_device(&e);
    return e;
}

hipError_t launch_bias_grad_noalloc(const float *grad_out, float *grad_bias, float scale, int batch,
                                    int planes, int hw, hipStream_t s)
{
    if (planes > kNoAllocMaxPlanes || bias_grad_scratch_bytes(batch, planes) > sizeof(float) * kNoAllocMaxPlanes * kNoAllocSlices)
        return hipErrorInvalidValue;
    hipError_t e = hipSuccess;
    float *ptr = scratch_on_current_device(&e);
    if (ptr == nullptr) return e;
    // The first kernel writes every partial sum the second one reads (planes x slices of this call),
    // so what an earlier, larger call left in the array is never read and nothing needs clearing.
    return launch_bias_grad(grad_out, grad_bias, scale, batch, planes, hw, ptr, s);
}

}  // namespace fbfc
