// Stores of results that the next kernel reads exactly once.
//  * store_wt (spectra, contraction results): write-through at device scope.  The data reaches the memory
//    side while the kernel runs instead of waiting in the L2 for the write-back at the end of the kernel, and
//    the 256 MB memory-side cache keeps it for the kernel that reads it next.
//  * store_nt (the inverse transform's real output, whose reader is another layer): non-temporal, streamed
//    past the caches.
// Measured on MI355X, training step of batch 128, 128 -> 128 planes, 13 x 13, k3 (19-MB spectra): spectra
// non-temporal 120.8 us, ordinary stores 117.2, write-through 115.4; with the contraction's result written
// through as well (it was non-temporal) 113.3 us.  Alone, the forward transform takes 9.3 us with either of
// the two hints and 11.3 us with ordinary stores (its dirty lines are written back when the kernel ends).
// (A non-temporal hint on the loads of the inverse transform or of the contraction made them slower: what
// they read is still in a cache.)
#pragma once
#include <hip/hip_runtime.h>

namespace fbfc {

typedef float floatx2_nt __attribute__((ext_vector_type(2)));
typedef float floatx4_nt __attribute__((ext_vector_type(4)));

__device__ __forceinline__ void store_nt(float2 *p, const float2 &v)
{
    floatx2_nt t = {v.x, v.y};
    __builtin_nontemporal_store(t, reinterpret_cast<floatx2_nt *>(p));
}

__device__ __forceinline__ void store_nt(float4 *p, const float4 &v)
{
    floatx4_nt t = {v.x, v.y, v.z, v.w};
    __builtin_nontemporal_store(t, reinterpret_cast<floatx4_nt *>(p));
}

__device__ __forceinline__ void store_wt(float2 *p, const float2 &v)
{
    unsigned long long bits;
    __builtin_memcpy(&bits, &v, sizeof bits);
    // a relaxed device-scope atomic store of the 8 bytes: an ordinary vector store with the write-through policy
    __hip_atomic_store(reinterpret_cast<unsigned long long *>(p), bits, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

}  // namespace fbfc
