// Streaming stores.  Results that a later kernel reads exactly once (spectra, contraction results)
// are written with the non-temporal hint: measured on MI355X, the contraction's result stores then
// cost 1.5 us less per launch at 144 x 128^3 and the kernel that reads them is no slower.  (The same
// hint on the loads of the inverse transform made it slower: what it reads is still in cache.)
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

}  // namespace fbfc
