// Launch geometry shared by the EP kernels (gfx950: 64-lane wavefronts, 256-thread workgroups).
#ifndef TILEXR_AMD_EP_KERNEL_COMMON_CUH
#define TILEXR_AMD_EP_KERNEL_COMMON_CUH

#include <cstdint>

#if defined(__HIPCC__)
#include <hip/hip_runtime.h>
#endif

namespace TileXREp {

constexpr int kThreads = 256;
constexpr int kWave = 64;
constexpr int kWavesPerBlock = kThreads / kWave;

inline bool Aligned16(const void *p)
{
    return (reinterpret_cast<uintptr_t>(p) & 15u) == 0;
}

inline bool Aligned8(const void *p)
{
    return (reinterpret_cast<uintptr_t>(p) & 7u) == 0;
}

#if defined(__HIPCC__)
// Workgroup barrier that orders LDS traffic only: global stores still in flight are not waited for (a plain
// __syncthreads() drains them first, which costs a full store round trip when nobody in the workgroup reads them).
__device__ __forceinline__ void LdsBarrier()
{
#if defined(__HIP_DEVICE_COMPILE__)
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup", "local");
    __builtin_amdgcn_s_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup", "local");
#endif
}
#endif

} // namespace TileXREp

#endif // TILEXR_AMD_EP_KERNEL_COMMON_CUH
