// Launch geometry shared by the EP kernels (gfx950: 64-lane wavefronts, 256-thread workgroups).
#ifndef TILEXR_AMD_EP_KERNEL_COMMON_CUH
#define TILEXR_AMD_EP_KERNEL_COMMON_CUH

#include <cstdint>

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

} // namespace TileXREp

#endif // TILEXR_AMD_EP_KERNEL_COMMON_CUH
