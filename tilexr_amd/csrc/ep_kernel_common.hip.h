// Launch geometry shared by the EP kernels (gfx950: 64-lane wavefronts, 256-thread workgroups).
#ifndef TILEXR_AMD_EP_KERNEL_COMMON_HIP_H
#define TILEXR_AMD_EP_KERNEL_COMMON_HIP_H

#include <cstdint>

#if defined(__HIPCC__)
#include <hip/hip_runtime.h>

#include "tilexr_ep_publish.hip.h"
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

// Cache-policy operand of raw buffer loads and stores on gfx950.  Each XCD has its own L2 and the L2s are not coherent
// with one another: an ordinary store may sit dirty in the writer's L2 until a release fence writes the whole L2 back
// (measured: a scatter of 32 768 rows with one such fence per row takes 965 us instead of 90 us), and an ordinary load
// may hit a stale line until an acquire fence invalidates the reader's L2 (measured: 240 us instead of 90 us for the
// reduce with one fence per token).  An agent-scope (sc1) store is written through to memory and is complete, for
// every XCD, when the wave's vmcnt reaches zero; an agent-scope load is served from memory.  Rows published through
// readiness flags therefore move with sc1 accesses and need no cache maintenance at all.  The streaming hint (nt)
// stays on: without it the written-through rows are also allocated in L2 and push out the input rows the sibling
// workgroups of a token share (measured: 132 us instead of 93 us for the scatter).
constexpr int kAuxAgentScope = 16 | 2;      // sc1 nt
constexpr int kAuxNonTemporal = 2;          // nt
constexpr int kAuxAgentScopeKept = 16;      // sc1 alone: for small tables a later kernel reads again (with nt on the
                                            // loads of the count kernel's histograms the scatter that resolves rows from
                                            // the same table afterwards ran 10 us slower: 92 instead of 82 us)
constexpr unsigned kRawBufferWord3 = 0x00020000u;

// Workgroup b of a launch runs on XCD b % kXcdCount.  Units (token x part) placed by XCD: unit u belongs to token
// (u / 8 / parts) * 8 + u % 8, part (u / 8) % parts, so that all parts of a token run on XCD token % 8; the tokens are
// padded to a multiple of eight.
constexpr int kXcdCount = 8;
__host__ __device__ inline int XcdPlacedUnits(int tokens, int parts)
{
    return (tokens + kXcdCount - 1) / kXcdCount * kXcdCount * parts;
}

__device__ __forceinline__ __amdgpu_buffer_rsrc_t RowResource(const void *row, int bytes)
{
    return __builtin_amdgcn_make_buffer_rsrc(const_cast<void *>(row), 0, bytes, kRawBufferWord3);
}

// Waits until every store this wave has issued is complete (vmcnt, expcnt and lgkmcnt all zero).
__device__ __forceinline__ void WaitOwnStores()
{
    TileXREpWaitOwnStores();
}

// Release / acquire at agent scope for rows that move with ordinary stores and loads: the installed header
// tilexr_ep_publish.hip.h holds the one implementation (and the ordering rule), so that a producer or consumer outside
// the library runs the same instructions as the kernels here.  Both spell out the wait that follows the cache
// operation: in the code hipcc 7.2 generates for the fence alone, the L2 write-back of a release is followed directly
// by the next store (the wait the fence asks for does not survive the compiler's wait-count pass), and a readiness word
// then reaches memory ahead of the rows now and then: one row in a few thousand was read before it was there.  The
// acquire side gets the same treatment, and every wave that reads rows with ordinary loads issues its own.
__device__ __forceinline__ void ReleaseRowsToAgent()
{
    TileXREpReleaseRowsToAgent();
}

__device__ __forceinline__ void AcquireRowsFromAgent()
{
    TileXREpAcquireRowsFromAgent();
}

// Device side of ep_tile_publish.h: relaxed agent-scope atomics.  The caller has made the row complete in memory
// first, so has every earlier counter of the tile, and the atomics on one counter are totally ordered: when the last
// one returns, all rows of the tile are in memory.
struct DeviceTileOps {
    __device__ __forceinline__ uint32_t FetchAdd(uint32_t *p)
    {
        return __hip_atomic_fetch_add(p, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
    __device__ __forceinline__ void Store(uint32_t *p, uint32_t v)
    {
        __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
    __device__ __forceinline__ void Store(uint64_t *p, uint64_t v)
    {
        __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
};
#endif

} // namespace TileXREp

#endif // TILEXR_AMD_EP_KERNEL_COMMON_HIP_H
