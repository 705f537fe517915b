// Device-side helpers for code that publishes or consumes the tile readiness words of libtilexr-ep (HIP, gfx950).
//
// The counterpart of the producer / consumer helpers the reference ships in a public header for its own flag protocol
// (src/include/tilexr_data_as_flag.h:22-53).  An expert stage that runs between TileXRMoeEpDispatchMemoryEx and
// TileXRMoeEpCombineMemoryEx and wants the combine to start on tiles as they complete includes this file instead of
// restating the rule below in its own words; the library's kernels use the same functions.
//
// A readiness word covers `tileRows` consecutive rows of a row buffer.  It is (epoch << 32) | rows in the tile, it is
// stored once per epoch, and it is never cleared: a word of any other epoch, and a zero-filled word, mean "not ready".
//
// The ordering rule.  gfx950 has one L2 per XCD and they are not coherent with one another, so "the rows are visible
// before the word" has to be made true explicitly, on both sides:
//
//   producer   1. every lane that wrote part of the tile waits for its own stores (TileXREpWaitOwnStores) and the
//                 lanes meet (a barrier, or whatever the kernel uses to know the tile is complete);
//              2. ONE lane calls TileXREpReleaseRowsToAgent() -- unless every row byte was written with
//                 TileXREpStoreRowVector (write-through), in which case step 1 already made the rows complete;
//              3. that lane calls TileXREpPublishTile().
//              The release in step 2 must be COMPLETE before the word is stored.  A bare
//              __builtin_amdgcn_fence(__ATOMIC_RELEASE, "agent") is not enough with hipcc 7.2: it becomes the L2
//              write-back instruction followed directly by the next store, the wait for the write-back is not in the
//              generated code, and the word then overtakes the rows now and then (seen as one wrongly summed token in
//              a few thousand).  TileXREpReleaseRowsToAgent spells the wait out.
//
//   consumer   1. look at the word with TileXREpTilePublished() (a relaxed load from memory: polling costs the
//                 producer nothing, no cache maintenance per poll);
//              2. then either read the rows with TileXREpLoadRowVector (served from memory, no stale line of this
//                 XCD's L2 can be hit), or have EVERY wave that will read the rows with ordinary loads call
//                 TileXREpAcquireRowsFromAgent() after the look that succeeded and before its first row load.  The
//                 acquire of one wave does not cover the loads of another: an invalidate that is still in flight when
//                 a sibling wave's load issues leaves that load free to hit the old line.
//
// Streams: a consumer that waits must be enqueued after its producer (streams of one process may share a hardware
// queue, where a waiting kernel keeps later kernels behind it).
#ifndef TILEXR_EP_PUBLISH_HIP_H
#define TILEXR_EP_PUBLISH_HIP_H

#include <cstdint>

#include <hip/hip_runtime.h>

// The word a complete tile is published with.
__host__ __device__ inline uint64_t TileXREpTileReadyWord(uint64_t epoch, int rowsInTile)
{
    return (epoch << 32) | static_cast<uint32_t>(rowsInTile);
}

// The consumer's test of a word it has loaded: published for exactly this epoch.
__host__ __device__ inline bool TileXREpTileWordReady(uint64_t word, uint64_t epoch)
{
    return (word >> 32) == epoch;
}

#if defined(__HIPCC__)

typedef uint32_t TileXREpRowVector __attribute__((ext_vector_type(4)));

// Waits until every store this wave has issued is complete.
__device__ __forceinline__ void TileXREpWaitOwnStores()
{
    __builtin_amdgcn_s_waitcnt(0);
}

// Release at agent scope for rows written with ordinary stores.  When the call returns, everything this wave has stored
// -- and, after a barrier that followed their own waits, what the other waves of its workgroup have stored -- is in
// memory for every XCD.  Writes this XCD's L2 back and waits for the write-back.
__device__ __forceinline__ void TileXREpReleaseRowsToAgent()
{
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "agent");
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
}

// Acquire at agent scope for rows that will be read with ordinary loads.  When the call returns, this XCD's L2 (and
// this compute unit's vector cache) hold no line older than the call, for the calling wave's later loads.  Invalidates,
// then waits for the invalidate: the same missing wait as on the release side would let a load that follows issue
// while the old line is still there.  Every wave that reads published rows calls it itself.
__device__ __forceinline__ void TileXREpAcquireRowsFromAgent()
{
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "agent");
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
}

// Stores the word of `tile`: call after the rows are complete in memory (see the ordering rule).
__device__ __forceinline__ void TileXREpPublishTile(uint64_t *tileFlags, int64_t tile, uint64_t epoch, int rowsInTile)
{
    __hip_atomic_store(&tileFlags[tile], TileXREpTileReadyWord(epoch, rowsInTile), __ATOMIC_RELAXED,
        __HIP_MEMORY_SCOPE_AGENT);
}

// One look at the word of `tile`, from memory.
__device__ __forceinline__ bool TileXREpTilePublished(const uint64_t *tileFlags, int64_t tile, uint64_t epoch)
{
    const uint64_t word = __hip_atomic_load(&tileFlags[tile], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    return TileXREpTileWordReady(word, epoch);
}

// 16 bytes of a row, written through to memory (complete for every XCD once the wave's own stores are waited for) and
// read from memory (never from a line this XCD's L2 kept from an earlier epoch).  `rowBytes` bounds the access: a
// byte offset at or beyond it stores nothing and loads zeros.
__device__ __forceinline__ void TileXREpStoreRowVector(void *row, int rowBytes, int byteOffset, TileXREpRowVector v)
{
    const __amdgpu_buffer_rsrc_t rsrc = __builtin_amdgcn_make_buffer_rsrc(row, 0, rowBytes, 0x00020000u);
    __builtin_amdgcn_raw_buffer_store_b128(v, rsrc, byteOffset, 0, 16 | 2);     // sc1 nt
}

__device__ __forceinline__ TileXREpRowVector TileXREpLoadRowVector(const void *row, int rowBytes, int byteOffset)
{
    const __amdgpu_buffer_rsrc_t rsrc = __builtin_amdgcn_make_buffer_rsrc(const_cast<void *>(row), 0, rowBytes,
        0x00020000u);
    return __builtin_amdgcn_raw_buffer_load_b128(rsrc, byteOffset, 0, 16 | 2);  // sc1 nt
}

#endif // __HIPCC__

#endif // TILEXR_EP_PUBLISH_HIP_H
