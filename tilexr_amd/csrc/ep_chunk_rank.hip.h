// Stable rank of every live route within (chunk, key) for one workgroup of 256 lanes, shared by the two routing kernels
// (ep_count.hip: ranks + histograms for a later scan; ep_rows.hip: destination rows in one launch).
//
// A workgroup takes kThreads * BPW consecutive routes, wave w the w-th quarter of them, in batches of 64.  Lanes of a
// batch with equal keys find each other with one ballot per key bit; a key's running count within the wave, and the
// waves' shares of the chunk, live in LDS.  The result for lane l, batch b: the number of live routes of the same key
// earlier in the chunk (flat route order), or -1 for a route that is not live.
// Restates the reference's per-route pass `CalTokenSendExpertCnt` (number of earlier routes with the same expert,
// src/ep/kernels/tilexr_ep_dispatch_memory_kernel.h:791-818) in O(n); route liveness: ids outside [0, E) are skipped
// (:686-687), mask modes as in ep_launch.h (reference: :1387-1410, 1483-1500, 1538-1544).
#ifndef TILEXR_AMD_EP_CHUNK_RANK_HIP_H
#define TILEXR_AMD_EP_CHUNK_RANK_HIP_H

#include <hip/hip_runtime.h>

#include "ep_kernel_common.hip.h"
#include "ep_launch.h"
#include "ep_numerics.hip.h"

namespace TileXREp {

struct ChunkRouteArgs {
    const int32_t *ids;
    const uint8_t *mask;
    int maskMode;
    int bs;
    int topK;
    int numExperts;
    int keyDiv;
    int numKeys;
    int keyBits;
};

__device__ __forceinline__ unsigned long long LaneMaskLt()
{
    return (1ull << (threadIdx.x & (kWave - 1))) - 1ull;
}

// Routes at or beyond the returned index are not dispatched (token-prefix mask: only the first sum(mask) tokens are;
// reference: tilexr_ep_dispatch_memory_kernel.h:1387-1410, 1538-1544).  `s_sum` is one zeroed LDS word; contains a barrier.
__device__ __forceinline__ int ChunkLiveLimit(const ChunkRouteArgs &a, int *s_sum)
{
    const int n = a.bs * a.topK;
    if (a.maskMode != kMaskTokenPrefix) {
        return n;
    }
    int local = 0;
    for (int t = threadIdx.x; t < a.bs; t += kThreads) {
        local += a.mask[t] != 0 ? 1 : 0;
    }
    for (int off = kWave / 2; off >= 1; off >>= 1) {
        local += __shfl_xor(local, off);
    }
    if ((threadIdx.x & (kWave - 1)) == 0) {
        atomicAdd(s_sum, local);
    }
    __syncthreads();
    return *s_sum * a.topK;
}

template <int BPW>
__device__ __forceinline__ int ChunkRouteIndex(int chunk, int b)
{
    constexpr int kChunkRoutes = kThreads * BPW;
    const int wave = threadIdx.x / kWave;
    const int lane = threadIdx.x & (kWave - 1);
    return chunk * kChunkRoutes + wave * (kChunkRoutes / kWavesPerBlock) + b * kWave + lane;
}

// Loads the lane's BPW routes (all loads in flight together) and decides liveness and key; -1 = not live.  With
// `s_exp` (keys coarser than experts) the chunk's per-expert histogram is accumulated there.
template <int BPW>
__device__ __forceinline__ void ChunkRouteKeys(const ChunkRouteArgs &a, int chunk, int liveLimit, int *s_exp, int (&keys)[BPW])
{
    const int n = a.bs * a.topK;
    int e[BPW];
    int m[BPW];
#pragma unroll
    for (int b = 0; b < BPW; ++b) {
        const int i = ChunkRouteIndex<BPW>(chunk, b);
        const bool inRange = i < n && i < liveLimit;
        e[b] = inRange ? a.ids[i] : -1;
        m[b] = 1;
        if (a.maskMode == kMaskPerToken) {
            m[b] = inRange ? a.mask[i / a.topK] : 0;
        } else if (a.maskMode == kMaskPerRoute) {
            m[b] = inRange ? a.mask[i] : 0;
        }
    }
#pragma unroll
    for (int b = 0; b < BPW; ++b) {
        const bool live = e[b] >= 0 && e[b] < a.numExperts && m[b] != 0;
        keys[b] = live ? (a.keyDiv == 1 ? e[b] : e[b] / a.keyDiv) : -1;
        if (s_exp != nullptr && live) {
            atomicAdd(&s_exp[e[b]], 1);
        }
    }
}

// packed[b] = lanes of the same key before this one | lanes of the same key << 8, and the wave's routes per key are
// added to s_cnt[wave * numKeys + key] (zeroed by the caller; one LDS atomic per distinct key of a batch).  The bit loop
// is outermost so that the BPW batches give independent instruction streams.
template <int BPW>
__device__ __forceinline__ void ChunkMatchPeers(const ChunkRouteArgs &a, const int (&keys)[BPW], int *s_cnt, int (&packed)[BPW])
{
    const int wave = threadIdx.x / kWave;
    unsigned long long peers[BPW];
#pragma unroll
    for (int b = 0; b < BPW; ++b) {
        peers[b] = __ballot(keys[b] >= 0);
    }
    for (int bit = 0; bit < a.keyBits; ++bit) {
#pragma unroll
        for (int b = 0; b < BPW; ++b) {
            const bool one = keys[b] >= 0 && ((keys[b] >> bit) & 1);
            const unsigned long long bal = __ballot(one);
            peers[b] &= one ? bal : ~bal;
        }
    }
    const unsigned long long lt = LaneMaskLt();
#pragma unroll
    for (int b = 0; b < BPW; ++b) {
        const int before = __popcll(peers[b] & lt);
        const int same = __popcll(peers[b]);
        packed[b] = before | (same << 8);
        if (keys[b] >= 0 && before == 0) {
            atomicAdd(&s_cnt[wave * a.numKeys + keys[b]], same);
        }
    }
}

// After the caller has turned s_cnt[wave][key] into the exclusive sum over the waves (and passed a barrier): batches in
// order, the running count of a key within the wave lives in LDS (a wave's LDS operations execute in program order, the
// wave barriers only stop the compiler from reordering them).  packed[b] becomes the rank within (chunk, key), or -1.
template <int BPW>
__device__ __forceinline__ void ChunkRankRoutes(const ChunkRouteArgs &a, const int (&keys)[BPW], int *s_cnt, int (&packed)[BPW])
{
    volatile int *cnt = s_cnt + (threadIdx.x / kWave) * a.numKeys;
#pragma unroll
    for (int b = 0; b < BPW; ++b) {
        const int key = keys[b];
        const bool live = key >= 0;
        const int before = packed[b] & 0xff;
        const int base = live ? cnt[key] : 0;
        __builtin_amdgcn_wave_barrier();
        if (live && before == 0) {
            cnt[key] = base + (packed[b] >> 8);
        }
        __builtin_amdgcn_wave_barrier();
        packed[b] = live ? base + before : -1;
    }
}

// Workgroups behind the routing ones read 8 KiB of the token rows each and drop them.  The scatter that follows finds
// the rows in the memory-side cache; when it has to fetch them from HBM between its own writes it runs at little more
// than half its speed (4096 x 7168 x top-8: 140 us instead of 83).  Two 16-byte loads per lane: 58.7 MB cost 2 us on
// top of the routing workgroups' own waits, eight loads per lane cost 5.
constexpr int kWarmLoads = 2;

template <int THREADS = kThreads, int LOADS = kWarmLoads>
__device__ __forceinline__ void WarmTokenRows(const u32x4 *rows, int64_t vecs, int64_t workgroup)
{
    const int64_t base = workgroup * (THREADS * LOADS) + threadIdx.x;
    u32x4 v[LOADS];
#pragma unroll
    for (int i = 0; i < LOADS; ++i) {
        const int64_t at = base + static_cast<int64_t>(i) * THREADS;
        v[i] = rows[at < vecs ? at : vecs - 1];
    }
#pragma unroll
    for (int i = 0; i < LOADS; ++i) {
        asm volatile("" ::"v"(v[i]));
    }
}

inline unsigned WarmWorkgroups(int64_t vecs, int threads = kThreads, int loads = kWarmLoads)
{
    return static_cast<unsigned>((vecs + threads * loads - 1) / (threads * loads));
}

inline int KeyBits(int64_t numKeys)
{
    int bits = 0;
    while ((1ll << bits) < numKeys) {
        ++bits;
    }
    return bits;
}

} // namespace TileXREp

#endif // TILEXR_AMD_EP_CHUNK_RANK_HIP_H
