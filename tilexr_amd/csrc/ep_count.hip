// Routing kernels of the EP dispatch / combine path for gfx950 (CDNA4, wave64): count, place and invert.
//
// They turn the [bs, topK] expert-id table into destinations without moving a single payload byte:
//   count   stable rank of every live route within its key + histograms; the last workgroup scans them
//   place   destination row of every route, assist tuples, inverse map
//   invert  (combine side) row -> (token, k) inverse rebuilt from assist tuples
// All integer work; the reference behaviour each kernel restates is cited at the kernel.
#include <type_traits>

#include <hip/hip_runtime.h>

#include "ep_block_scan.hip.h"
#include "ep_kernel_common.hip.h"
#include "ep_launch.h"
#include "ep_numerics.hip.h"
#include "ep_place.hip.h"
#include "tilexr_ep.h"

namespace TileXREp {
namespace {


__device__ __forceinline__ unsigned long long LaneMaskLt()
{
    return (1ull << (threadIdx.x & (kWave - 1))) - 1ull;
}

// -------------------------------------------------------------------------------------------------------------
// count: stable rank of every live route within (chunk, key), per-chunk key histogram, and -- in the last
// workgroup to finish -- the scans that turn histograms into destinations and the count outputs.
//
// Replaces the reference's per-route O(n) pass (`CalTokenSendExpertCnt`, number of earlier routes with the same
// expert, src/ep/kernels/tilexr_ep_dispatch_memory_kernel.h:791-818), its count exchange and cumulative sum
// (:820-1089) and the count outputs (:1142-1168); for the MVP route the same machinery with a single key gives the
// token-major, k-minor compaction of src/ep/kernels/tilexr_ep_dispatch_kernel.cpp:501-571.
// Route liveness: ids outside [0, E) are skipped (:686-687); mask modes are described in ep_launch.h.
// -------------------------------------------------------------------------------------------------------------
struct RouteCountArgs {
    const int32_t *ids;
    const uint8_t *mask;
    int maskMode;
    int bs;
    int topK;
    int numExperts;
    int keyDiv;
    int numKeys;
    int keyBits;
    int capacity;
    int numChunks;
    CountScratch s;
    int32_t *sendCountsOut;
    int32_t *recvCountOut;
    int64_t *expertTokenNumsOut;
    int tokenNumsType;
    const u32x4 *warmRows;       // read once by the workgroups after the counting ones
    int64_t warmVecs;
};

constexpr int kWarmLoads = 2;    // 16-byte loads per lane of a warming workgroup (8 KiB per workgroup; 11.4 us for 58.7 MB, 14.3 us with eight)

// BPW = batches of 64 routes per wave: a workgroup counts 256 * BPW consecutive routes.
template <int BPW>
__global__ __launch_bounds__(kThreads) void ep_route_count_kernel(RouteCountArgs a)
{
    constexpr int kChunkRoutes = kThreads * BPW;
    __shared__ int s_cnt[kWavesPerBlock * kMaxKeys];
    __shared__ int s_exp[kMaxKeys];
    __shared__ int s_tot[kMaxKeys];     // single-chunk launches: the chunk's (= the launch's) routes per key
    __shared__ int s_part[kThreads];
    __shared__ int s_misc[4];

    const int tid = threadIdx.x;
    const int wave = tid / kWave;
    const int lane = tid & (kWave - 1);
    const int n = a.bs * a.topK;
    const int chunk = blockIdx.x;
    const bool expHist = a.s.chunkExpHist != nullptr;

    if (a.warmRows != nullptr && chunk >= a.numChunks) {
        // Not a counting workgroup: reads 8 KiB of the token rows and drops them.  The scatter that follows finds the
        // rows in the memory-side cache; when it has to fetch them from HBM between its own writes it runs at little
        // more than half its speed (4096 x 7168 x top-8: 140 us instead of 83).
        const int64_t base = static_cast<int64_t>(chunk - a.numChunks) * (kThreads * kWarmLoads) + tid;
        u32x4 v[kWarmLoads];
#pragma unroll
        for (int i = 0; i < kWarmLoads; ++i) {
            const int64_t at = base + static_cast<int64_t>(i) * kThreads;
            v[i] = a.warmRows[at < a.warmVecs ? at : a.warmVecs - 1];
        }
#pragma unroll
        for (int i = 0; i < kWarmLoads; ++i) {
            asm volatile("" ::"v"(v[i]));
        }
        return;
    }

    for (int i = tid; i < kWavesPerBlock * a.numKeys; i += kThreads) {
        s_cnt[i] = 0;
    }
    if (expHist) {
        for (int i = tid; i < a.numExperts; i += kThreads) {
            s_exp[i] = 0;
        }
    }
    if (tid == 0) {
        s_misc[0] = 0;
    }
    __syncthreads();

    int liveLimit = n;
    if (a.maskMode == kMaskTokenPrefix) {
        // activeCnt = sum(mask); only the first activeCnt tokens are dispatched
        // (reference: tilexr_ep_dispatch_memory_kernel.h:1387-1410, 1538-1544)
        int local = 0;
        for (int t = tid; t < a.bs; t += kThreads) {
            local += a.mask[t] != 0 ? 1 : 0;
        }
        for (int off = kWave / 2; off >= 1; off >>= 1) {
            local += __shfl_xor(local, off);
        }
        if (lane == 0) {
            atomicAdd(&s_misc[0], local);
        }
        __syncthreads();
        liveLimit = s_misc[0] * a.topK;
    }

    // phase A: load the wave's 64 * BPW consecutive routes (all loads in flight together), decide liveness and key
    int keys[BPW];
    {
        int e[BPW];
        int m[BPW];
#pragma unroll
        for (int b = 0; b < BPW; ++b) {
            const int i = chunk * kChunkRoutes + wave * (kChunkRoutes / kWavesPerBlock) + b * kWave + lane;
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
            if (expHist && live) {
                atomicAdd(&s_exp[e[b]], 1);
            }
        }
    }
    // lanes of a batch with equal keys find each other with one ballot per key bit; the bit loop is outermost so
    // that the BPW batches give independent instruction streams
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
    int packed[BPW];            // lanes of the same key before this one | lanes of the same key << 8
#pragma unroll
    for (int b = 0; b < BPW; ++b) {
        const int before = __popcll(peers[b] & lt);
        const int same = __popcll(peers[b]);
        packed[b] = before | (same << 8);
        if (keys[b] >= 0 && before == 0) {
            atomicAdd(&s_cnt[wave * a.numKeys + keys[b]], same);      // one LDS atomic per distinct key of a batch
        }
    }
    __syncthreads();

    // phase B: exclusive sum over the four waves; chunk totals to HBM
    for (int key = tid; key < a.numKeys; key += kThreads) {
        int run = 0;
#pragma unroll
        for (int w = 0; w < kWavesPerBlock; ++w) {
            const int v = s_cnt[w * a.numKeys + key];
            s_cnt[w * a.numKeys + key] = run;
            run += v;
        }
        if (a.numChunks == 1) {
            // the only chunk: its totals stay in LDS, its base within every key is zero, nobody has to be waited for
            s_tot[key] = run;
            a.s.chunkHist[key] = 0;
            continue;
        }
        // written through (agent scope): complete for the scanning workgroup, on whatever XCD it runs, once this
        // wave's stores have drained, with no write-back of the L2
        __hip_atomic_store(&a.s.chunkHist[static_cast<int64_t>(chunk) * a.numKeys + key], run, __ATOMIC_RELAXED,
            __HIP_MEMORY_SCOPE_AGENT);
    }
    if (expHist && a.numChunks > 1) {
        for (int e = tid; e < a.numExperts; e += kThreads) {
            __hip_atomic_store(&a.s.chunkExpHist[static_cast<int64_t>(chunk) * a.numExperts + e], s_exp[e],
                __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
    }
    __syncthreads();

    // phase C: batches in order; the running count of a key within the wave lives in LDS (a wave's LDS operations
    // execute in program order, the barriers only stop the compiler from reordering them)
    volatile int *cnt = s_cnt + wave * a.numKeys;
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

    // The last workgroup to arrive performs the scans.  Only the chunk histograms (stored in phase B, long since
    // on their way) have to be complete for it, so the ticket is taken before the rank stores are issued.
    if (a.numChunks > 1) {
        WaitOwnStores();
        __syncthreads();
        if (tid == 0) {
            const unsigned prev = atomicAdd(a.s.ticket, 1u);
            s_misc[1] = prev == static_cast<unsigned>(a.numChunks - 1) ? 1 : 0;
        }
    } else if (tid == 0) {
        s_misc[1] = 1;
    }
#pragma unroll
    for (int b = 0; b < BPW; ++b) {
        const int i = chunk * kChunkRoutes + wave * (kChunkRoutes / kWavesPerBlock) + b * kWave + lane;
        if (i < n) {
            a.s.localRank[i] = packed[b];
        }
    }
    LdsBarrier();
    if (s_misc[1] == 0) {
        return;
    }

    // per key: exclusive sum over chunks (becomes the chunk's base rank within the key), total, kept
    int *kept = s_cnt;                 // reuse: [numKeys]
    for (int key = tid; key < a.numKeys; key += kThreads) {
        int run = a.numChunks == 1 ? s_tot[key] : 0;
        // the loads of a batch are independent: one round trip per 32 chunks.  Whole batches run without a test per
        // load: this workgroup is alone on the launch's critical path and runs code nobody has fetched before it, so
        // the instructions it needs count as much as the memory round trips
        // (hence also buffer accesses: the chunk's offset is a scalar, one instruction per load)
        constexpr int kBatch = 32;
        int32_t *col = a.s.chunkHist + key;
        const int rowBytes = a.numKeys * 4;
        int c0 = 0;
        if (a.numChunks > 1 && static_cast<int64_t>(a.numChunks) * rowBytes < (int64_t{1} << 31)) {
            // chunks past the last one lie outside the buffer: their loads return zero, their stores are dropped
            const __amdgpu_buffer_rsrc_t hist = RowResource(a.s.chunkHist, a.numChunks * rowBytes);
            auto batches = [&](auto width) {
                constexpr int kWidth = decltype(width)::value;
                for (; c0 < a.numChunks; c0 += kWidth) {
                    int v[kWidth];
#pragma unroll
                    for (int u = 0; u < kWidth; ++u) {
                        v[u] = __builtin_amdgcn_raw_buffer_load_b32(hist, (c0 + u) * rowBytes + key * 4, 0, kAuxAgentScopeKept);
                    }
#pragma unroll
                    for (int u = 0; u < kWidth; ++u) {
                        __builtin_amdgcn_raw_buffer_store_b32(run, hist, (c0 + u) * rowBytes + key * 4, 0, 0);
                        run += v[u];
                    }
                }
            };
            if (a.numChunks <= kBatch) {
                batches(std::integral_constant<int, kBatch>{});
            } else {
                batches(std::integral_constant<int, 2 * kBatch>{});
            }
        }
#pragma unroll 1
        for (; c0 < a.numChunks && a.numChunks > 1; c0 += 4) {
            int v[4];
#pragma unroll
            for (int u = 0; u < 4; ++u) {
                const int c = c0 + u;
                v[u] = c < a.numChunks ? __hip_atomic_load(col + static_cast<int64_t>(c) * a.numKeys, __ATOMIC_RELAXED,
                    __HIP_MEMORY_SCOPE_AGENT) : 0;
            }
#pragma unroll
            for (int u = 0; u < 4; ++u) {
                const int c = c0 + u;
                if (c < a.numChunks) {
                    col[static_cast<int64_t>(c) * a.numKeys] = run;
                    run += v[u];
                }
            }
        }
        const int k = (a.capacity > 0 && run > a.capacity) ? a.capacity : run;
        kept[key] = k;
        a.s.keyKept[key] = k;
    }
    LdsBarrier();
    int *offs = s_cnt + kMaxKeys;      // [numKeys] exclusive offsets
    for (int key = tid; key < a.numKeys; key += kThreads) {
        offs[key] = kept[key];
    }
    LdsBarrier();
    const int totalRows = BlockExclusiveScan(offs, a.numKeys, s_part);
    for (int key = tid; key < a.numKeys; key += kThreads) {
        a.s.keyOffset[key] = offs[key];
        if (a.sendCountsOut != nullptr) {
            a.sendCountsOut[key] = offs[key] + kept[key];
        }
    }
    if (tid == 0) {
        a.s.keyOffset[a.numKeys] = totalRows;
        if (a.recvCountOut != nullptr) {
            a.recvCountOut[0] = totalRows;
        }
    }

    // per expert totals
    //   keys == experts: rows kept per expert (reference: tilexr_ep_dispatch_memory_kernel.h:1159-1168)
    //   coarser keys:    live routes per expert (reference: tilexr_ep_combine_helpers.h:49-80)
    int *etot = s_cnt + 2 * kMaxKeys;  // [numExperts]
    if (expHist) {
        for (int e = tid; e < a.numExperts; e += kThreads) {
            int run = a.numChunks == 1 ? s_exp[e] : 0;
            for (int c = 0; c < a.numChunks && a.numChunks > 1; ++c) {
                run += __hip_atomic_load(&a.s.chunkExpHist[static_cast<int64_t>(c) * a.numExperts + e], __ATOMIC_RELAXED,
                    __HIP_MEMORY_SCOPE_AGENT);
            }
            etot[e] = run;
        }
    } else {
        for (int e = tid; e < a.numExperts; e += kThreads) {
            etot[e] = e < a.numKeys ? kept[e] : 0;
        }
    }
    LdsBarrier();
    for (int e = tid; e < a.numExperts; e += kThreads) {
        a.s.expertTotal[e] = etot[e];
    }
    if (a.expertTokenNumsOut != nullptr) {
        if (a.tokenNumsType == 0 && !expHist) {
            // keys are experts: the inclusive prefix sum is the one already computed for the counts output
            for (int e = tid; e < a.numExperts; e += kThreads) {
                a.expertTokenNumsOut[e] = e < a.numKeys ? static_cast<int64_t>(offs[e]) + kept[e] : totalRows;
            }
        } else if (a.tokenNumsType == 0) {
            int *pref = s_cnt + 3 * kMaxKeys;
            for (int e = tid; e < a.numExperts; e += kThreads) {
                pref[e] = etot[e];
            }
            LdsBarrier();
            BlockExclusiveScan(pref, a.numExperts, s_part);
            for (int e = tid; e < a.numExperts; e += kThreads) {
                a.expertTokenNumsOut[e] = static_cast<int64_t>(pref[e]) + etot[e];
            }
        } else {
            for (int e = tid; e < a.numExperts; e += kThreads) {
                a.expertTokenNumsOut[e] = etot[e];
            }
        }
    }
    if (tid == 0 && a.numChunks > 1) {
        *a.s.ticket = 0u;
    }
}

// -------------------------------------------------------------------------------------------------------------
// place (stand-alone): destination row of every route + assist tuple + inverse map.  Used when they must be complete
// before the first row lands (readiness flags, a metadata-ready event) or when the rows go to a staging area;
// otherwise the scatter kernel resolves the rows of its own tokens (ep_place.hip.h).
// -------------------------------------------------------------------------------------------------------------
struct RoutePlaceArgs {
    PlaceArgs p;
};

__global__ __launch_bounds__(kThreads) void ep_route_place_kernel(RoutePlaceArgs a)
{
    const int i = blockIdx.x * kThreads + threadIdx.x;
    if (i < a.p.n) {
        PlaceRoute(a.p, i);
    }
}

// -------------------------------------------------------------------------------------------------------------
// invert: (token, k) -> row from the assist tuples, tagged with the call's epoch so the table never needs clearing.
//   memory route: rows [0, counts[last]) whose tuple names this rank and lies in range
//                 (reference: tilexr_ep_combine_memory_kernel.h:256-266, 329-342)
//   MVP route:    rows [0, sum of counts clamped to [0, maxCountPerEntry]); the tuple's rank field is not tested
//                 because the reference overwrites it while scattering (tilexr_ep_combine_kernel.cpp:28-52, 94-97)
// -------------------------------------------------------------------------------------------------------------
struct InvertArgs {
    const int32_t *assist;
    const int32_t *counts;
    int numCounts;
    int countsArePrefix;
    int maxRows;
    int maxCountPerEntry;
    int32_t rank;
    int bs;
    int topK;
    uint64_t epoch;
    uint64_t *inverse;
};

__global__ __launch_bounds__(kThreads) void ep_invert_kernel(InvertArgs a)
{
    __shared__ int s_rows;
    if (threadIdx.x == 0) {
        int rows = 0;
        if (a.countsArePrefix) {
            rows = a.counts[a.numCounts - 1];
        } else {
            for (int i = 0; i < a.numCounts; ++i) {
                const int c = a.counts[i];
                rows += (c < 0 || c > a.maxCountPerEntry) ? 0 : c;
            }
        }
        s_rows = rows < 0 ? 0 : (rows > a.maxRows ? a.maxRows : rows);
    }
    __syncthreads();
    const int row = blockIdx.x * kThreads + threadIdx.x;
    if (row >= s_rows) {
        return;
    }
    const int32_t *t = a.assist + static_cast<int64_t>(row) * 4;
    const int srcRank = t[0];
    const int token = t[1];
    const int k = t[2];
    if ((a.countsArePrefix && srcRank != a.rank) || token < 0 || token >= a.bs || k < 0 || k >= a.topK) {
        return;
    }
    // Two rows that name the same (token, k) -- only a corrupted table has them -- leave the higher row, whatever the
    // order the threads run in (the reference's sequential walk lets the later row win as well).  A word of another
    // epoch is stale and always replaced.
    unsigned long long *slot = reinterpret_cast<unsigned long long *>(&a.inverse[static_cast<int64_t>(token) * a.topK + k]);
    const unsigned long long mine = (a.epoch << 32) | static_cast<uint32_t>(row);
    unsigned long long seen = *slot;
    while ((seen >> 32) != a.epoch || seen < mine) {
        const unsigned long long prev = atomicCAS(slot, seen, mine);
        if (prev == seen) {
            break;
        }
        seen = prev;
    }
}

int KeyBits(int64_t numKeys)
{
    int bits = 0;
    while ((1ll << bits) < numKeys) {
        ++bits;
    }
    return bits;
}

} // namespace

// -------------------------------------------------------------------------------------------------------------
// host-side launchers
// -------------------------------------------------------------------------------------------------------------
CountScratchLayout PlanCountScratch(int64_t routes, int64_t numKeys, int64_t numExperts, bool expertHist)
{
    auto align = [](int64_t v) { return (v + 255) / 256 * 256; };
    CountScratchLayout p {};
    p.chunkShift = kMinChunkShift;
    while (p.chunkShift < kMaxChunkShift && ((routes + (1ll << p.chunkShift) - 1) >> p.chunkShift) > kTargetChunks) {
        ++p.chunkShift;
    }

    p.chunks = (routes + (1ll << p.chunkShift) - 1) >> p.chunkShift;
    int64_t off = 256;   // word 0 is the ticket
    p.localRankOff = off;
    off += align(routes * 4);
    p.rowOfOff = off;
    off += align(routes * 4);
    p.chunkHistOff = off;
    off += align(p.chunks * numKeys * 4);
    p.chunkExpHistOff = off;
    off += expertHist ? align(p.chunks * numExperts * 4) : 0;
    p.keyOffsetOff = off;
    off += align((numKeys + 1) * 4);
    p.keyKeptOff = off;
    off += align(numKeys * 4);
    p.expertTotalOff = off;
    off += align(numExperts * 4);
    p.totalBytes = off;
    return p;
}

hipError_t LaunchRouteCount(const RouteCountLaunch &l)
{
    RouteCountArgs a {};
    a.ids = l.ids;
    a.mask = l.mask;
    a.maskMode = l.maskMode;
    a.bs = static_cast<int>(l.bs);
    a.topK = static_cast<int>(l.topK);
    a.numExperts = static_cast<int>(l.numExperts);
    a.keyDiv = static_cast<int>(l.keyDiv);
    a.numKeys = static_cast<int>(l.numKeys);
    a.keyBits = KeyBits(l.numKeys);
    a.capacity = static_cast<int>(l.capacity);
    const int64_t n = l.bs * l.topK;
    const int shift = l.scratch.chunkShift;
    a.numChunks = static_cast<int>((n + (1ll << shift) - 1) >> shift);
    a.s = l.scratch;
    a.sendCountsOut = l.sendCountsOut;
    a.recvCountOut = l.recvCountOut;
    a.expertTokenNumsOut = l.expertTokenNumsOut;
    a.tokenNumsType = l.tokenNumsType;
    unsigned blocks = static_cast<unsigned>(a.numChunks > 0 ? a.numChunks : 1);
    if (a.numChunks > 0 && l.warmRows != nullptr && l.warmBytes >= 16 && Aligned16(l.warmRows)) {
        a.warmRows = static_cast<const u32x4 *>(l.warmRows);
        a.warmVecs = l.warmBytes / 16;
        blocks += static_cast<unsigned>((a.warmVecs + kThreads * kWarmLoads - 1) / (kThreads * kWarmLoads));
    }
    const dim3 grid(blocks);
    switch (shift) {
        case 10:
            hipLaunchKernelGGL(ep_route_count_kernel<4>, grid, dim3(kThreads), 0, l.stream, a);
            break;
        case 11:
            hipLaunchKernelGGL(ep_route_count_kernel<8>, grid, dim3(kThreads), 0, l.stream, a);
            break;
        case 12:
            hipLaunchKernelGGL(ep_route_count_kernel<16>, grid, dim3(kThreads), 0, l.stream, a);
            break;
        case 13:
            hipLaunchKernelGGL(ep_route_count_kernel<32>, grid, dim3(kThreads), 0, l.stream, a);
            break;
        default:
            return hipErrorInvalidValue;
    }
    return hipGetLastError();
}

hipError_t LaunchRoutePlace(const RoutePlaceLaunch &l)
{
    RoutePlaceArgs a {};
    a.p = MakePlaceArgs(l);
    const int grid = (a.p.n + kThreads - 1) / kThreads;
    hipLaunchKernelGGL(ep_route_place_kernel, dim3(grid > 0 ? grid : 1), dim3(kThreads), 0, l.stream, a);
    return hipGetLastError();
}

hipError_t LaunchInvert(const InvertLaunch &l)
{
    InvertArgs a {};
    a.assist = l.assist;
    a.counts = l.counts;
    a.numCounts = static_cast<int>(l.numCounts);
    a.countsArePrefix = l.countsArePrefix ? 1 : 0;
    a.maxRows = static_cast<int>(l.maxRows);
    a.maxCountPerEntry = static_cast<int>(l.maxCountPerEntry);
    a.rank = l.rank;
    a.bs = static_cast<int>(l.bs);
    a.topK = static_cast<int>(l.topK);
    a.epoch = l.epoch;
    a.inverse = l.inverse;
    const int grid = static_cast<int>((l.maxRows + kThreads - 1) / kThreads);
    hipLaunchKernelGGL(ep_invert_kernel, dim3(grid > 0 ? grid : 1), dim3(kThreads), 0, l.stream, a);
    return hipGetLastError();
}

} // namespace TileXREp
