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
#include "ep_chunk_rank.hip.h"
#include "ep_kernel_common.hip.h"
#include "ep_launch.h"
#include "ep_numerics.hip.h"
#include "ep_place.hip.h"
#include "tilexr_ep.h"

namespace TileXREp {
namespace {


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
    ChunkRouteArgs r;
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

// BPW = batches of 64 routes per wave: a workgroup counts 256 * BPW consecutive routes.
template <int BPW>
__global__ __launch_bounds__(kThreads) void ep_route_count_kernel(RouteCountArgs a)
{
    __shared__ int s_cnt[kWavesPerBlock * kMaxKeys];
    __shared__ int s_exp[kMaxKeys];
    __shared__ int s_tot[kMaxKeys];     // single-chunk launches: the chunk's (= the launch's) routes per key
    __shared__ int s_part[kThreads];
    __shared__ int s_misc[4];

    const int tid = threadIdx.x;
    const int numKeys = a.r.numKeys;
    const int numExperts = a.r.numExperts;
    const int n = a.r.bs * a.r.topK;
    const int chunk = blockIdx.x;
    const bool expHist = a.s.chunkExpHist != nullptr;

    if (a.warmRows != nullptr && chunk >= a.numChunks) {
        WarmTokenRows(a.warmRows, a.warmVecs, chunk - a.numChunks);     // not a counting workgroup
        return;
    }

    for (int i = tid; i < kWavesPerBlock * numKeys; i += kThreads) {
        s_cnt[i] = 0;
    }
    if (expHist) {
        for (int i = tid; i < numExperts; i += kThreads) {
            s_exp[i] = 0;
        }
    }
    if (tid == 0) {
        s_misc[0] = 0;
    }
    __syncthreads();

    // phase A: the lane's routes, their keys, their peers within each batch of 64
    const int liveLimit = ChunkLiveLimit(a.r, &s_misc[0]);
    int keys[BPW];
    int packed[BPW];
    ChunkRouteKeys<BPW>(a.r, chunk, liveLimit, expHist ? s_exp : nullptr, keys);
    ChunkMatchPeers<BPW>(a.r, keys, s_cnt, packed);
    __syncthreads();

    // phase B: exclusive sum over the four waves; chunk totals to HBM
    for (int key = tid; key < numKeys; key += kThreads) {
        int run = 0;
#pragma unroll
        for (int w = 0; w < kWavesPerBlock; ++w) {
            const int v = s_cnt[w * numKeys + key];
            s_cnt[w * numKeys + key] = run;
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
        __hip_atomic_store(&a.s.chunkHist[static_cast<int64_t>(chunk) * numKeys + key], run, __ATOMIC_RELAXED,
            __HIP_MEMORY_SCOPE_AGENT);
    }
    if (expHist && a.numChunks > 1) {
        for (int e = tid; e < numExperts; e += kThreads) {
            __hip_atomic_store(&a.s.chunkExpHist[static_cast<int64_t>(chunk) * numExperts + e], s_exp[e],
                __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
    }
    __syncthreads();

    // phase C: rank of every route within (chunk, key)
    ChunkRankRoutes<BPW>(a.r, keys, s_cnt, packed);

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
        const int i = ChunkRouteIndex<BPW>(chunk, b);
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
    for (int key = tid; key < numKeys; key += kThreads) {
        int run = a.numChunks == 1 ? s_tot[key] : 0;
        // the loads of a batch are independent: one round trip per 32 chunks.  Whole batches run without a test per
        // load: this workgroup is alone on the launch's critical path and runs code nobody has fetched before it, so
        // the instructions it needs count as much as the memory round trips
        // (hence also buffer accesses: the chunk's offset is a scalar, one instruction per load)
        constexpr int kBatch = 32;
        int32_t *col = a.s.chunkHist + key;
        const int rowBytes = numKeys * 4;
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
                v[u] = c < a.numChunks ? __hip_atomic_load(col + static_cast<int64_t>(c) * numKeys, __ATOMIC_RELAXED,
                    __HIP_MEMORY_SCOPE_AGENT) : 0;
            }
#pragma unroll
            for (int u = 0; u < 4; ++u) {
                const int c = c0 + u;
                if (c < a.numChunks) {
                    col[static_cast<int64_t>(c) * numKeys] = run;
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
    for (int key = tid; key < numKeys; key += kThreads) {
        offs[key] = kept[key];
    }
    LdsBarrier();
    const int totalRows = BlockExclusiveScan(offs, numKeys, s_part);
    for (int key = tid; key < numKeys; key += kThreads) {
        a.s.keyOffset[key] = offs[key];
        if (a.sendCountsOut != nullptr) {
            a.sendCountsOut[key] = offs[key] + kept[key];
        }
    }
    if (tid == 0) {
        a.s.keyOffset[numKeys] = totalRows;
        if (a.recvCountOut != nullptr) {
            a.recvCountOut[0] = totalRows;
        }
    }

    // per expert totals
    //   keys == experts: rows kept per expert (reference: tilexr_ep_dispatch_memory_kernel.h:1159-1168)
    //   coarser keys:    live routes per expert (reference: tilexr_ep_combine_helpers.h:49-80)
    int *etot = s_cnt + 2 * kMaxKeys;  // [numExperts]
    if (expHist) {
        for (int e = tid; e < numExperts; e += kThreads) {
            int run = a.numChunks == 1 ? s_exp[e] : 0;
            for (int c = 0; c < a.numChunks && a.numChunks > 1; ++c) {
                run += __hip_atomic_load(&a.s.chunkExpHist[static_cast<int64_t>(c) * numExperts + e], __ATOMIC_RELAXED,
                    __HIP_MEMORY_SCOPE_AGENT);
            }
            etot[e] = run;
        }
    } else {
        for (int e = tid; e < numExperts; e += kThreads) {
            etot[e] = e < numKeys ? kept[e] : 0;
        }
    }
    LdsBarrier();
    for (int e = tid; e < numExperts; e += kThreads) {
        a.s.expertTotal[e] = etot[e];
    }
    if (a.expertTokenNumsOut != nullptr) {
        if (a.tokenNumsType == 0 && !expHist) {
            // keys are experts: the inclusive prefix sum is the one already computed for the counts output
            for (int e = tid; e < numExperts; e += kThreads) {
                a.expertTokenNumsOut[e] = e < numKeys ? static_cast<int64_t>(offs[e]) + kept[e] : totalRows;
            }
        } else if (a.tokenNumsType == 0) {
            int *pref = s_cnt + 3 * kMaxKeys;
            for (int e = tid; e < numExperts; e += kThreads) {
                pref[e] = etot[e];
            }
            LdsBarrier();
            BlockExclusiveScan(pref, numExperts, s_part);
            for (int e = tid; e < numExperts; e += kThreads) {
                a.expertTokenNumsOut[e] = static_cast<int64_t>(pref[e]) + etot[e];
            }
        } else {
            for (int e = tid; e < numExperts; e += kThreads) {
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

} // namespace

// -------------------------------------------------------------------------------------------------------------
// host-side launchers
// -------------------------------------------------------------------------------------------------------------
CountScratchLayout PlanCountScratch(int64_t routes, int64_t numKeys, int64_t numExperts, bool expertHist)
{
    auto align = [](int64_t v) { return (v + 255) / 256 * 256; };
    CountScratchLayout p {};
    p.chunkShift = kMinChunkShift;
    const int64_t targetChunks = numKeys > 1024 ? kTargetChunks / 2 : kTargetChunks;
    while (p.chunkShift < kMaxChunkShift && ((routes + (1ll << p.chunkShift) - 1) >> p.chunkShift) > targetChunks) {
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
    a.r.ids = l.ids;
    a.r.mask = l.mask;
    a.r.maskMode = l.maskMode;
    a.r.bs = static_cast<int>(l.bs);
    a.r.topK = static_cast<int>(l.topK);
    a.r.numExperts = static_cast<int>(l.numExperts);
    a.r.keyDiv = static_cast<int>(l.keyDiv);
    a.r.numKeys = static_cast<int>(l.numKeys);
    a.r.keyBits = KeyBits(l.numKeys);
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
        blocks += WarmWorkgroups(a.warmVecs);
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
