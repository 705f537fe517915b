// Exchange kernels for logical ranks that share one device (gfx950): drain (dispatch) and return (combine).
//
// They stand where the reference moves rows between peer windows:
//   MVP route      per-source slots drained in source-rank order, recvCounts[src], expertTokenNums
//                  (reference: src/ep/kernels/tilexr_ep_combine_helpers.h:81-145, tilexr_ep_dispatch_kernel.cpp:783-817)
//   memory route   segments ordered local expert -> source rank, sendCounts = inclusive sum, expertTokenNums from it
//                  (reference: src/ep/kernels/tilexr_ep_dispatch_memory_kernel.h:1017-1089, 1142-1168, 1208-1317)
//   combine        rows go back to the slot (token, k) of their source rank
//                  (reference: tilexr_ep_combine_memory_kernel.h:329-386, tilexr_ep_combine_kernel.cpp:28-52)
// On one device the "window" is ordinary HBM owned by the world, and readiness is stream order, not flags.
#include <hip/hip_runtime.h>

#include "ep_block_scan.hip.h"
#include "ep_exchange.h"
#include "ep_kernel_common.hip.h"
#include "ep_launch.h"

namespace TileXREp {
namespace {

// Segment idx of destination rank dstRank: which source's staging area it comes from and under which key.
//   memory route             local expert major, source minor
//   MVP route                one segment per source
//   MVP route, tp lanes      the sources of the rank's own lane first (in expert-rank order), then those of the other
//                            lanes of its group in lane order; the key is the expert rank
//                            (reference: src/ep/kernels/tilexr_ep_dispatch_kernel.cpp:809-827, 662-697)
__device__ __forceinline__ void SegmentOf(int idx, int rankSize, int dstRank, int localExperts, bool memoryRoute, int tp,
    int *src, int *key)
{
    if (memoryRoute) {
        *src = idx % rankSize;
        *key = dstRank * localExperts + idx / rankSize;
    } else if (tp <= 1) {
        *src = idx;
        *key = dstRank;
    } else {
        const int expertRanks = rankSize / tp;
        const int myLane = dstRank % tp;
        const int block = idx / expertRanks;
        const int lane = block == 0 ? myLane : (block - 1 < myLane ? block - 1 : block);
        *src = (idx % expertRanks) * tp + lane;
        *key = dstRank / tp;
    }
}

// Shared experts: route table of one source rank in the world's key space.
//   shared route s   -> rank srcRank % per + s * per (per = sharedRanks / sharedNum), tuple expert id s
//   routed id e      -> rank sharedRanks + e / localExperts, local index e % localExperts, tuple expert id sharedNum + e
// (reference: src/ep/kernels/tilexr_ep_dispatch_helpers.h:78-103, tilexr_ep_dispatch_memory_kernel.h:635-643,686-688,
//  tests/ep/demo/tilexr_ep_dispatch_demo.cpp:647-673)
struct AugmentArgs {
    const int32_t *ids;
    int n;                   // bs * (sharedNum + topK)
    int topK;
    int moeExpertNum;
    int srcRank;
    int sharedNum;
    int sharedRanks;
    int localExperts;
    int keysPerRank;
    int sharedAtExpertId;
    int32_t *keyIdsOut;
    int32_t *tupleExpertsOut;
    const uint8_t *routeMask;
    uint8_t *routeMaskOut;
};

__global__ __launch_bounds__(kThreads) void ep_augment_kernel(AugmentArgs a)
{
    const int i = blockIdx.x * kThreads + threadIdx.x;
    if (i >= a.n) {
        return;
    }
    const int perToken = a.sharedNum + a.topK;
    const int token = i / perToken;
    const int pos = i % perToken;
    int keyId = -1;
    int tupleExpert = -1;
    if (pos < a.sharedNum) {
        const int per = a.sharedRanks / a.sharedNum;
        const int dst = a.srcRank % per + pos * per;
        keyId = dst * a.keysPerRank + (a.sharedAtExpertId ? pos : 0);
        tupleExpert = pos;
    } else {
        const int e = a.ids[token * a.topK + (pos - a.sharedNum)];
        if (e >= 0 && e < a.moeExpertNum) {
            keyId = (a.sharedRanks + e / a.localExperts) * a.keysPerRank + e % a.localExperts;
            tupleExpert = a.sharedNum + e;
        }
    }
    a.keyIdsOut[i] = keyId;
    a.tupleExpertsOut[i] = tupleExpert;
    if (a.routeMaskOut != nullptr) {
        // (reference: src/ep/kernels/tilexr_ep_dispatch_memory_kernel.h:1412-1441 keeps the tokens whose mask row
        // has a set byte and walks the shared routes over those, :641-647)
        uint8_t live = 0;
        if (pos < a.sharedNum) {
            for (int k = 0; k < a.topK; ++k) {
                live |= a.routeMask[token * a.topK + k];
            }
        } else {
            live = a.routeMask[token * a.topK + (pos - a.sharedNum)];
        }
        a.routeMaskOut[i] = live != 0 ? 1 : 0;
    }
}

struct DrainPlanArgs {
    StageLayout stage;
    int rankSize;
    int dstRank;
    int localExperts;
    int outLocalExperts;
    int tokenNumsCount;
    int tp;
    int memoryRoute;
    int32_t *planOffsets;
    int32_t *countsOut;
    int32_t *tpCountsOut;
    int64_t *expertTokenNumsOut;
    int tokenNumsType;
};

__global__ __launch_bounds__(kThreads) void ep_drain_plan_kernel(DrainPlanArgs a)
{
    __shared__ int s_cnt[kMaxKeys];
    __shared__ int s_off[kMaxKeys];
    __shared__ int s_tok[kMaxKeys];
    __shared__ int s_part[kThreads];
    const int tid = threadIdx.x;
    const int numSeg = a.memoryRoute ? a.outLocalExperts * a.rankSize : a.rankSize;
    for (int idx = tid; idx < numSeg; idx += kThreads) {
        int src, key;
        SegmentOf(idx, a.rankSize, a.dstRank, a.localExperts, a.memoryRoute != 0, a.tp, &src, &key);
        const int32_t *ko = a.stage.counts + static_cast<int64_t>(src) * a.stage.countsStride;
        const int c = ko[key + 1] - ko[key];
        s_cnt[idx] = c;
        s_off[idx] = c;
    }
    __syncthreads();
    const int total = BlockExclusiveScan(s_off, numSeg, s_part);
    const int expertRanks = a.tp > 1 ? a.rankSize / a.tp : a.rankSize;
    for (int idx = tid; idx < numSeg; idx += kThreads) {
        a.planOffsets[idx] = s_off[idx];
        if (a.memoryRoute) {
            a.countsOut[idx] = s_off[idx] + s_cnt[idx];
        } else if (idx < expertRanks) {
            // plain per-source counts, indexed by the source's rank; with tp lanes only the rank's own lane is
            // counted here and the other entries are left alone (reference: tilexr_ep_combine_helpers.h:92-95)
            int src, key;
            SegmentOf(idx, a.rankSize, a.dstRank, a.localExperts, false, a.tp, &src, &key);
            a.countsOut[src] = s_cnt[idx];
            if (a.tpCountsOut != nullptr) {
                a.tpCountsOut[src] = s_cnt[idx];
            }
        }
    }
    if (tid == 0) {
        a.planOffsets[numSeg] = total;
    }
    if (a.tp > 1 && a.tpCountsOut != nullptr) {
        // afterwards the first tp entries become rows per lane (reference: tilexr_ep_dispatch_kernel.cpp:818-827)
        __syncthreads();
        if (tid < a.tp) {
            int rows = 0;
            for (int es = 0; es < expertRanks; ++es) {
                rows += s_cnt[tid * expertRanks + es];
            }
            const int myLane = a.dstRank % a.tp;
            const int lane = tid == 0 ? myLane : (tid - 1 < myLane ? tid - 1 : tid);
            a.tpCountsOut[lane] = rows;
        }
    }
    // rows per local expert
    for (int le = tid; le < a.tokenNumsCount; le += kThreads) {
        int n = 0;
        if (a.memoryRoute) {
            for (int s = 0; s < a.rankSize; ++s) {
                n += s_cnt[le * a.rankSize + s];
            }
        } else {
            for (int s = 0; s < a.rankSize; ++s) {
                const int32_t *et = a.stage.counts + static_cast<int64_t>(s) * a.stage.countsStride +
                    a.stage.expertTotalOffset;
                n += et[(a.tp > 1 ? a.dstRank / a.tp : a.dstRank) * a.localExperts + le];
            }
        }
        s_tok[le] = n;
    }
    __syncthreads();
    if (a.tokenNumsType == 0) {
        for (int le = tid; le < a.tokenNumsCount; le += kThreads) {
            s_cnt[le] = s_tok[le];
        }
        __syncthreads();
        BlockExclusiveScan(s_cnt, a.tokenNumsCount, s_part);
        for (int le = tid; le < a.tokenNumsCount; le += kThreads) {
            a.expertTokenNumsOut[le] = static_cast<int64_t>(s_cnt[le]) + s_tok[le];
        }
    } else {
        for (int le = tid; le < a.tokenNumsCount; le += kThreads) {
            a.expertTokenNumsOut[le] = s_tok[le];
        }
    }
}

__device__ __forceinline__ void CopyBytes(char *dst, const char *src, int64_t bytes, int tid)
{
    if (((reinterpret_cast<uintptr_t>(dst) | reinterpret_cast<uintptr_t>(src) | static_cast<uintptr_t>(bytes)) & 15u) == 0) {
        const uint4 *s = reinterpret_cast<const uint4 *>(src);
        uint4 *d = reinterpret_cast<uint4 *>(dst);
        for (int64_t i = tid; i < bytes / 16; i += kThreads) {
            d[i] = s[i];
        }
    } else {
        for (int64_t i = tid; i < bytes; i += kThreads) {
            dst[i] = src[i];
        }
    }
}

struct DrainCopyArgs {
    StageLayout stage;
    int rankSize;
    int dstRank;
    int localExperts;
    int outLocalExperts;
    int tp;
    int memoryRoute;
    const int32_t *planOffsets;
    int64_t rowBytes;
    int64_t scaleBytesPerRow;
    char *expandXOut;
    int32_t *assistOut;
    char *scalesOut;
};

__global__ __launch_bounds__(kThreads) void ep_drain_copy_kernel(DrainCopyArgs a)
{
    const int numSeg = a.memoryRoute ? a.outLocalExperts * a.rankSize : a.rankSize;
    const int row = blockIdx.x;
    if (row >= a.planOffsets[numSeg]) {
        return;
    }
    // last segment whose exclusive offset is <= row (empty segments share an offset with their successor)
    int lo = 0;
    int hi = numSeg - 1;
    while (lo < hi) {
        const int mid = (lo + hi + 1) / 2;
        if (a.planOffsets[mid] <= row) {
            lo = mid;
        } else {
            hi = mid - 1;
        }
    }
    int src, key;
    SegmentOf(lo, a.rankSize, a.dstRank, a.localExperts, a.memoryRoute != 0, a.tp, &src, &key);
    const int32_t *ko = a.stage.counts + static_cast<int64_t>(src) * a.stage.countsStride;
    const int64_t srcRow = ko[key] + (row - a.planOffsets[lo]);
    const char *rows = a.stage.rows + static_cast<int64_t>(src) * a.stage.rowsStride;
    const char *aux = a.stage.aux + static_cast<int64_t>(src) * a.stage.auxStride;
    const int tid = threadIdx.x;
    CopyBytes(a.expandXOut + static_cast<int64_t>(row) * a.rowBytes, rows + srcRow * a.rowBytes, a.rowBytes, tid);
    if (tid < 4) {
        a.assistOut[static_cast<int64_t>(row) * 4 + tid] = reinterpret_cast<const int32_t *>(aux)[srcRow * 4 + tid];
    }
    if (a.scaleBytesPerRow > 0) {
        CopyBytes(a.scalesOut + static_cast<int64_t>(row) * a.scaleBytesPerRow,
            aux + a.stage.scalesOffset + srcRow * a.scaleBytesPerRow, a.scaleBytesPerRow, tid);
    }
}

struct ReturnRowsArgs {
    const char *expertOut;
    const int32_t *assist;
    const int32_t *counts;
    int numCounts;
    int memoryRoute;
    int maxCountPerEntry;
    int maxRows;
    int64_t rowBytes;
    int rankSize;
    int expertRank;
    int bs;
    int topK;
    uint64_t epoch;
    char *slots;
    int64_t slotsStride;
    uint64_t *meta;
    int64_t metaStride;
};

__global__ __launch_bounds__(kThreads) void ep_return_rows_kernel(ReturnRowsArgs a)
{
    __shared__ int s_src;
    __shared__ int s_total;
    const int row = blockIdx.x;
    if (threadIdx.x == 0) {
        int src = -1;
        int total = 0;
        if (a.memoryRoute) {
            total = a.counts[a.numCounts - 1];
        } else {
            // rows are grouped by the per-source counts; entries outside [0, max] read as 0
            for (int s = 0; s < a.numCounts; ++s) {
                int c = a.counts[s];
                c = (c < 0 || c > a.maxCountPerEntry) ? 0 : c;
                if (row >= total && row < total + c) {
                    src = s;
                }
                total += c;
            }
        }
        s_src = src;
        s_total = total < 0 ? 0 : (total > a.maxRows ? a.maxRows : total);
    }
    __syncthreads();
    if (row >= s_total) {
        return;
    }
    const int32_t *t = a.assist + static_cast<int64_t>(row) * 4;
    const int src = a.memoryRoute ? t[0] : s_src;
    const int token = t[1];
    const int k = t[2];
    if (src < 0 || src >= a.rankSize || token < 0 || token >= a.bs || k < 0 || k >= a.topK) {
        return;
    }
    const int64_t slot = static_cast<int64_t>(token) * a.topK + k;
    CopyBytes(a.slots + static_cast<int64_t>(src) * a.slotsStride + slot * a.rowBytes,
        a.expertOut + static_cast<int64_t>(row) * a.rowBytes, a.rowBytes, threadIdx.x);
    if (threadIdx.x == 0) {
        uint64_t *meta = a.meta + static_cast<int64_t>(src) * a.metaStride;
        meta[slot] = (a.epoch << 32) | static_cast<uint32_t>(slot);
        meta[static_cast<int64_t>(a.bs) * a.topK + slot] =
            (static_cast<uint64_t>(static_cast<uint32_t>(a.expertRank)) << 32) | static_cast<uint32_t>(row);
    }
}

} // namespace

hipError_t LaunchAugment(const AugmentLaunch &l)
{
    AugmentArgs a {};
    a.ids = l.ids;
    a.n = static_cast<int>(l.bs * (l.sharedNum + l.topK));
    a.topK = static_cast<int>(l.topK);
    a.moeExpertNum = static_cast<int>(l.moeExpertNum);
    a.srcRank = l.srcRank;
    a.sharedNum = l.sharedNum;
    a.sharedRanks = l.sharedRanks;
    a.localExperts = l.localExperts;
    a.keysPerRank = l.keysPerRank;
    a.sharedAtExpertId = l.sharedAtExpertId ? 1 : 0;
    a.keyIdsOut = l.keyIdsOut;
    a.tupleExpertsOut = l.tupleExpertsOut;
    a.routeMask = l.routeMask;
    a.routeMaskOut = l.routeMaskOut;
    const int grid = (a.n + kThreads - 1) / kThreads;
    hipLaunchKernelGGL(ep_augment_kernel, dim3(grid > 0 ? grid : 1), dim3(kThreads), 0, l.stream, a);
    return hipGetLastError();
}

hipError_t LaunchDrainPlan(const DrainPlanLaunch &l)
{
    DrainPlanArgs a {};
    a.stage = l.stage;
    a.rankSize = l.rankSize;
    a.dstRank = l.dstRank;
    a.localExperts = l.localExperts;
    a.outLocalExperts = l.outLocalExperts;
    a.tokenNumsCount = l.tokenNumsCount;
    a.tp = l.tp;
    a.memoryRoute = l.memoryRoute ? 1 : 0;
    a.planOffsets = l.planOffsets;
    a.countsOut = l.countsOut;
    a.tpCountsOut = l.tpCountsOut;
    a.expertTokenNumsOut = l.expertTokenNumsOut;
    a.tokenNumsType = l.tokenNumsType;
    hipLaunchKernelGGL(ep_drain_plan_kernel, dim3(1), dim3(kThreads), 0, l.stream, a);
    return hipGetLastError();
}

hipError_t LaunchDrainCopy(const DrainCopyLaunch &l)
{
    DrainCopyArgs a {};
    a.stage = l.stage;
    a.rankSize = l.rankSize;
    a.dstRank = l.dstRank;
    a.localExperts = l.localExperts;
    a.outLocalExperts = l.outLocalExperts;
    a.tp = l.tp;
    a.memoryRoute = l.memoryRoute ? 1 : 0;
    a.planOffsets = l.planOffsets;
    a.rowBytes = l.rowBytes;
    a.scaleBytesPerRow = l.scaleBytesPerRow;
    a.expandXOut = static_cast<char *>(l.expandXOut);
    a.assistOut = l.assistOut;
    a.scalesOut = static_cast<char *>(l.scalesOut);
    hipLaunchKernelGGL(ep_drain_copy_kernel, dim3(static_cast<unsigned>(l.maxRows)), dim3(kThreads), 0, l.stream, a);
    return hipGetLastError();
}

hipError_t LaunchReturnRows(const ReturnRowsLaunch &l)
{
    ReturnRowsArgs a {};
    a.expertOut = static_cast<const char *>(l.expertOut);
    a.assist = l.assist;
    a.counts = l.counts;
    a.numCounts = static_cast<int>(l.numCounts);
    a.memoryRoute = l.memoryRoute ? 1 : 0;
    a.maxCountPerEntry = static_cast<int>(l.maxCountPerEntry);
    a.maxRows = static_cast<int>(l.maxRows);
    a.rowBytes = l.rowBytes;
    a.rankSize = l.rankSize;
    a.expertRank = l.expertRank;
    a.bs = static_cast<int>(l.bs);
    a.topK = static_cast<int>(l.topK);
    a.epoch = l.epoch;
    a.slots = l.slots;
    a.slotsStride = l.slotsStride;
    a.meta = l.meta;
    a.metaStride = l.metaStride;
    hipLaunchKernelGGL(ep_return_rows_kernel, dim3(static_cast<unsigned>(l.maxRows)), dim3(kThreads), 0, l.stream, a);
    return hipGetLastError();
}

} // namespace TileXREp
