// Small-batch dispatch in one launch (gfx950, wave64): decode-sized calls are bound by launch latency, not by HBM.
//
// Up to kSmallRoutes routes fit one workgroup's registers, so every workgroup counts the whole expert-id table for
// itself -- per-expert histogram in LDS, exclusive offsets, rank of its own token's routes among the earlier routes of
// the same expert -- while its token's row is already on its way from HBM, and then writes the row to its topK
// destination rows.  Workgroup 0 also writes the count outputs.  The results are the same as those of the count +
// scatter pair (same definitions, reference: src/ep/kernels/tilexr_ep_dispatch_memory_kernel.h:791-818, 1059-1074,
// 1159-1168, 1240-1258); only the number of launches differs.  With readiness flags the rows are written through to memory
// and reported landed as in the scatter kernels (ep_tile_publish.h); the rows the whole dispatch keeps, which the size of
// the last tile depends on, every workgroup has counted anyway or counts with four more ballots.
#include <type_traits>

#include <hip/hip_runtime.h>

#include "ep_block_scan.hip.h"
#include "ep_kernel_common.hip.h"
#include "ep_launch.h"
#include "ep_numerics.hip.h"
#include "ep_tile_publish.h"

namespace TileXREp {
namespace {

constexpr int kIdsPerLane = kSmallRoutes / kThreads;

struct SmallArgs {
    const void *x;
    const int32_t *ids;
    int bs;
    int h;
    int topK;
    int numExperts;
    int capacity;
    int32_t srcRank;
    int32_t expertIdBias;
    void *out;
    int32_t *assist;
    int32_t *rowOf;              // optional [bs, topK]
    int32_t *sendCountsOut;
    int64_t *expertTokenNumsOut;
    int tokenNumsType;
    TilePublishArgs tiles;       // flags == nullptr: none (totalRows is filled in by the kernels)
};

// A row's vectors: streaming stores, or -- when readiness flags are published -- stores written through to memory, which
// are complete for every XCD once the issuing wave's memory counter is zero.
template <bool WT>
__device__ __forceinline__ void SmallRowStore(const u32x4 &v, u32x4 *dst, __amdgpu_buffer_rsrc_t rsrc, int idx)
{
    if (WT) {
        __builtin_amdgcn_raw_buffer_store_b128(v, rsrc, idx * 16, 0, kAuxAgentScope);
    } else {
        __builtin_nontemporal_store(v, dst + idx);
    }
}

template <int V, bool WT>
__global__ __launch_bounds__(kThreads) void ep_dispatch_small_kernel(SmallArgs a)
{
    __shared__ int s_hist[kMaxKeys];     // routes per expert, then exclusive row offsets
    __shared__ int s_kept[kMaxKeys];
    __shared__ int s_rank[kMaxTopK];
    __shared__ int s_key[kMaxTopK];
    __shared__ int s_pos[kMaxTopK];
    __shared__ int s_part[kThreads];

    const int tid = threadIdx.x;
    const int token = blockIdx.x;
    const int n = a.bs * a.topK;
    const int vecs = a.h / 8;

    // the token's row: in flight while the routing is worked out
    const u32x4 *src = reinterpret_cast<const u32x4 *>(static_cast<const char *>(a.x) + static_cast<int64_t>(token) * a.h * 2);
    u32x4 v[V];
#pragma unroll
    for (int j = 0; j < V; ++j) {
        const int idx = j * kThreads + tid;
        v[j] = idx < vecs ? src[idx] : u32x4{0u, 0u, 0u, 0u};
    }
    int e[kIdsPerLane];
#pragma unroll
    for (int j = 0; j < kIdsPerLane; ++j) {
        const int i = j * kThreads + tid;
        const int id = i < n ? a.ids[i] : -1;
        e[j] = (id >= 0 && id < a.numExperts) ? id : -1;      // ids outside [0, E) are skipped, not errors
    }
    for (int k = tid; k < a.numExperts; k += kThreads) {
        s_hist[k] = 0;
    }
    if (tid < a.topK) {
        const int id = a.ids[token * a.topK + tid];
        s_key[tid] = (id >= 0 && id < a.numExperts) ? id : -1;
        s_rank[tid] = 0;
    }
    __syncthreads();
    const int first = token * a.topK;
#pragma unroll
    for (int j = 0; j < kIdsPerLane; ++j) {
        const int i = j * kThreads + tid;
        if (e[j] < 0) {
            continue;
        }
        atomicAdd(&s_hist[e[j]], 1);
        // rank of the token's route k within its expert = earlier routes (flat order) with the same expert
        if (i < first + a.topK) {
            for (int k = 0; k < a.topK; ++k) {
                if (i < first + k && s_key[k] == e[j]) {
                    atomicAdd(&s_rank[k], 1);
                }
            }
        }
    }
    __syncthreads();
    for (int k = tid; k < a.numExperts; k += kThreads) {
        const int c = s_hist[k];
        const int kept = (a.capacity > 0 && c > a.capacity) ? a.capacity : c;
        s_kept[k] = kept;
        s_hist[k] = kept;
    }
    __syncthreads();
    const int totalRows = BlockExclusiveScan(s_hist, a.numExperts, s_part);
    if (tid < a.topK) {
        const int key = s_key[tid];
        int row = -1;
        if (key >= 0 && (a.capacity <= 0 || s_rank[tid] < a.capacity)) {
            row = s_hist[key] + s_rank[tid];
            int32_t *tuple = a.assist + static_cast<int64_t>(row) * 4;
            tuple[0] = a.srcRank;
            tuple[1] = token;
            tuple[2] = tid;
            tuple[3] = key + a.expertIdBias;
        }
        s_pos[tid] = row;
        if (a.rowOf != nullptr) {
            a.rowOf[first + tid] = row;
        }
    }
    if (token == 0) {
        for (int k = tid; k < a.numExperts; k += kThreads) {
            const int incl = s_hist[k] + s_kept[k];
            a.sendCountsOut[k] = incl;
            if (a.expertTokenNumsOut != nullptr) {
                a.expertTokenNumsOut[k] = a.tokenNumsType == 0 ? incl : s_kept[k];
            }
        }
    }
    __syncthreads();
    for (int k = 0; k < a.topK; ++k) {
        const int row = __builtin_amdgcn_readfirstlane(s_pos[k]);
        if (row < 0) {
            continue;
        }
        u32x4 *dst = reinterpret_cast<u32x4 *>(static_cast<char *>(a.out) + static_cast<int64_t>(row) * a.h * 2);
        const __amdgpu_buffer_rsrc_t rsrc = RowResource(dst, vecs * 16);
#pragma unroll
        for (int j = 0; j < V; ++j) {
            const int idx = j * kThreads + tid;
            if (idx < vecs) {
                SmallRowStore<WT>(v[j], dst, rsrc, idx);
            }
        }
    }
    if (WT) {
        // every wave waits for its own stores, the barrier collects the waves, then the rows are reported landed
        WaitOwnStores();
        __syncthreads();
        if (tid < a.topK && s_pos[tid] >= 0) {
            TilePublishArgs t = a.tiles;
            t.totalRows = totalRows;
            DeviceTileOps ops;
            PublishLanded(ops, t, s_pos[tid], 1);
        }
    }
}

// Without a capacity limit a route's row needs no histogram at all:
//   row = (valid routes with a smaller expert id) + (earlier routes with the same expert id)
// so one workgroup per route counts those two sets over the id table and writes its one row.  Workgroup b < E also
// counts expert b's routes for the count outputs.  Eight times as many workgroups as tokens spread a decode batch
// over the whole chip.
//
// The launch is two round trips to memory (id table and token row out, the row's stores back) with the counting in
// between, and at this size the counting is paid in instructions: a wave that runs alone on its SIMD issues a dependent
// instruction every 4 ns or so.  So every lane counts its own ids with compares and adds (no ballot and scalar count
// per id), the four sets share two registers (16 bits each: at most 2048 ids), one pair of reductions per wave and one
// LDS exchange between the four waves finish it.  IDS = ids per lane (4: up to 1024 routes, 8: up to 2048).
template <int V, bool WT, int IDS>
__global__ __launch_bounds__(kThreads) void ep_dispatch_small_route_kernel(SmallArgs a)
{
    __shared__ int s_sum[kWavesPerBlock][3];     // per wave: smaller | earlier equal << 16, equal to blockIdx | not above << 16, valid

    const int tid = threadIdx.x;
    const int lane = tid & (kWave - 1);
    const int wave = tid / kWave;
    // Workgroup b runs on XCD b % 8: the K routes of token t go to workgroups of XCD t % 8, where the decode-sized
    // combine places the token's slices as well, so that the rows it reads are still in the L2 that they were written
    // through (the tokens are padded to a multiple of eight: a workgroup of the padding has no route, only an expert to
    // count for).
    const int placed = static_cast<int>(blockIdx.x) / kXcdCount;
    const int token = (placed / a.topK) * kXcdCount + static_cast<int>(blockIdx.x) % kXcdCount;
    const bool hasRoute = token < a.bs;
    const int route = hasRoute ? token * a.topK + placed % a.topK : 0;
    const int n = a.bs * a.topK;
    const int vecs = a.h / 8;

    const u32x4 *src = reinterpret_cast<const u32x4 *>(static_cast<const char *>(a.x) + static_cast<int64_t>(hasRoute ? token : 0) * a.h * 2);
    u32x4 v[V];
#pragma unroll
    for (int j = 0; j < V; ++j) {
        const int idx = j * kThreads + tid;
        v[j] = idx < vecs ? src[idx] : u32x4{0u, 0u, 0u, 0u};
    }
    int e[IDS];
#pragma unroll
    for (int j = 0; j < IDS; ++j) {
        const int i = j * kThreads + tid;
        e[j] = i < n ? a.ids[i] : -1;
    }
    const int mine = a.ids[route];
    const unsigned experts = static_cast<unsigned>(a.numExperts);
    const int key = hasRoute && static_cast<unsigned>(mine) < experts ? mine : -1;       // ids outside [0, E) are skipped, not errors
    const int expert = blockIdx.x;       // the expert this workgroup counts for the outputs (if there is one)
    int rowCounts = 0;      // valid ids below the key | earlier ids equal to it << 16
    int outCounts = 0;      // ids equal to `expert` | valid ids not above it << 16
    int valid = 0;
#pragma unroll
    for (int j = 0; j < IDS; ++j) {
        const int i = j * kThreads + tid;
        const unsigned id = static_cast<unsigned>(e[j]);
        const bool ok = id < experts;
        rowCounts += (ok && e[j] < key ? 1 : 0) + (e[j] == key && i < route ? 0x10000 : 0);
        outCounts += (e[j] == expert ? 1 : 0) + (ok && e[j] <= expert ? 0x10000 : 0);
        valid += ok ? 1 : 0;
    }
#pragma unroll
    for (int off = kWave / 2; off >= 1; off >>= 1) {
        rowCounts += __shfl_xor(rowCounts, off);
        outCounts += __shfl_xor(outCounts, off);
        if (WT) {
            valid += __shfl_xor(valid, off);
        }
    }
    if (lane == 0) {
        s_sum[wave][0] = rowCounts;
        s_sum[wave][1] = outCounts;
        s_sum[wave][2] = valid;
    }
    __syncthreads();
    const int rowSum = s_sum[0][0] + s_sum[1][0] + s_sum[2][0] + s_sum[3][0];
    const int row = key >= 0 ? (rowSum & 0xffff) + (rowSum >> 16) : -1;
    if (tid == 0) {
        if (row >= 0) {
            int32_t *tuple = a.assist + static_cast<int64_t>(row) * 4;
            tuple[0] = a.srcRank;
            tuple[1] = token;
            tuple[2] = route % a.topK;
            tuple[3] = key + a.expertIdBias;
        }
        if (a.rowOf != nullptr && hasRoute) {
            a.rowOf[route] = row;
        }
        if (expert < a.numExperts) {
            const int outSum = s_sum[0][1] + s_sum[1][1] + s_sum[2][1] + s_sum[3][1];
            a.sendCountsOut[expert] = outSum >> 16;
            if (a.expertTokenNumsOut != nullptr) {
                a.expertTokenNumsOut[expert] = a.tokenNumsType == 0 ? outSum >> 16 : outSum & 0xffff;
            }
        }
    }
    if (row < 0) {
        return;
    }
    u32x4 *dst = reinterpret_cast<u32x4 *>(static_cast<char *>(a.out) + static_cast<int64_t>(row) * a.h * 2);
    const __amdgpu_buffer_rsrc_t rsrc = RowResource(dst, vecs * 16);
#pragma unroll
    for (int j = 0; j < V; ++j) {
        const int idx = j * kThreads + tid;
        if (idx < vecs) {
            SmallRowStore<WT>(v[j], dst, rsrc, idx);
        }
    }
    if (WT) {
        WaitOwnStores();
        __syncthreads();        // uniform: a workgroup without a row has left as a whole
        if (tid == 0) {
            TilePublishArgs t = a.tiles;
            t.totalRows = s_sum[0][2] + s_sum[1][2] + s_sum[2][2] + s_sum[3][2];      // rows the whole dispatch keeps: the size of the last tile
            DeviceTileOps ops;
            PublishLanded(ops, t, row, 1);
        }
    }
}

} // namespace

bool SmallDispatchFits(const SmallDispatchLaunch &l)
{
    return l.bs * l.topK <= kSmallRoutes && l.numExperts <= kMaxKeys && l.topK <= kMaxTopK && l.h % 8 == 0 &&
        l.h / 8 <= 8 * kThreads && Aligned16(l.x) && Aligned16(l.out);
}

hipError_t LaunchSmallDispatch(const SmallDispatchLaunch &l)
{
    SmallArgs a {};
    a.x = l.x;
    a.ids = l.ids;
    a.bs = static_cast<int>(l.bs);
    a.h = static_cast<int>(l.h);
    a.topK = static_cast<int>(l.topK);
    a.numExperts = static_cast<int>(l.numExperts);
    a.capacity = static_cast<int>(l.capacity);
    a.srcRank = l.srcRank;
    a.expertIdBias = l.expertIdBias;
    a.out = l.out;
    a.assist = l.assist;
    a.rowOf = l.rowOf;
    a.sendCountsOut = l.sendCountsOut;
    a.expertTokenNumsOut = l.expertTokenNumsOut;
    a.tokenNumsType = l.tokenNumsType;
    const bool flags = l.tileFlags != nullptr;
    if (flags) {
        a.tiles.flags = l.tileFlags;
        a.tiles.counters = l.tileCounters;
        a.tiles.tileRows = static_cast<int>(l.tileRows);
        a.tiles.maxTiles = static_cast<int>((l.bs * l.topK + l.tileRows - 1) / l.tileRows);
        a.tiles.epoch = l.epoch;
    }
    const int64_t vecs = l.h / 8;
    const int v = vecs <= 2 * kThreads ? 2 : (vecs <= 4 * kThreads ? 4 : 8);
    auto launch = [&](auto kernel, dim3 grid) { hipLaunchKernelGGL(kernel, grid, dim3(kThreads), 0, l.stream, a); };
    if (l.capacity <= 0 && l.bs * l.topK >= l.numExperts) {
        // one workgroup per route (there are enough of them to cover the experts' count outputs)
        if (l.kernelNameOut != nullptr) {
            *l.kernelNameOut = "ep_dispatch_small_route_kernel";
        }
        const dim3 routes(static_cast<unsigned>(XcdPlacedUnits(static_cast<int>(l.bs), static_cast<int>(l.topK))));
        const bool few = l.bs * l.topK <= 4 * kThreads;
        auto pick = [&](auto vecsPerLane) {
            constexpr int kV = decltype(vecsPerLane)::value;
            if (few) {
                flags ? launch(ep_dispatch_small_route_kernel<kV, true, 4>, routes) : launch(ep_dispatch_small_route_kernel<kV, false, 4>, routes);
            } else {
                flags ? launch(ep_dispatch_small_route_kernel<kV, true, kIdsPerLane>, routes) : launch(ep_dispatch_small_route_kernel<kV, false, kIdsPerLane>, routes);
            }
        };
        if (v == 2) {
            pick(std::integral_constant<int, 2>{});
        } else if (v == 4) {
            pick(std::integral_constant<int, 4>{});
        } else {
            pick(std::integral_constant<int, 8>{});
        }
        return hipGetLastError();
    }
    const dim3 grid(static_cast<unsigned>(l.bs));
    if (l.kernelNameOut != nullptr) {
        *l.kernelNameOut = "ep_dispatch_small_kernel";
    }
    if (v == 2) {
        flags ? launch(ep_dispatch_small_kernel<2, true>, grid) : launch(ep_dispatch_small_kernel<2, false>, grid);
    } else if (v == 4) {
        flags ? launch(ep_dispatch_small_kernel<4, true>, grid) : launch(ep_dispatch_small_kernel<4, false>, grid);
    } else {
        flags ? launch(ep_dispatch_small_kernel<8, true>, grid) : launch(ep_dispatch_small_kernel<8, false>, grid);
    }
    return hipGetLastError();
}

} // namespace TileXREp
