// Small-batch dispatch in one launch (gfx950, wave64): decode-sized calls are bound by launch latency, not by HBM.
//
// Up to kSmallRoutes routes fit one workgroup's registers, so every workgroup counts the whole expert-id table for
// itself -- per-expert histogram in LDS, exclusive offsets, rank of its own token's routes among the earlier routes of
// the same expert -- while its token's row is already on its way from HBM, and then writes the row to its topK
// destination rows.  Workgroup 0 also writes the count outputs.  The results are the same as those of the count +
// scatter pair (same definitions, reference: src/ep/kernels/tilexr_ep_dispatch_memory_kernel.h:791-818, 1059-1074,
// 1159-1168, 1240-1258); only the number of launches differs.
#include <hip/hip_runtime.h>

#include "ep_block_scan.cuh"
#include "ep_kernel_common.cuh"
#include "ep_launch.h"
#include "ep_numerics.cuh"

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
};

template <int V>
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
    BlockExclusiveScan(s_hist, a.numExperts, s_part);
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
#pragma unroll
        for (int j = 0; j < V; ++j) {
            const int idx = j * kThreads + tid;
            if (idx < vecs) {
                __builtin_nontemporal_store(v[j], dst + idx);
            }
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
    const dim3 grid(static_cast<unsigned>(l.bs));
    const int64_t vecs = l.h / 8;
    if (vecs <= 2 * kThreads) {
        hipLaunchKernelGGL(ep_dispatch_small_kernel<2>, grid, dim3(kThreads), 0, l.stream, a);
    } else if (vecs <= 4 * kThreads) {
        hipLaunchKernelGGL(ep_dispatch_small_kernel<4>, grid, dim3(kThreads), 0, l.stream, a);
    } else {
        hipLaunchKernelGGL(ep_dispatch_small_kernel<8>, grid, dim3(kThreads), 0, l.stream, a);
    }
    return hipGetLastError();
}

} // namespace TileXREp
