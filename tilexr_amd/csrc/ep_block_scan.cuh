// Workgroup-wide exclusive scan in LDS (256 threads), shared by the routing and exchange kernels.
#ifndef TILEXR_AMD_EP_BLOCK_SCAN_CUH
#define TILEXR_AMD_EP_BLOCK_SCAN_CUH

#include <hip/hip_runtime.h>

#include "ep_kernel_common.cuh"

namespace TileXREp {

// Exclusive scan of vals[0..m) in place (LDS), m <= 2048, by all 256 threads.  part[] is 256 ints of LDS.
// Returns the total.
__device__ inline int BlockExclusiveScan(int *vals, int m, int *part)
{
    const int tid = threadIdx.x;
    const int per = (m + kThreads - 1) / kThreads;
    const int begin = tid * per;
    int local = 0;
    for (int i = begin; i < begin + per && i < m; ++i) {
        local += vals[i];
    }
    part[tid] = local;
    __syncthreads();
    for (int off = 1; off < kThreads; off <<= 1) {
        const int add = tid >= off ? part[tid - off] : 0;
        __syncthreads();
        part[tid] += add;
        __syncthreads();
    }
    int run = part[tid] - local;
    const int total = part[kThreads - 1];
    for (int i = begin; i < begin + per && i < m; ++i) {
        const int v = vals[i];
        vals[i] = run;
        run += v;
    }
    __syncthreads();
    return total;
}

} // namespace TileXREp

#endif // TILEXR_AMD_EP_BLOCK_SCAN_CUH
