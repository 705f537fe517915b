// Workgroup-wide exclusive scan in LDS (256 threads), shared by the routing and exchange kernels.
#ifndef TILEXR_AMD_EP_BLOCK_SCAN_HIP_H
#define TILEXR_AMD_EP_BLOCK_SCAN_HIP_H

#include <hip/hip_runtime.h>

#include "ep_kernel_common.hip.h"

namespace TileXREp {

// Exclusive scan of vals[0..m) in place (LDS), m <= 2048, by all 256 threads.  part[] is 256 ints of LDS.
// Returns the total.  Orders LDS traffic only (see LdsBarrier).
__device__ inline int BlockExclusiveScan(int *vals, int m, int *part)
{
    const int tid = threadIdx.x;
    const int lane = tid & (kWave - 1);
    const int wave = tid / kWave;
    const int per = (m + kThreads - 1) / kThreads;
    const int begin = tid * per;
    int local = 0;
    for (int i = begin; i < begin + per && i < m; ++i) {
        local += vals[i];
    }
    // inclusive scan of the per-thread sums inside each wave (shuffles), then across the four waves through LDS
    int incl = local;
#pragma unroll
    for (int off = 1; off < kWave; off <<= 1) {
        const int up = __shfl_up(incl, off);
        incl += lane >= off ? up : 0;
    }
    if (lane == kWave - 1) {
        part[wave] = incl;
    }
    LdsBarrier();
    int waveBase = 0;
    int total = 0;
#pragma unroll
    for (int w = 0; w < kWavesPerBlock; ++w) {
        const int v = part[w];
        waveBase += w < wave ? v : 0;
        total += v;
    }
    int run = waveBase + incl - local;
    for (int i = begin; i < begin + per && i < m; ++i) {
        const int v = vals[i];
        vals[i] = run;
        run += v;
    }
    LdsBarrier();
    return total;
}

} // namespace TileXREp

#endif // TILEXR_AMD_EP_BLOCK_SCAN_HIP_H
