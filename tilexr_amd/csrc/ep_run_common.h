// Helpers shared by the single-rank (api.cpp) and multi-rank (multi_rank.cpp) orchestration (internal header).
#ifndef TILEXR_AMD_EP_RUN_COMMON_H
#define TILEXR_AMD_EP_RUN_COMMON_H

#include <cstdio>
#include <limits>

#include <hip/hip_runtime_api.h>

#include "ep_context.h"
#include "ep_launch.h"
#include "tilexr_types.h"

namespace TileXREp {

inline int LaunchStatus(hipError_t err, const char *what)
{
    if (err == hipSuccess) {
        return TileXR::TILEXR_SUCCESS;
    }
    // reference: src/ep/host/ep_kernel_launch.cpp:153,177 reports launch failures on stderr and returns MKIRT
    std::fprintf(stderr, "tilexr-ep: launching %s failed: %s\n", what, hipGetErrorString(err));
    return TileXR::TILEXR_ERROR_MKIRT;
}

// Records the caller's timing events (if any) around one kernel launch.
template <typename Launch>
int Timed(EpComm *comm, int kernel, hipStream_t stream, const char *what, Launch launch)
{
    hipEvent_t start = comm->timing[kernel][0];
    hipEvent_t stop = comm->timing[kernel][1];
    DebugState &dbg = comm->debug;
    auto stamp = [&](int edge) {
        if (dbg.phaseStamps == nullptr || dbg.capacity <= 0) {
            return true;
        }
        uint64_t *record = dbg.phaseStamps + (dbg.next++ % dbg.capacity) * kDebugStampWords;
        return LaunchDebugStamp(record, static_cast<uint64_t>(dbg.magic), kernel, edge, stream) == hipSuccess;
    };
    if (!stamp(0)) {
        return TileXR::TILEXR_ERROR_MKIRT;
    }
    if (start != nullptr && hipEventRecord(start, stream) != hipSuccess) {
        return TileXR::TILEXR_ERROR_INTERNAL;
    }
    const int ret = LaunchStatus(launch(), what);
    if (ret == TileXR::TILEXR_SUCCESS && stop != nullptr && hipEventRecord(stop, stream) != hipSuccess) {
        return TileXR::TILEXR_ERROR_INTERNAL;
    }
    if (ret == TileXR::TILEXR_SUCCESS && !stamp(1)) {
        return TileXR::TILEXR_ERROR_MKIRT;
    }
    return ret;
}

// Shapes the kernels' 32-bit indexing and LDS tables can hold.
inline bool WithinKernelLimits(int64_t bs, int64_t h, int64_t topK, int64_t experts, int64_t rankSize = 1)
{
    const int64_t intMax = std::numeric_limits<int32_t>::max();
    return experts <= kMaxKeys && topK <= kMaxTopK && bs <= intMax / topK && h <= intMax / 2 &&
        bs * topK <= intMax / (4 * rankSize);
}

inline CountScratch CarveCountScratch(void *base, const CountScratchLayout &plan, bool expertHist)
{
    auto at = [base](int64_t off) { return reinterpret_cast<int32_t *>(static_cast<char *>(base) + off); };
    CountScratch s {};
    s.chunkShift = plan.chunkShift;
    s.ticket = static_cast<uint32_t *>(base);
    s.localRank = at(plan.localRankOff);
    s.chunkHist = at(plan.chunkHistOff);
    s.chunkExpHist = expertHist ? at(plan.chunkExpHistOff) : nullptr;
    s.keyOffset = at(plan.keyOffsetOff);
    s.keyKept = at(plan.keyKeptOff);
    s.expertTotal = at(plan.expertTotalOff);
    return s;
}

constexpr int64_t kDefaultWaitUs = 2 * 1000 * 1000;
constexpr int64_t kWallClockTicksPerUs = 100;      // wall_clock64() counts at 100 MHz on CDNA3/CDNA4

} // namespace TileXREp

#endif // TILEXR_AMD_EP_RUN_COMMON_H
