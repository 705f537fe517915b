// Per-world bookkeeping of the plan-driven (MoonEP) stages (internal header).
#ifndef TILEXR_AMD_MOONEP_HOST_H
#define TILEXR_AMD_MOONEP_HOST_H

#include <cstdint>
#include <vector>

#include <hip/hip_runtime_api.h>

#include "ep_context.h"

namespace TileXRMoon {

// What one rank asked for, copied out of the caller's argument structures (which need not outlive the call).
struct StageCall {
    bool present = false;
    hipStream_t stream = nullptr;
    int64_t s = 0, k = 0, h = 0, nvS = 0;
    uint64_t flags = 0;
    const int32_t *dst = nullptr;
    int32_t *dupGroups = nullptr;
    int32_t *dupLoffs = nullptr;
    int32_t *dupCounts = nullptr;
    int32_t *status = nullptr;
    // dispatch: hiddenSh / weightsSk in, hiddenNvsh / weightsNvs out; combine: hiddenNvsh / weightsNvs in
    const void *hiddenSh = nullptr;
    const float *weightsSk = nullptr;
    void *hiddenNvsh = nullptr;
    float *weightsNvs = nullptr;
    // combine only
    const int32_t *dstLocal = nullptr;
    void *hiddenShOut = nullptr;
    float *weightsSkOut = nullptr;
};

struct RankEvents {
    hipEvent_t arrived = nullptr;   // the rank's stream has reached its call
};

struct WorldState {
    uint64_t epochCounter = 0;
    TileXREp::DeviceBuffer tables;
    std::vector<StageCall> dispatch;    // calls waiting for the rest of the world, by rank
    std::vector<StageCall> combine;
    std::vector<RankEvents> events;
    hipStream_t stream = nullptr;       // worlds of several ranks: the stream their exchanges run on (default priority)
    hipEvent_t done = nullptr;          // end of the last exchange
    bool doneArmed = false;
};

void ReleaseWorldState(WorldState *st);

} // namespace TileXRMoon

#endif // TILEXR_AMD_MOONEP_HOST_H
