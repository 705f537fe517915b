// Debug aids of the dispatch / combine path (internal header, see ep_debug.hip).
#ifndef TILEXR_AMD_EP_DEBUG_H
#define TILEXR_AMD_EP_DEBUG_H

#include <cstdint>

#include <hip/hip_runtime_api.h>

namespace TileXREp {

constexpr uint32_t kDebugPoisonWord = 0x7f7f7f7fu;
constexpr int kDebugStampWords = 4;     // {call magic, kernel id, edge (0 before / 1 after), device clock}

struct DebugState {
    uint64_t *phaseStamps = nullptr;    // caller-owned device ring of capacity records
    int64_t capacity = 0;
    int64_t next = 0;                   // records written so far (the ring index is next % capacity)
    bool poison = false;
    int64_t magic = 0;                  // magic of the call in progress
};

hipError_t LaunchDebugStamp(uint64_t *record, uint64_t magic, int kernelId, int edge, hipStream_t stream);
hipError_t LaunchDebugPoison(void *base, int64_t bytes, hipStream_t stream);

} // namespace TileXREp

#endif // TILEXR_AMD_EP_DEBUG_H
