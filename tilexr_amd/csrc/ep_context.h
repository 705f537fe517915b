// Communicator state for logical ranks that share one MI355X (internal header).
//
// The reference keeps per-rank peer windows mapped over IPC and bootstraps ranks over sockets
// (src/comm/tilexr_comm.cpp); on one device a "world" is simply the set of communicators created with the same
// rankSize in one process.  A world owns
//   * a small flag area per rank (what CommArgs::peerMems[] points at),
//   * for rankSize > 1, the staging buffers rows pass through between the send half of a call (issued by the source
//     rank) and the drain half (issued for every rank once all ranks have sent), plus the bookkeeping of which ranks
//     have already called.
// A communicator owns its epoch counter and the scratch of the count / place / invert kernels.
#ifndef TILEXR_AMD_EP_CONTEXT_H
#define TILEXR_AMD_EP_CONTEXT_H

#include <atomic>
#include <cstddef>
#include <cstdint>
#include <mutex>
#include <vector>

#include <hip/hip_runtime_api.h>

#include "comm_args.h"
#include "ep_host.h"

namespace TileXREp {

constexpr int64_t kFlagAreaBytesPerRank = 64 * 1024;
constexpr uint32_t kCommTag = 0x54584550u;   // "TXEP"

// Grow-only device buffer.  Growing frees the old block (which synchronises the device) and allocates a new one.
struct DeviceBuffer {
    void *ptr = nullptr;
    size_t bytes = 0;
    bool Reserve(size_t want, bool zero);
    void Release();
};

struct PendingDispatch {
    bool present = false;
    EpDispatchParams params {};
    bool memoryRoute = false;
    int64_t magic = 0;
    hipEvent_t sent = nullptr;
};

struct PendingCombine {
    bool present = false;
    EpCombineParams params {};
    bool memoryRoute = false;
    int64_t magic = 0;
    hipEvent_t sent = nullptr;
};

struct EpComm;

struct EpWorld {
    int rankSize = 0;
    int device = -1;
    int live = 0;
    bool deviceReady = false;
    int numComputeUnits = 0;
    std::vector<EpComm *> comms;
    uint8_t *flagArea = nullptr;
    std::mutex mu;
    // multi-rank exchange (rankSize > 1)
    std::vector<PendingDispatch> pendingDispatch;
    std::vector<PendingCombine> pendingCombine;
    std::vector<DeviceBuffer> stageRows;      // per source rank: rows grouped by key
    std::vector<DeviceBuffer> stageAux;       // per source rank: assist tuples + per-row scales
    std::vector<DeviceBuffer> combineSlots;   // per source rank: [bs, topK] rows returned by the expert ranks
    std::vector<DeviceBuffer> combineMeta;    // per source rank: [bs, topK] tagged origin of each slot
};

struct EpComm {
    uint32_t tag = kCommTag;
    EpWorld *world = nullptr;
    int rank = 0;
    TileXR::CommArgs host {};
    GM_ADDR dev = nullptr;
    std::atomic<int64_t> nextMagic {1};
    DeviceBuffer dispatchScratch;
    DeviceBuffer combineScratch;
    hipEvent_t timing[5][2] = {};     // optional (start, stop) pairs around each kernel, see tilexr_ep.h
    std::mutex mu;
};

enum KernelId : int { kKernelCount = 0, kKernelPlace = 1, kKernelScatter = 2, kKernelInvert = 3, kKernelReduce = 4 };

// Returns the communicator when `comm` was created by TileXRCommInitRankLocal and not destroyed, else nullptr.
EpComm *LookupComm(TileXRCommPtr comm);

} // namespace TileXREp

#endif // TILEXR_AMD_EP_CONTEXT_H
