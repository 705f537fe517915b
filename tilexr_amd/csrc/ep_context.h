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
#include "ep_debug.h"
#include "ep_host.h"

namespace TileXRMoon {
struct WorldState;     // per-world state of the plan-driven stages (moonep_host.h)
}

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

// What all ranks of one exchange must agree on.
struct ExchangeShape {
    int64_t bs = 0;
    int64_t h = 0;
    int64_t topK = 0;
    int64_t experts = 0;
    int64_t quantMode = 0;
    int64_t sharedNum = 0;       // shared experts every active token is also sent to
    int64_t sharedRanks = 0;     // ranks [0, sharedRanks) host them
    int64_t tp = 1;              // MVP route: lanes per tensor-parallel group
    int dtype = 0;
    int outDtype = 0;
    bool memoryRoute = false;
    bool operator==(const ExchangeShape &o) const
    {
        return bs == o.bs && h == o.h && topK == o.topK && experts == o.experts && quantMode == o.quantMode &&
            sharedNum == o.sharedNum && sharedRanks == o.sharedRanks && tp == o.tp && dtype == o.dtype && outDtype == o.outDtype &&
            memoryRoute == o.memoryRoute;
    }
};

struct PendingDispatch {
    bool present = false;
    EpDispatchParams params {};
};

struct PendingCombine {
    bool present = false;
    EpCombineParams params {};
};

// Per-rank events of the two-half exchange; created on first use, `armed` once recorded.
struct RankEvents {
    hipEvent_t sent = nullptr;       // this rank's send half is enqueued
    hipEvent_t drained = nullptr;    // this rank's drain half is enqueued (staging may be reused after it)
    bool drainedArmed = false;
};

struct EpComm;

struct EpWorld {
    int rankSize = 0;
    int device = -1;
    int live = 0;
    bool deviceReady = false;
    bool staticScratchReady = false;   // the static per-GPU scratch has an address on `device`
    int numComputeUnits = 0;
    std::vector<EpComm *> comms;
    uint8_t *flagArea = nullptr;
    std::mutex mu;
    // multi-rank exchange (rankSize > 1)
    ExchangeShape dispatchShape {};
    ExchangeShape combineShape {};
    std::vector<PendingDispatch> pendingDispatch;
    std::vector<PendingCombine> pendingCombine;
    std::vector<RankEvents> dispatchEvents;
    std::vector<RankEvents> combineEvents;
    uint64_t combineEpoch = 0;
    DeviceBuffer stageRows;       // [R] payload rows grouped by key
    DeviceBuffer stageAux;        // [R] assist tuples + per-row scales
    DeviceBuffer stageCounts;     // [R] keyOffset + expertTotal
    DeviceBuffer combineSlots;    // [R] [bs, topK] rows returned by the expert ranks
    DeviceBuffer combineMeta;     // [R] tagged slot table + order keys
    TileXRMoon::WorldState *moon = nullptr;   // created by the first plan-driven call of the world
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
    DeviceBuffer claimWord;           // token claims of a combine that waits on readiness flags
    DeviceBuffer drainScratch;
    DeviceBuffer tileCounters;        // rows landed per readiness tile; all zero whenever no dispatch is in flight
    // The last dispatch of this communicator that published readiness flags: a combine on the same stream that waits for
    // the same words and epoch finds every tile published (stream order), so it needs no room left for a producer.
    const void *lastFlagWords = nullptr;
    uint64_t lastFlagEpoch = 0;
    hipStream_t lastFlagStream = nullptr;
    // TILEXR_EP_ROUTING when the communicator was created (a switch for tests): unset = the library picks the routing
    // kernels by the size of the call; "legacy" = count (+ place) launches everywhere; "one-launch" = the one-launch
    // routing wherever it can take the call, also where the other is measured to be faster
    enum class Routing { kAuto, kLegacy, kOneLaunch };
    Routing routing = Routing::kAuto;
    DebugState debug;                 // TileXREpSetDebugOptions
    hipEvent_t timing[5][2] = {};     // optional (start, stop) pairs around each kernel, see tilexr_ep.h
    const char *lastKernel[5] = {};   // name of the kernel template last launched for each kernel id
    std::mutex mu;
};

enum KernelId : int { kKernelCount = 0, kKernelPlace = 1, kKernelScatter = 2, kKernelInvert = 3, kKernelReduce = 4 };

// Next tag for tile readiness words: one counter for the whole process, 32 bits wide, never 0 (a zero-filled flag
// array must read as "not ready" for every epoch).
uint64_t NextFlagEpoch();

// Returns the communicator when `comm` was created by TileXRCommInitRankLocal and not destroyed, else nullptr.
EpComm *LookupComm(TileXRCommPtr comm);

} // namespace TileXREp

#endif // TILEXR_AMD_EP_CONTEXT_H
