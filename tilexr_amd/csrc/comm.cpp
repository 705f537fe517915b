// Communicator calls for logical ranks that share one MI355X.
//
// Stands in for the part of libtile-comm that the EP host code calls (reference: src/comm/comm_wrap.cpp:173-182,
// src/comm/tilexr_comm.cpp:1235-1238).  Nothing here talks to another process or another device.
#include <algorithm>
#include <cstdlib>
#include <cstring>
#include <unordered_set>

#include <hip/hip_runtime_api.h>

#include "ep_context.h"
#include "ep_static_scratch.h"
#include "moonep_host.h"
#include "tilexr_api.h"
#include "tilexr_types.h"

namespace TileXREp {
namespace {

std::mutex gRegistryMutex;
std::unordered_set<EpComm *> gComms;
std::vector<EpWorld *> gOpenWorlds;      // worlds that still miss ranks

void ReleaseWorld(EpWorld *world)
{
    if (world->flagArea != nullptr) {
        (void)hipFree(world->flagArea);
    }
    for (DeviceBuffer *b : {&world->stageRows, &world->stageAux, &world->stageCounts, &world->combineSlots,
             &world->combineMeta}) {
        b->Release();
    }
    for (auto *list : {&world->dispatchEvents, &world->combineEvents}) {
        for (RankEvents &e : *list) {
            if (e.sent != nullptr) {
                (void)hipEventDestroy(e.sent);
            }
            if (e.drained != nullptr) {
                (void)hipEventDestroy(e.drained);
            }
        }
    }
    TileXRMoon::ReleaseWorldState(world->moon);
    delete world;
}

EpWorld *CreateWorld(int rankSize)
{
    EpWorld *world = new EpWorld();
    world->rankSize = rankSize;
    world->comms.assign(static_cast<size_t>(rankSize), nullptr);
    world->pendingDispatch.resize(static_cast<size_t>(rankSize));
    world->pendingCombine.resize(static_cast<size_t>(rankSize));
    world->dispatchEvents.resize(static_cast<size_t>(rankSize));
    world->combineEvents.resize(static_cast<size_t>(rankSize));
    int device = -1;
    if (hipGetDevice(&device) == hipSuccess) {
        world->device = device;
        void *area = nullptr;
        const size_t bytes = static_cast<size_t>(rankSize) * kFlagAreaBytesPerRank;
        if (hipMalloc(&area, bytes) == hipSuccess && hipMemset(area, 0, bytes) == hipSuccess &&
            hipStreamSynchronize(nullptr) == hipSuccess) {
            world->flagArea = static_cast<uint8_t *>(area);
            world->deviceReady = true;
            // the per-GPU scratch of the entry point that allocates nothing: its address on this device
            world->staticScratchReady = ResolveStaticScratch(device) == hipSuccess;
            int cus = 0;
            if (hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, device) == hipSuccess) {
                world->numComputeUnits = cus;
            }
        } else if (area != nullptr) {
            (void)hipFree(area);
        }
    }
    (void)hipGetLastError();     // a box without a GPU leaves an error behind; it must not leak into later calls
    return world;
}

} // namespace

bool DeviceBuffer::Reserve(size_t want, bool zero)
{
    if (want <= bytes && ptr != nullptr) {
        return true;
    }
    Release();
    const size_t rounded = (want + 4095) / 4096 * 4096;
    void *p = nullptr;
    if (hipMalloc(&p, rounded) != hipSuccess) {
        (void)hipGetLastError();
        return false;
    }
    // The fill runs on the null stream, which a caller's non-blocking stream does not wait for: the kernels that
    // are about to use the buffer on that stream must not be able to overtake it.
    if (zero && (hipMemset(p, 0, rounded) != hipSuccess || hipStreamSynchronize(nullptr) != hipSuccess)) {
        (void)hipFree(p);
        return false;
    }
    ptr = p;
    bytes = rounded;
    return true;
}

void DeviceBuffer::Release()
{
    if (ptr != nullptr) {
        (void)hipFree(ptr);
    }
    ptr = nullptr;
    bytes = 0;
}

uint64_t NextFlagEpoch()
{
    static std::atomic<uint32_t> counter {0};
    uint32_t v = 0;
    do {
        v = counter.fetch_add(1, std::memory_order_relaxed) + 1;
    } while (v == 0);
    return v;
}

EpComm *LookupComm(TileXRCommPtr comm)
{
    std::lock_guard<std::mutex> lock(gRegistryMutex);
    EpComm *c = static_cast<EpComm *>(comm);
    return gComms.count(c) != 0 ? c : nullptr;
}

} // namespace TileXREp

using TileXREp::EpComm;
using TileXREp::EpWorld;

extern "C" {

int TileXRCommInitRankLocal(int rankSize, int rank, TileXRCommPtr *comm)
{
    if (comm == nullptr || rankSize <= 0 || rankSize > TileXR::TILEXR_MAX_RANK_SIZE || rank < 0 || rank >= rankSize) {
        return TileXR::TILEXR_ERROR_PARA_CHECK_FAIL;
    }
    std::lock_guard<std::mutex> lock(TileXREp::gRegistryMutex);
    EpWorld *world = nullptr;
    for (EpWorld *w : TileXREp::gOpenWorlds) {
        if (w->rankSize == rankSize && w->comms[static_cast<size_t>(rank)] == nullptr) {
            world = w;
            break;
        }
    }
    if (world == nullptr) {
        world = TileXREp::CreateWorld(rankSize);
        TileXREp::gOpenWorlds.push_back(world);
    } else if (world->deviceReady) {
        int device = -1;
        if (hipGetDevice(&device) != hipSuccess || device != world->device) {
            return TileXR::TILEXR_ERROR_PARA_CHECK_FAIL;   // all logical ranks of a world share one device
        }
    }

    EpComm *c = new EpComm();
    c->world = world;
    c->rank = rank;
    const char *routing = std::getenv("TILEXR_EP_ROUTING");
    if (routing != nullptr && std::strcmp(routing, "legacy") == 0) {
        c->routing = EpComm::Routing::kLegacy;
    } else if (routing != nullptr && std::strcmp(routing, "one-launch") == 0) {
        c->routing = EpComm::Routing::kOneLaunch;
    }
    c->host.rank = rank;
    c->host.localRank = rank;
    c->host.rankSize = rankSize;
    c->host.localRankSize = rankSize;
    c->host.extraFlag = TileXR::ExtraFlag::MEMORY_ONLY;
    c->host.peerMemBytes = static_cast<uint64_t>(TileXREp::kFlagAreaBytesPerRank);
    for (int r = 0; r < rankSize; ++r) {
        c->host.peerMems[r] = world->flagArea == nullptr ? nullptr :
            world->flagArea + static_cast<int64_t>(r) * TileXREp::kFlagAreaBytesPerRank;
    }
    world->comms[static_cast<size_t>(rank)] = c;
    ++world->live;
    if (std::none_of(world->comms.begin(), world->comms.end(), [](EpComm *p) { return p == nullptr; })) {
        auto &open = TileXREp::gOpenWorlds;
        open.erase(std::remove(open.begin(), open.end(), world), open.end());
    }
    TileXREp::gComms.insert(c);
    *comm = c;
    return TileXR::TILEXR_SUCCESS;
}

int TileXRCommDestroy(TileXRCommPtr comm)
{
    std::lock_guard<std::mutex> lock(TileXREp::gRegistryMutex);
    EpComm *c = static_cast<EpComm *>(comm);
    if (TileXREp::gComms.erase(c) == 0) {
        return TileXR::TILEXR_ERROR_PARA_CHECK_FAIL;
    }
    EpWorld *world = c->world;
    if (world->deviceReady) {
        (void)hipDeviceSynchronize();       // nothing of this communicator may still be running
    }
    c->dispatchScratch.Release();
    c->combineScratch.Release();
    c->claimWord.Release();
    c->drainScratch.Release();
    c->tileCounters.Release();
    if (c->dev != nullptr) {
        (void)hipFree(c->dev);
    }
    world->comms[static_cast<size_t>(c->rank)] = nullptr;
    c->tag = 0;
    delete c;
    if (--world->live == 0) {
        auto &open = TileXREp::gOpenWorlds;
        open.erase(std::remove(open.begin(), open.end(), world), open.end());
        TileXREp::ReleaseWorld(world);
    }
    return TileXR::TILEXR_SUCCESS;
}

int TileXRGetCommArgsHost(TileXRCommPtr comm, TileXR::CommArgs *&commArgsPtr)
{
    commArgsPtr = nullptr;
    EpComm *c = TileXREp::LookupComm(comm);
    if (c == nullptr) {
        return TileXR::TILEXR_ERROR_NOT_INITIALIZED;
    }
    commArgsPtr = &c->host;
    return TileXR::TILEXR_SUCCESS;
}

int TileXRGetCommArgsDev(TileXRCommPtr comm, GM_ADDR &commArgsPtr)
{
    commArgsPtr = nullptr;
    EpComm *c = TileXREp::LookupComm(comm);
    if (c == nullptr || !c->world->deviceReady) {
        return TileXR::TILEXR_ERROR_NOT_INITIALIZED;
    }
    std::lock_guard<std::mutex> lock(c->mu);
    if (c->dev == nullptr) {
        void *p = nullptr;
        if (hipMalloc(&p, sizeof(TileXR::CommArgs)) != hipSuccess ||
            hipMemcpy(p, &c->host, sizeof(TileXR::CommArgs), hipMemcpyHostToDevice) != hipSuccess) {
            if (p != nullptr) {
                (void)hipFree(p);
            }
            return TileXR::TILEXR_ERROR_NOT_INITIALIZED;
        }
        c->dev = static_cast<GM_ADDR>(p);
    }
    commArgsPtr = c->dev;
    return TileXR::TILEXR_SUCCESS;
}

int TileXRCommNextMagic(TileXRCommPtr comm, int64_t *magic)
{
    EpComm *c = TileXREp::LookupComm(comm);
    if (c == nullptr || magic == nullptr) {
        return TileXR::TILEXR_ERROR_PARA_CHECK_FAIL;
    }
    *magic = c->nextMagic.fetch_add(1);
    return TileXR::TILEXR_SUCCESS;
}

}
