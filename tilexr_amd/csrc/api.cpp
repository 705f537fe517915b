// Entry points of libtilexr-ep and the orchestration of one call: validate -> draw a magic -> enqueue kernels.
//
// The order of the host-side steps follows the reference (src/ep/host/tilexr_ep_dispatch.cpp:8-22,
// tilexr_ep_memory_dispatch.cpp:9-23, tilexr_ep_memory_combine.cpp:9-21, ep_kernel_launch.cpp:252-416):
// basic argument check, communicator lookup, configuration check, magic, launch.  Success means "enqueued on the
// caller's stream"; nothing here waits for the device.
#include <algorithm>
#include <cstdio>
#include <limits>

#include <hip/hip_runtime_api.h>

#include "ep_context.h"
#include "ep_host.h"
#include "ep_launch.h"
#include "ep_run_common.h"
#include "ep_static_scratch.h"
#include "tilexr_ep.h"

namespace TileXREp {

int RunDispatchMulti(EpComm *comm, const EpDispatchParams &p, bool memoryRoute, int64_t magic);
int RunCombineMulti(EpComm *comm, const EpCombineParams &p, bool memoryRoute, int64_t magic);

namespace {

constexpr int kOk = TileXR::TILEXR_SUCCESS;
// ---------------------------------------------------------------------------------------------------------
// one rank per device: rows go straight from x to expandXOut
// ---------------------------------------------------------------------------------------------------------
int RunDispatchSingle(EpComm *comm, const EpDispatchParams &p, bool memoryRoute, int64_t magic, uint64_t flagEpoch)
{
    if (!WithinKernelLimits(p.bs, p.h, p.topK, p.moeExpertNum)) {
        return TileXR::TILEXR_ERROR_NOT_SUPPORT;
    }
    hipStream_t stream = static_cast<hipStream_t>(p.stream);
    const int64_t n = p.bs * p.topK;
    const int64_t experts = p.moeExpertNum;
    const int64_t numKeys = memoryRoute ? experts : 1;
    const int64_t keyDiv = memoryRoute ? 1 : experts;
    const bool expertHist = !memoryRoute;

    std::lock_guard<std::mutex> lock(comm->mu);
    comm->debug.magic = magic;
    if (comm->debug.poison) {
        // every row this dispatch may write, its tuple and its scales: a row that is counted but never written shows
        const int64_t rows = p.expertCapacity > 0 ? std::min<int64_t>(n, experts * p.expertCapacity) : n;
        const int64_t rowBytes = p.quantMode == TILEXR_EP_QUANT_NONE ? p.h * 2 : p.h;
        int64_t scaleBytes = 0;
        if (p.quantMode == TILEXR_EP_QUANT_TOKEN_INT8) {
            scaleBytes = 4;
        } else if (p.quantMode == TILEXR_EP_QUANT_MXFP8) {
            scaleBytes = ((p.h + 31) / 32 + 1) / 2 * 2;
        } else if (p.quantMode == TILEXR_EP_QUANT_FP8_BLOCK128) {
            scaleBytes = (p.h + 127) / 128 * 4;
        }
        if (LaunchDebugPoison(p.expandXOut, rows * rowBytes, stream) != hipSuccess ||
            LaunchDebugPoison(p.assistInfoForCombineOut, rows * 16, stream) != hipSuccess ||
            LaunchDebugPoison(p.dynamicScalesOut, rows * scaleBytes, stream) != hipSuccess) {
            return TileXR::TILEXR_ERROR_MKIRT;
        }
    }
    if (memoryRoute && p.quantMode == TILEXR_EP_QUANT_NONE && p.xActiveMask == nullptr && p.metaReadyEvent == nullptr) {
        // decode-sized calls: one launch instead of count + scatter (a consumer that is to run beside the dispatch needs
        // the row map ahead of the rows, which takes the separate launches)
        SmallDispatchLaunch small {};
        small.x = p.x;
        small.ids = p.expertIds;
        small.bs = p.bs;
        small.h = p.h;
        small.topK = p.topK;
        small.numExperts = experts;
        small.capacity = p.expertCapacity;
        small.srcRank = comm->rank;
        small.expertIdBias = static_cast<int32_t>(p.sharedExpertNum);
        small.out = p.expandXOut;
        small.assist = p.assistInfoForCombineOut;
        small.rowOf = p.rowIndexMapOut;
        small.sendCountsOut = p.epRecvCountsOut;
        small.expertTokenNumsOut = p.expertTokenNumsOut;
        small.tokenNumsType = static_cast<int>(p.expertTokenNumsType);
        small.stream = stream;
        if (SmallDispatchFits(small)) {
            if (p.tileFlagsOut != nullptr) {
                // a tile never holds more rows than the dispatch can produce: larger values name the same single tile
                small.tileRows = std::min<int64_t>(p.tileRows, std::max<int64_t>(n, 1));
                if (!comm->tileCounters.Reserve(static_cast<size_t>(TileCounterWords(n, small.tileRows)) * sizeof(uint32_t), true)) {
                    return TileXR::TILEXR_ERROR_INTERNAL;
                }
                small.tileFlags = p.tileFlagsOut;
                small.tileCounters = static_cast<uint32_t *>(comm->tileCounters.ptr);
                small.epoch = flagEpoch;
            }
            small.kernelNameOut = &comm->lastKernel[kKernelScatter];
            const int ret = Timed(comm, kKernelScatter, stream, "small dispatch", [&] { return LaunchSmallDispatch(small); });
            if (ret == kOk && p.tileFlagsOut != nullptr) {
                comm->lastFlagWords = p.tileFlagsOut;
                comm->lastFlagEpoch = flagEpoch;
                comm->lastFlagStream = stream;
            }
            return ret;
        }
    }
    const CountScratchLayout plan = PlanCountScratch(n, numKeys, experts, expertHist);
    int maskMode = kMaskNone;
    if (p.xActiveMask != nullptr && !memoryRoute) {
        maskMode = kMaskPerToken;              // reference: tilexr_ep_dispatch_helpers.h:3-21
    } else if (p.xActiveMask != nullptr) {
        maskMode = p.activeMaskType == TILEXR_EP_ACTIVE_MASK_EXPERT ? kMaskPerRoute : kMaskTokenPrefix;
    }
    // One launch resolves every route's row where every expert's workgroup can afford to read the whole id table
    // (ep_rows.hip); otherwise count (ticket, last workgroup scans) and place, the latter folded into the scatter
    // unless something needs the rows ahead of it.
    const bool rowsAhead = p.tileFlagsOut != nullptr || p.metaReadyEvent != nullptr;
    // the scatter kernel that copies per route wants the token rows close by: the routing launch reads them ahead
    const bool warm = ScatterCopiesPerRoute(p.x, p.expandXOut, p.bs, p.h, p.topK, static_cast<int>(p.quantMode));
    const bool oneLaunch = memoryRoute && comm->routing != EpComm::Routing::kLegacy &&
        RouteRowsFits(p.expertIds, n, numKeys, maskMode, p.expertCapacity) &&
        (comm->routing == EpComm::Routing::kOneLaunch || RouteRowsPays(n, numKeys, rowsAhead, warm));
    void *scratchBase = nullptr;
    if (p.noAlloc) {
        // this call may not allocate: the per-GPU static array or nothing
        void *staticScratch = comm->world->staticScratchReady ? StaticScratchOnDevice(comm->world->device) : nullptr;
        if (staticScratch == nullptr) {
            return TileXR::TILEXR_ERROR_NOT_INITIALIZED;
        }
        if (plan.totalBytes > static_cast<int64_t>(kStaticScratchBytes)) {
            return TileXR::TILEXR_ERROR_NOT_SUPPORT;     // DispatchMemory has said why
        }
        scratchBase = staticScratch;
        // the array keeps what the previous call left: the count kernel's ticket has to start at zero (the one-launch
        // routing keeps nothing in scratch but its outputs)
        if (!oneLaunch && ClearScratchWord(scratchBase, stream) != hipSuccess) {
            return TileXR::TILEXR_ERROR_MKIRT;
        }
    } else {
        if (!comm->dispatchScratch.Reserve(static_cast<size_t>(plan.totalBytes), true)) {
            return TileXR::TILEXR_ERROR_INTERNAL;
        }
        scratchBase = comm->dispatchScratch.ptr;
    }
    const CountScratch scratch = CarveCountScratch(scratchBase, plan, expertHist);
    int32_t *rowOf = p.rowIndexMapOut != nullptr ? p.rowIndexMapOut :
        reinterpret_cast<int32_t *>(static_cast<char *>(scratchBase) + plan.rowOfOff);
    int ret = kOk;
    RoutePlaceLaunch place {};
    bool separatePlace = false;
    if (oneLaunch) {
        RouteRowsLaunch rows {};
        rows.ids = p.expertIds;
        rows.bs = p.bs;
        rows.topK = p.topK;
        rows.numKeys = numKeys;
        rows.srcRank = comm->rank;
        rows.expertIdBias = static_cast<int32_t>(p.sharedExpertNum);
        rows.rowOf = rowOf;
        rows.assist = p.assistInfoForCombineOut;
        rows.totalRowsOut = scratch.keyOffset + numKeys;
        rows.sendCountsOut = p.epRecvCountsOut;
        rows.expertTokenNumsOut = p.expertTokenNumsOut;
        rows.tokenNumsType = static_cast<int>(p.expertTokenNumsType);
        rows.warmRows = warm ? p.x : nullptr;
        rows.warmBytes = p.bs * p.h * 2;
        rows.stream = stream;
        comm->lastKernel[kKernelCount] = "ep_route_rows_kernel";
        ret = Timed(comm, kKernelCount, stream, "route rows", [&] { return LaunchRouteRows(rows); });
        if (ret != kOk) {
            return ret;
        }
        if (p.metaReadyEvent != nullptr &&
            hipEventRecord(static_cast<hipEvent_t>(p.metaReadyEvent), stream) != hipSuccess) {
            return TileXR::TILEXR_ERROR_INTERNAL;
        }
    } else {
        RouteCountLaunch count {};
        count.ids = p.expertIds;
        count.mask = reinterpret_cast<const uint8_t *>(p.xActiveMask);
        count.maskMode = maskMode;
        count.bs = p.bs;
        count.topK = p.topK;
        count.numExperts = experts;
        count.keyDiv = keyDiv;
        count.numKeys = numKeys;
        count.capacity = p.expertCapacity;
        count.scratch = scratch;
        count.sendCountsOut = memoryRoute ? p.epRecvCountsOut : nullptr;
        count.recvCountOut = memoryRoute ? nullptr : p.epRecvCountsOut;
        count.expertTokenNumsOut = p.expertTokenNumsOut;
        count.tokenNumsType = static_cast<int>(p.expertTokenNumsType);
        count.stream = stream;
        count.warmRows = warm ? p.x : nullptr;
        count.warmBytes = p.bs * p.h * 2;
        comm->lastKernel[kKernelCount] = "ep_route_count_kernel";
        ret = Timed(comm, kKernelCount, stream, "route count", [&] { return LaunchRouteCount(count); });
        if (ret != kOk) {
            return ret;
        }
        if (!memoryRoute && p.tpRecvCountsOut != nullptr) {
            // reference: tilexr_ep_combine_helpers.h:93-95 mirrors the per-source count into tpRecvCounts
            if (hipMemcpyAsync(p.tpRecvCountsOut, p.epRecvCountsOut, sizeof(int32_t), hipMemcpyDeviceToDevice, stream) !=
                hipSuccess) {
                return TileXR::TILEXR_ERROR_INTERNAL;
            }
        }

        place.ids = p.expertIds;
        place.bs = p.bs;
        place.topK = p.topK;
        place.keyDiv = keyDiv;
        place.numKeys = numKeys;
        place.capacity = p.expertCapacity;
        place.scratch = scratch;
        place.srcRank = comm->rank;
        place.expertIdBias = static_cast<int32_t>(p.sharedExpertNum);
        place.rowOf = rowOf;
        place.assist = p.assistInfoForCombineOut;
        place.stream = stream;
        // The scatter kernel can resolve the rows of its own tokens.  A separate launch is needed when the row map and
        // the assist tuples have to be complete before the first row lands (metaReadyEvent), and it pays when readiness
        // flags are published: a workgroup that publishes stays until its stores have landed, and resolving the row
        // first (three dependent loads) makes that stay longer (measured on 4096 x 7168 x top-8: scatter 105 us fused,
        // 87 + 4 us apart).
        separatePlace = rowsAhead;
        if (separatePlace) {
            ret = Timed(comm, kKernelPlace, stream, "route place", [&] { return LaunchRoutePlace(place); });
            if (ret != kOk) {
                return ret;
            }
            if (p.metaReadyEvent != nullptr &&
                hipEventRecord(static_cast<hipEvent_t>(p.metaReadyEvent), stream) != hipSuccess) {
                return TileXR::TILEXR_ERROR_INTERNAL;
            }
        } else {
            place.rowOf = p.rowIndexMapOut;      // only written when the caller asked for the map
        }
    }

    ScatterLaunch scatter {};
    scatter.x = p.x;
    scatter.rowOf = rowOf;
    scatter.fusedPlace = (oneLaunch || separatePlace) ? nullptr : &place;
    scatter.bs = p.bs;
    scatter.h = p.h;
    scatter.topK = p.topK;
    scatter.quantMode = static_cast<int>(p.quantMode);
    // the MVP route's quantisers decode the input as fp16 whatever the caller's tensor holds
    // (reference: tilexr_ep_dispatch_helpers.h:121,167)
    scatter.inputBf16 = memoryRoute && p.dtype == TileXR::TILEXR_DATA_TYPE_BFP16;
    scatter.fp8E5m2 = p.expandXOutDtype == TileXR::TILEXR_DATA_TYPE_FP8E5M2;
    scatter.staticScale = static_cast<const float *>(p.scales);
    scatter.out = p.expandXOut;
    scatter.scalesOut = p.dynamicScalesOut;
    scatter.tileFlags = p.tileFlagsOut;
    scatter.consumerBeside = p.metaReadyEvent != nullptr;
    // a tile never holds more rows than the dispatch can produce: larger values name the same single tile
    scatter.tileRows = std::min<int64_t>(p.tileRows, std::max<int64_t>(n, 1));
    scatter.epoch = flagEpoch;
    scatter.totalRowsPtr = scratch.keyOffset + numKeys;
    if (p.tileFlagsOut != nullptr) {
        if (!comm->tileCounters.Reserve(static_cast<size_t>(TileCounterWords(n, scatter.tileRows)) * sizeof(uint32_t), true)) {
            return TileXR::TILEXR_ERROR_INTERNAL;
        }
        scatter.tileCounters = static_cast<uint32_t *>(comm->tileCounters.ptr);
    }
    scatter.kernelNameOut = &comm->lastKernel[kKernelScatter];
    scatter.stream = stream;
    ret = Timed(comm, kKernelScatter, stream, "scatter", [&] { return LaunchScatter(scatter); });
    if (ret == kOk && p.tileFlagsOut != nullptr) {
        comm->lastFlagWords = p.tileFlagsOut;
        comm->lastFlagEpoch = flagEpoch;
        comm->lastFlagStream = stream;
    }
    return ret;
}

int RunCombineSingle(EpComm *comm, const EpCombineParams &p, bool memoryRoute, int64_t magic)
{
    if (!WithinKernelLimits(p.bs, p.h, p.topK, p.moeExpertNum)) {
        return TileXR::TILEXR_ERROR_NOT_SUPPORT;
    }
    hipStream_t stream = static_cast<hipStream_t>(p.stream);
    const int64_t n = p.bs * p.topK;
    std::lock_guard<std::mutex> lock(comm->mu);
    comm->debug.magic = magic;

    const uint64_t epoch = static_cast<uint64_t>(magic) & 0xffffffffull;
    InvertLaunch inv {};
    if (p.rowIndexMap == nullptr) {
        inv.assist = p.assistInfoForCombine;
        inv.counts = p.epRecvCounts;
        inv.numCounts = memoryRoute ? p.moeExpertNum : 1;
        inv.countsArePrefix = memoryRoute;
        inv.maxRows = n;
        inv.maxCountPerEntry = n;
        inv.rank = comm->rank;
        inv.bs = p.bs;
        inv.topK = p.topK;
        inv.epoch = epoch;
        inv.stream = stream;
    }

    ReduceLaunch red {};
    red.expertOut = p.expertOut;
    red.rowBytes = p.expertOutQuantMode == 0 ? p.h * 2 : p.h;
    red.epoch = epoch;
    red.rowIndexMap = p.rowIndexMap;
    red.assistTable = p.rowIndexMap == nullptr ? &inv : nullptr;
    red.expertScales = memoryRoute ? p.expertScales : nullptr;
    red.tokenMask = memoryRoute ? reinterpret_cast<const uint8_t *>(p.xActiveMask) : nullptr;
    red.sharedExpertX = memoryRoute ? p.sharedExpertX : nullptr;
    red.reduceKind = memoryRoute ? kReduceFp32 : kReducePerAdd;
    red.commQuant = memoryRoute ? static_cast<int>(p.quantMode) : 0;
    red.inQuant = static_cast<int>(p.expertOutQuantMode);
    red.inScales = static_cast<const float *>(p.expertOutScales);
    red.bf16 = p.dtype == TileXR::TILEXR_DATA_TYPE_BFP16;
    red.bs = p.bs;
    red.h = p.h;
    red.topK = p.topK;
    red.maxRows = n;
    red.y = p.yOut;
    red.tileFlags = p.tileFlags;
    red.tileRows = std::min<int64_t>(p.tileRows, std::max<int64_t>(n, 1));
    red.flagEpoch = static_cast<uint64_t>(p.flagEpoch) & 0xffffffffull;
    red.producerOrdered = p.tileFlags != nullptr && p.tileFlags == comm->lastFlagWords &&
        red.flagEpoch == comm->lastFlagEpoch && stream == comm->lastFlagStream;
    if (red.tileFlags != nullptr && !red.producerOrdered) {
        // a launch that may wait: its workgroups claim their tokens from a shared counter (ep_token_claim.h).  The words
        // are zeroed when they are allocated and left at zero by every launch: nothing to clear here
        if (!comm->claimWord.Reserve(256, true)) {
            return TileXR::TILEXR_ERROR_INTERNAL;
        }
        red.claimWord = static_cast<uint32_t *>(comm->claimWord.ptr);
    }
    red.waitTimeoutTicks = (p.waitTimeoutUs > 0 ? p.waitTimeoutUs : kDefaultWaitUs) * kWallClockTicksPerUs;
    red.deviceStatus = p.deviceStatusOut;
    red.numComputeUnits = comm->world->numComputeUnits;
    red.kernelNameOut = &comm->lastKernel[kKernelReduce];
    red.stream = stream;
    if (SmallReduceFits(red)) {
        // decode-sized: the reduce reads the assist table itself
        return Timed(comm, kKernelReduce, stream, "reduce", [&] { return LaunchSmallReduce(red); });
    }
    if (p.rowIndexMap == nullptr) {
        if (!comm->combineScratch.Reserve(static_cast<size_t>(n) * sizeof(uint64_t), true)) {
            return TileXR::TILEXR_ERROR_INTERNAL;
        }
        inv.inverse = static_cast<uint64_t *>(comm->combineScratch.ptr);
        const int ret = Timed(comm, kKernelInvert, stream, "invert", [&] { return LaunchInvert(inv); });
        if (ret != kOk) {
            return ret;
        }
        red.inverseTagged = inv.inverse;
        red.assistTable = nullptr;
    }
    return Timed(comm, kKernelReduce, stream, "reduce", [&] { return LaunchReduce(red); });
}

// ---------------------------------------------------------------------------------------------------------
// shared call prologues
// ---------------------------------------------------------------------------------------------------------
int CommArgsOf(TileXRCommPtr handle, EpComm **comm, TileXR::CommArgs **args)
{
    // reference: src/ep/host/ep_launch_context.cpp:61-99, ep_dispatch_memory_host.cpp:108-135
    *comm = LookupComm(handle);
    if (*comm == nullptr) {
        return TileXR::TILEXR_ERROR_NOT_INITIALIZED;
    }
    *args = &(*comm)->host;
    return kOk;
}

int DispatchMvp(const EpDispatchParams &p)
{
    int ret = TileXREpValidateBasicDispatchParams(p);
    if (ret != kOk) {
        return ret;
    }
    EpComm *comm = nullptr;
    TileXR::CommArgs *args = nullptr;
    ret = CommArgsOf(p.comm, &comm, &args);
    if (ret != kOk) {
        return ret;
    }
    EpWindowConfig window {};
    ret = TileXREpValidateDispatchConfigUncapped(p, *args, &window);
    if (ret != kOk) {
        return ret;
    }
    int64_t magic = 0;
    ret = TileXRCommNextMagic(p.comm, &magic);
    if (ret != kOk) {
        return ret;
    }
    return args->rankSize == 1 ? RunDispatchSingle(comm, p, false, magic, static_cast<uint64_t>(magic) & 0xffffffffull) :
                                 RunDispatchMulti(comm, p, false, magic);
}

int DispatchMemory(const EpDispatchParams &p)
{
    int ret = TileXREpValidateBasicDispatchParams(p);
    if (ret != kOk) {
        return ret;
    }
    EpComm *comm = nullptr;
    TileXR::CommArgs *args = nullptr;
    ret = CommArgsOf(p.comm, &comm, &args);
    if (ret != kOk) {
        return ret;
    }
    EpMemoryDispatchReferenceConfig config {};
    EpDispatchParams rules = p;
    if (p.extended) {
        // the extended call accepts payload formats the reference's memory route rejects; its rule check runs with
        // the nearest reference mode and the additions are checked here
        if (p.quantMode != TILEXR_EP_QUANT_NONE && p.quantMode != TILEXR_EP_QUANT_TOKEN_INT8 &&
            p.quantMode != TILEXR_EP_QUANT_MXFP8 && p.quantMode != TILEXR_EP_QUANT_FP8_BLOCK128) {
            return TileXR::TILEXR_ERROR_NOT_SUPPORT;
        }
        if (p.expertCapacity < 0 ||
            (p.tileFlagsOut != nullptr && (p.tileRows <= 0 || p.tileRows > std::numeric_limits<int32_t>::max()))) {
            return TileXR::TILEXR_ERROR_PARA_CHECK_FAIL;
        }
        if (p.quantMode == TILEXR_EP_QUANT_TOKEN_INT8 || p.quantMode == TILEXR_EP_QUANT_FP8_BLOCK128) {
            const TileXR::TileXRDataType want = p.quantMode == TILEXR_EP_QUANT_TOKEN_INT8 ?
                TileXR::TILEXR_DATA_TYPE_INT8 : TileXR::TILEXR_DATA_TYPE_FP8E4M3;
            if (p.dynamicScalesOut == nullptr || p.expandXOutDtype != want) {
                return TileXR::TILEXR_ERROR_PARA_CHECK_FAIL;
            }
            rules.quantMode = TILEXR_EP_QUANT_NONE;
            rules.dynamicScalesOut = nullptr;
            rules.expandXOutDtype = p.dtype;
        }
        if (args->rankSize != 1) {
            return TileXR::TILEXR_ERROR_NOT_SUPPORT;
        }
    }
    ret = TileXREpValidateDispatchMemoryConfig(rules, *args, kEpReferenceBlockDim, &config, false);
    if (ret != kOk) {
        return ret;
    }
    if (p.noAlloc) {
        // worlds of several logical ranks stage rows in allocated buffers; and the static scratch has a fixed size
        if (args->rankSize != 1 || !WithinKernelLimits(p.bs, p.h, p.topK, p.moeExpertNum)) {
            return TileXR::TILEXR_ERROR_NOT_SUPPORT;
        }
        const CountScratchLayout plan = PlanCountScratch(p.bs * p.topK, p.moeExpertNum, p.moeExpertNum, false);
        if (plan.totalBytes > static_cast<int64_t>(kStaticScratchBytes)) {
            std::fprintf(stderr, "tilexr-ep: %lld routes over %lld experts need %lld bytes of scratch, the entry point that "
                "allocates nothing holds %lld\n", static_cast<long long>(p.bs * p.topK), static_cast<long long>(p.moeExpertNum),
                static_cast<long long>(plan.totalBytes), static_cast<long long>(kStaticScratchBytes));
            return TileXR::TILEXR_ERROR_NOT_SUPPORT;
        }
    }
    int64_t magic = 0;
    ret = TileXRCommNextMagic(p.comm, &magic);
    if (ret != kOk) {
        return ret;
    }
    // Readiness words are tagged from one counter for the whole process, so that two communicators that are handed the
    // same flag array (one after the other, or a destroyed and re-created one) can never tag it with the same value.
    const uint64_t flagEpoch = p.tileFlagsOut != nullptr ? NextFlagEpoch() : (static_cast<uint64_t>(magic) & 0xffffffffull);
    if (p.epochOut != nullptr) {
        *p.epochOut = static_cast<int64_t>(flagEpoch);
    }
    return args->rankSize == 1 ? RunDispatchSingle(comm, p, true, magic, flagEpoch) : RunDispatchMulti(comm, p, true, magic);
}

int CombineMvp(const EpCombineParams &p)
{
    int ret = TileXREpValidateBasicCombineParams(p);
    if (ret != kOk) {
        return ret;
    }
    EpComm *comm = nullptr;
    TileXR::CommArgs *args = nullptr;
    ret = CommArgsOf(p.comm, &comm, &args);
    if (ret != kOk) {
        return ret;
    }
    EpWindowConfig window {};
    ret = TileXREpValidateCombineConfig(p, *args, &window, false);
    if (ret != kOk) {
        return ret;
    }
    if (p.dtype != TileXR::TILEXR_DATA_TYPE_FP16 && p.dtype != TileXR::TILEXR_DATA_TYPE_BFP16) {
        // the reference's kernel leaves yOut untouched unless dtype is fp16 (tilexr_ep_combine_kernel.cpp:125);
        // int8 rows cannot be summed, so that case is reported instead of silently skipped
        return TileXR::TILEXR_ERROR_NOT_SUPPORT;
    }
    int64_t magic = 0;
    ret = TileXRCommNextMagic(p.comm, &magic);
    if (ret != kOk) {
        return ret;
    }
    return args->rankSize == 1 ? RunCombineSingle(comm, p, false, magic) : RunCombineMulti(comm, p, false, magic);
}

int CombineMemory(const EpCombineParams &p)
{
    int ret = TileXREpValidateBasicCombineParams(p);
    if (ret != kOk) {
        return ret;
    }
    EpComm *comm = nullptr;
    TileXR::CommArgs *args = nullptr;
    ret = CommArgsOf(p.comm, &comm, &args);
    if (ret != kOk) {
        return ret;
    }
    if (p.extended) {
        if (p.expertOutQuantMode != 0 && p.expertOutQuantMode != TILEXR_EP_QUANT_TOKEN_INT8 &&
            p.expertOutQuantMode != TILEXR_EP_QUANT_FP8_BLOCK128) {
            return TileXR::TILEXR_ERROR_NOT_SUPPORT;
        }
        // a combine that waits on flags must be able to report an expired wait: the status word is required
        if ((p.expertOutQuantMode != 0 && (p.expertOutScales == nullptr || p.quantMode != 0)) ||
            (p.tileFlags != nullptr && (p.tileRows <= 0 || p.tileRows > std::numeric_limits<int32_t>::max() ||
                                        p.deviceStatusOut == nullptr)) ||
            p.waitTimeoutUs < 0) {
            return TileXR::TILEXR_ERROR_PARA_CHECK_FAIL;
        }
        if (args->rankSize != 1) {
            return TileXR::TILEXR_ERROR_NOT_SUPPORT;
        }
    }
    EpMemoryCombineReferenceConfig config {};
    ret = TileXREpValidateCombineMemoryConfig(p, *args, kEpReferenceBlockDim, &config, false);
    if (ret != kOk) {
        return ret;
    }
    int64_t magic = 0;
    ret = TileXRCommNextMagic(p.comm, &magic);
    if (ret != kOk) {
        return ret;
    }
    return args->rankSize == 1 ? RunCombineSingle(comm, p, true, magic) : RunCombineMulti(comm, p, true, magic);
}

} // namespace
} // namespace TileXREp

using namespace TileXREp;

extern "C" {

const char *TileXREpVersion(void)
{
    return "tilexr-ep gfx950 abi-1";
}

int TileXREpSetKernelTimingEvents(TileXRCommPtr comm, int kernel, void *startEvent, void *stopEvent)
{
    EpComm *c = LookupComm(comm);
    if (c == nullptr) {
        return TileXR::TILEXR_ERROR_NOT_INITIALIZED;
    }
    if (kernel < 0 || kernel > kKernelReduce || ((startEvent == nullptr) != (stopEvent == nullptr))) {
        return TileXR::TILEXR_ERROR_PARA_CHECK_FAIL;
    }
    std::lock_guard<std::mutex> lock(c->mu);
    c->timing[kernel][0] = static_cast<hipEvent_t>(startEvent);
    c->timing[kernel][1] = static_cast<hipEvent_t>(stopEvent);
    return TileXR::TILEXR_SUCCESS;
}

int TileXREpSetDebugOptions(TileXRCommPtr comm, const TileXREpDebugOptions *options)
{
    EpComm *c = LookupComm(comm);
    if (c == nullptr) {
        return TileXR::TILEXR_ERROR_NOT_INITIALIZED;
    }
    if (options != nullptr && ((options->phaseStamps != nullptr) != (options->phaseStampCapacity > 0) ||
                               options->phaseStampCapacity < 0 || options->phaseStampCapacity > (int64_t{1} << 24))) {
        return TileXR::TILEXR_ERROR_PARA_CHECK_FAIL;
    }
    std::lock_guard<std::mutex> lock(c->mu);
    c->debug = DebugState {};
    if (options != nullptr) {
        c->debug.phaseStamps = options->phaseStamps;
        c->debug.capacity = options->phaseStampCapacity;
        c->debug.poison = options->poisonUnwrittenRows != 0;
    }
    return TileXR::TILEXR_SUCCESS;
}

const char *TileXREpLastKernelName(TileXRCommPtr comm, int kernel)
{
    EpComm *c = LookupComm(comm);
    if (c == nullptr || kernel < 0 || kernel > kKernelReduce) {
        return nullptr;
    }
    static const char *const fixed[5] = {nullptr, "ep_route_place_kernel", nullptr, "ep_invert_kernel", nullptr};
    std::lock_guard<std::mutex> lock(c->mu);
    return fixed[kernel] != nullptr ? fixed[kernel] : c->lastKernel[kernel];
}

int TileXRMoeEpDispatchV2(void *x, int32_t *expertIds, void *scales, bool *xActiveMask, void *expertScales,
    TileXRCommPtr comm, int64_t bs, int64_t h, int64_t topK, int64_t moeExpertNum, int64_t epWorldSize,
    int64_t epRankId, int64_t tpWorldSize, int64_t tpRankId, int64_t expertShardType, int64_t sharedExpertNum,
    int64_t sharedExpertRankNum, int64_t quantMode, int64_t globalBs, int64_t expertTokenNumsType, void *expandXOut,
    void *dynamicScalesOut, int32_t *assistInfoForCombineOut, int64_t *expertTokenNumsOut, int32_t *epRecvCountsOut,
    int32_t *tpRecvCountsOut, void *expandScalesOut, void *workspace, TileXR::TileXRDataType dtype,
    aclrtStream stream)
{
    EpDispatchParams p {};
    p.x = x;
    p.expertIds = expertIds;
    p.scales = scales;
    p.xActiveMask = xActiveMask;
    p.expertScales = expertScales;
    p.comm = comm;
    p.bs = bs;
    p.h = h;
    p.topK = topK;
    p.moeExpertNum = moeExpertNum;
    p.epWorldSize = epWorldSize;
    p.epRankId = epRankId;
    p.tpWorldSize = tpWorldSize;
    p.tpRankId = tpRankId;
    p.expertShardType = expertShardType;
    p.sharedExpertNum = sharedExpertNum;
    p.sharedExpertRankNum = sharedExpertRankNum;
    p.quantMode = quantMode;
    p.globalBs = globalBs;
    p.expertTokenNumsType = expertTokenNumsType;
    p.expandXOut = expandXOut;
    p.dynamicScalesOut = dynamicScalesOut;
    p.assistInfoForCombineOut = assistInfoForCombineOut;
    p.expertTokenNumsOut = expertTokenNumsOut;
    p.epRecvCountsOut = epRecvCountsOut;
    p.tpRecvCountsOut = tpRecvCountsOut;
    p.expandScalesOut = expandScalesOut;
    p.workspace = workspace;
    p.dtype = dtype;
    p.stream = stream;
    return DispatchMvp(p);
}

int TileXRMoeEpDispatch(void *x, int32_t *expertIds, TileXRCommPtr comm, int64_t bs, int64_t h, int64_t topK,
    int64_t moeExpertNum, void *expandXOut, int64_t *expertTokenNumsOut, int32_t *epRecvCountsOut,
    int32_t *assistInfoForCombineOut, TileXR::TileXRDataType dtype, aclrtStream stream)
{
    // reference: tilexr_ep_dispatch.cpp:85-94 -- V2 with everything optional off and counts (type 1)
    return TileXRMoeEpDispatchV2(x, expertIds, nullptr, nullptr, nullptr, comm, bs, h, topK, moeExpertNum, 0, 0, 0, 0,
        0, 0, 0, 0, 0, kEpExpertTokenNumsTypeCount, expandXOut, nullptr, assistInfoForCombineOut, expertTokenNumsOut,
        epRecvCountsOut, nullptr, nullptr, nullptr, dtype, stream);
}

int TileXRMoeEpDispatchMemoryV2(void *x, int32_t *expertIds, void *scales, bool *xActiveMask,
    int64_t activeMaskType, void *expertScales, TileXRCommPtr comm, int64_t bs, int64_t h, int64_t topK,
    int64_t moeExpertNum, int64_t epWorldSize, int64_t epRankId, int64_t tpWorldSize, int64_t tpRankId,
    int64_t expertShardType, int64_t sharedExpertNum, int64_t sharedExpertRankNum, int64_t quantMode,
    int64_t globalBs, int64_t expertTokenNumsType, void *expandXOut, void *dynamicScalesOut,
    int32_t *assistInfoForCombineOut, int64_t *expertTokenNumsOut, int32_t *sendCountsOut, int32_t *tpRecvCountsOut,
    void *expandScalesOut, TileXR::TileXRDataType dtype, TileXR::TileXRDataType expandXOutDtype, aclrtStream stream)
{
    EpDispatchParams p {};
    p.x = x;
    p.expertIds = expertIds;
    p.scales = scales;
    p.xActiveMask = xActiveMask;
    p.activeMaskType = activeMaskType;
    p.expertScales = expertScales;
    p.comm = comm;
    p.bs = bs;
    p.h = h;
    p.topK = topK;
    p.moeExpertNum = moeExpertNum;
    p.epWorldSize = epWorldSize;
    p.epRankId = epRankId;
    p.tpWorldSize = tpWorldSize;
    p.tpRankId = tpRankId;
    p.expertShardType = expertShardType;
    p.sharedExpertNum = sharedExpertNum;
    p.sharedExpertRankNum = sharedExpertRankNum;
    p.quantMode = quantMode;
    p.globalBs = globalBs;
    p.expertTokenNumsType = expertTokenNumsType;
    p.expandXOut = expandXOut;
    p.dynamicScalesOut = dynamicScalesOut;
    p.assistInfoForCombineOut = assistInfoForCombineOut;
    p.expertTokenNumsOut = expertTokenNumsOut;
    p.epRecvCountsOut = sendCountsOut;
    p.tpRecvCountsOut = tpRecvCountsOut;
    p.expandScalesOut = expandScalesOut;
    p.dtype = dtype;
    p.expandXOutDtype = expandXOutDtype;
    p.stream = stream;
    return DispatchMemory(p);
}

int TileXRMoeEpDispatchMemory(void *x, int32_t *expertIds, TileXRCommPtr comm, int64_t bs, int64_t h, int64_t topK,
    int64_t moeExpertNum, void *expandXOut, int64_t *expertTokenNumsOut, int32_t *sendCountsOut,
    int32_t *assistInfoForCombineOut, TileXR::TileXRDataType dtype, aclrtStream stream)
{
    // reference: tilexr_ep_memory_dispatch.cpp:73-82 -- no mask, no quantisation, counts (type 1)
    return TileXRMoeEpDispatchMemoryV2(x, expertIds, nullptr, nullptr, TILEXR_EP_ACTIVE_MASK_NONE, nullptr, comm, bs, h,
        topK, moeExpertNum, 0, 0, 1, 0, 0, 0, 0, 0, 0, kEpExpertTokenNumsTypeCount, expandXOut, nullptr,
        assistInfoForCombineOut, expertTokenNumsOut, sendCountsOut, nullptr, nullptr, dtype, dtype, stream);
}

int TileXRMoeEpDispatchMemoryNoAlloc(void *x, int32_t *expertIds, TileXRCommPtr comm, int64_t bs, int64_t h,
    int64_t topK, int64_t moeExpertNum, void *expandXOut, int64_t *expertTokenNumsOut, int32_t *sendCountsOut,
    int32_t *assistInfoForCombineOut, TileXR::TileXRDataType dtype, aclrtStream stream)
{
    EpDispatchParams p {};
    p.x = x;
    p.expertIds = expertIds;
    p.comm = comm;
    p.bs = bs;
    p.h = h;
    p.topK = topK;
    p.moeExpertNum = moeExpertNum;
    p.tpWorldSize = 1;
    p.expertTokenNumsType = kEpExpertTokenNumsTypeCount;
    p.expandXOut = expandXOut;
    p.assistInfoForCombineOut = assistInfoForCombineOut;
    p.expertTokenNumsOut = expertTokenNumsOut;
    p.epRecvCountsOut = sendCountsOut;
    p.dtype = dtype;
    p.expandXOutDtype = dtype;
    p.stream = stream;
    p.noAlloc = true;
    return DispatchMemory(p);
}

int TileXRMoeEpDispatchMemoryEx(void *x, int32_t *expertIds, TileXRCommPtr comm, int64_t bs, int64_t h,
    int64_t topK, int64_t moeExpertNum, const TileXREpDispatchExOptions *options, void *expandXOut,
    void *dynamicScalesOut, int32_t *assistInfoForCombineOut, int64_t *expertTokenNumsOut, int32_t *sendCountsOut,
    TileXR::TileXRDataType dtype, TileXR::TileXRDataType expandXOutDtype, aclrtStream stream)
{
    if (options == nullptr) {
        return TileXR::TILEXR_ERROR_PARA_CHECK_FAIL;
    }
    EpDispatchParams p {};
    p.x = x;
    p.expertIds = expertIds;
    p.xActiveMask = options->xActiveMask;
    p.activeMaskType = options->activeMaskType;
    p.comm = comm;
    p.bs = bs;
    p.h = h;
    p.topK = topK;
    p.moeExpertNum = moeExpertNum;
    p.tpWorldSize = 1;
    p.quantMode = options->quantMode;
    p.expertTokenNumsType = options->expertTokenNumsType;
    p.expandXOut = expandXOut;
    p.dynamicScalesOut = dynamicScalesOut;
    p.assistInfoForCombineOut = assistInfoForCombineOut;
    p.expertTokenNumsOut = expertTokenNumsOut;
    p.epRecvCountsOut = sendCountsOut;
    p.dtype = dtype;
    p.expandXOutDtype = expandXOutDtype;
    p.stream = stream;
    p.expertCapacity = options->expertCapacity;
    p.rowIndexMapOut = options->rowIndexMapOut;
    p.tileFlagsOut = options->tileFlagsOut;
    p.tileRows = options->tileRows;
    p.epochOut = options->epochOut;
    p.metaReadyEvent = options->metaReadyEvent;
    p.extended = true;
    return DispatchMemory(p);
}

int TileXRMoeEpCombineV2(void *expertOut, int32_t *assistInfoForCombine, int32_t *epRecvCounts, TileXRCommPtr comm,
    int64_t bs, int64_t h, int64_t topK, int64_t moeExpertNum, void *yOut, void *workspace,
    TileXR::TileXRDataType dtype, aclrtStream stream)
{
    EpCombineParams p {};
    p.expertOut = expertOut;
    p.assistInfoForCombine = assistInfoForCombine;
    p.epRecvCounts = epRecvCounts;
    p.comm = comm;
    p.bs = bs;
    p.h = h;
    p.topK = topK;
    p.moeExpertNum = moeExpertNum;
    p.yOut = yOut;
    p.workspace = workspace;
    p.dtype = dtype;
    p.stream = stream;
    return CombineMvp(p);
}

int TileXRMoeEpCombine(void *expertOut, int32_t *assistInfoForCombine, int32_t *epRecvCounts, TileXRCommPtr comm,
    int64_t bs, int64_t h, int64_t topK, int64_t moeExpertNum, void *yOut, TileXR::TileXRDataType dtype,
    aclrtStream stream)
{
    return TileXRMoeEpCombineV2(expertOut, assistInfoForCombine, epRecvCounts, comm, bs, h, topK, moeExpertNum, yOut,
        nullptr, dtype, stream);
}

int TileXRMoeEpCombineMemoryV2(void *expertOut, int32_t *assistInfoForCombine, int32_t *sendCounts,
    float *expertScales, bool *xActiveMask, int64_t activeMaskType, void *sharedExpertX, TileXRCommPtr comm,
    int64_t bs, int64_t h, int64_t topK, int64_t moeExpertNum, int64_t epWorldSize, int64_t epRankId,
    int64_t tpWorldSize, int64_t tpRankId, int64_t expertShardType, int64_t sharedExpertNum,
    int64_t sharedExpertRankNum, int64_t quantMode, int64_t globalBs, void *yOut, TileXR::TileXRDataType dtype,
    aclrtStream stream)
{
    EpCombineParams p {};
    p.expertOut = expertOut;
    p.assistInfoForCombine = assistInfoForCombine;
    p.epRecvCounts = sendCounts;
    p.expertScales = expertScales;
    p.xActiveMask = xActiveMask;
    p.activeMaskType = activeMaskType;
    p.sharedExpertX = sharedExpertX;
    p.comm = comm;
    p.bs = bs;
    p.h = h;
    p.topK = topK;
    p.moeExpertNum = moeExpertNum;
    p.epWorldSize = epWorldSize;
    p.epRankId = epRankId;
    p.tpWorldSize = tpWorldSize;
    p.tpRankId = tpRankId;
    p.expertShardType = expertShardType;
    p.sharedExpertNum = sharedExpertNum;
    p.sharedExpertRankNum = sharedExpertRankNum;
    p.quantMode = quantMode;
    p.globalBs = globalBs;
    p.yOut = yOut;
    p.dtype = dtype;
    p.stream = stream;
    return CombineMemory(p);
}

int TileXRMoeEpCombineMemory(void *expertOut, int32_t *assistInfoForCombine, int32_t *epRecvCounts,
    TileXRCommPtr comm, int64_t bs, int64_t h, int64_t topK, int64_t moeExpertNum, void *yOut,
    TileXR::TileXRDataType dtype, aclrtStream stream)
{
    // reference: tilexr_ep_memory_combine.cpp:61-68
    return TileXRMoeEpCombineMemoryV2(expertOut, assistInfoForCombine, epRecvCounts, nullptr, nullptr,
        TILEXR_EP_ACTIVE_MASK_NONE, nullptr, comm, bs, h, topK, moeExpertNum, 0, 0, 1, 0, 0, 0, 0, 0, 0, yOut, dtype,
        stream);
}

int TileXRMoeEpCombineMemoryEx(void *expertOut, int32_t *assistInfoForCombine, int32_t *sendCounts,
    TileXRCommPtr comm, int64_t bs, int64_t h, int64_t topK, int64_t moeExpertNum,
    const TileXREpCombineExOptions *options, void *yOut, TileXR::TileXRDataType dtype, aclrtStream stream)
{
    if (options == nullptr) {
        return TileXR::TILEXR_ERROR_PARA_CHECK_FAIL;
    }
    EpCombineParams p {};
    p.expertOut = expertOut;
    p.assistInfoForCombine = assistInfoForCombine;
    p.epRecvCounts = sendCounts;
    p.expertScales = options->expertScales;
    p.xActiveMask = options->xActiveMask;
    p.activeMaskType = options->activeMaskType;
    p.sharedExpertX = options->sharedExpertX;
    p.comm = comm;
    p.bs = bs;
    p.h = h;
    p.topK = topK;
    p.moeExpertNum = moeExpertNum;
    p.tpWorldSize = 1;
    p.quantMode = options->commQuantMode;
    p.yOut = yOut;
    p.dtype = dtype;
    p.stream = stream;
    p.expertOutQuantMode = options->expertOutQuantMode;
    p.expertOutScales = options->expertOutScales;
    p.rowIndexMap = options->rowIndexMap;
    p.tileFlags = options->tileFlags;
    p.tileRows = options->tileRows;
    p.flagEpoch = options->flagEpoch;
    p.waitTimeoutUs = options->waitTimeoutUs;
    p.deviceStatusOut = options->deviceStatusOut;
    p.extended = true;
    return CombineMemory(p);
}

}
