// Dispatch / combine across several logical ranks that share the device (rankSize > 1).
//
// The reference runs one process per rank and lets kernels spin on flags in each other's peer windows
// (src/ep/kernels/tilexr_ep_dispatch_kernel.cpp:700-836, tilexr_ep_dispatch_memory_kernel.h:1549-1562).  With every
// rank in one process and on one device, spinning kernels could starve each other, so the exchange is ordered by
// the host instead: a call enqueues its rank's SEND half on the caller's stream immediately; when the last rank of
// the world has called, the DRAIN half of every rank is enqueued on that rank's own stream behind events of all
// send halves.  A rank's outputs are therefore complete once every rank has made the call and the rank's stream
// has been synchronised -- the same moment the reference's kernels would pass their barriers.
#include <algorithm>

#include "ep_context.h"
#include "ep_exchange.h"
#include "ep_host.h"
#include "ep_launch.h"
#include "ep_run_common.h"

namespace TileXREp {
namespace {

constexpr int kOk = TileXR::TILEXR_SUCCESS;

int64_t Align256(int64_t v)
{
    return (v + 255) / 256 * 256;
}

int64_t MxScaleBytes(int64_t h)
{
    return ((h + 31) / 32 + 1) / 2 * 2;
}

bool EnsureEvents(RankEvents *e)
{
    if (e->sent == nullptr && hipEventCreateWithFlags(&e->sent, hipEventDisableTiming) != hipSuccess) {
        return false;
    }
    if (e->drained == nullptr && hipEventCreateWithFlags(&e->drained, hipEventDisableTiming) != hipSuccess) {
        return false;
    }
    return true;
}

// Key space of a world: position = rank * keysPerRank + local index on that rank.  Without shared experts this is
// the expert id itself (keysPerRank = experts per rank).  With shared experts (reference: expert placement in
// src/ep/kernels/tilexr_ep_dispatch_helpers.h:63-103) ranks [0, sharedRanks) host them, the routed experts are spread
// over the other ranks, and a shared route takes local index 0 on its rank (memory route: a shared rank presents one
// local expert, tilexr_ep_dispatch_memory_kernel.h:1153) or its own expert id (MVP route: the drain files a shared row
// under index expertId, tilexr_ep_combine_helpers.h:124-128), hence keysPerRank = max(localExperts, sharedNum) there.
struct StagePlan {
    StageLayout layout {};
    int64_t rowBytes = 0;
    int64_t scaleBytesPerRow = 0;
    int64_t numKeys = 0;
    int64_t keyDiv = 1;
    int64_t localExperts = 0;    // routed experts per non-shared rank
    int64_t keysPerRank = 0;
    int64_t keySpace = 0;        // rankSize * keysPerRank
    int64_t perToken = 0;        // routes per token: shared + topK
    bool expertHist = false;
};

// Sizes the world's staging for one dispatch shape and points `layout` at it.
bool PlanStage(EpWorld *world, const ExchangeShape &shape, bool reserve, StagePlan *plan)
{
    const int64_t R = world->rankSize;
    plan->perToken = shape.topK + shape.sharedNum;
    const int64_t n = shape.bs * plan->perToken;
    // with tensor-parallel groups (MVP route) experts are placed on the R / tp expert ranks and a key names an
    // expert rank; the lane a row travels on is the source's own (reference: tilexr_ep_dispatch_kernel.cpp:382-392)
    const int64_t expertRanks = R / shape.tp;
    plan->localExperts = shape.experts / (expertRanks - shape.sharedRanks);
    plan->keysPerRank = shape.memoryRoute ? plan->localExperts : std::max(plan->localExperts, shape.sharedNum);
    plan->keySpace = expertRanks * plan->keysPerRank;
    plan->rowBytes = shape.quantMode == TILEXR_EP_QUANT_NONE ? shape.h * 2 : shape.h;
    plan->scaleBytesPerRow = shape.quantMode == TILEXR_EP_QUANT_TOKEN_INT8 ? 4 :
        (shape.quantMode == TILEXR_EP_QUANT_MXFP8 ? MxScaleBytes(shape.h) : 0);
    plan->numKeys = shape.memoryRoute ? plan->keySpace : expertRanks;
    plan->keyDiv = shape.memoryRoute ? 1 : plan->keysPerRank;
    plan->expertHist = !shape.memoryRoute;
    StageLayout &l = plan->layout;
    l.rowsStride = Align256(n * plan->rowBytes);
    l.scalesOffset = Align256(n * 16);
    l.auxStride = l.scalesOffset + Align256(n * plan->scaleBytesPerRow);
    l.expertTotalOffset = plan->numKeys + 1;
    l.countsStride = (plan->numKeys + 1 + plan->keySpace + 63) / 64 * 64;
    if (reserve) {
        if (!world->stageRows.Reserve(static_cast<size_t>(R * l.rowsStride), false) ||
            !world->stageAux.Reserve(static_cast<size_t>(R * l.auxStride), false) ||
            !world->stageCounts.Reserve(static_cast<size_t>(R * l.countsStride * 4), true)) {
            return false;
        }
    }
    l.rows = static_cast<char *>(world->stageRows.ptr);
    l.aux = static_cast<char *>(world->stageAux.ptr);
    l.counts = static_cast<int32_t *>(world->stageCounts.ptr);
    return true;
}

int DrainRank(EpWorld *world, int q, const ExchangeShape &shape, const StagePlan &plan)
{
    EpComm *comm = world->comms[static_cast<size_t>(q)];
    const EpDispatchParams &p = world->pendingDispatch[static_cast<size_t>(q)].params;
    hipStream_t stream = static_cast<hipStream_t>(p.stream);
    const int R = world->rankSize;
    const int localExperts = static_cast<int>(plan.keysPerRank);
    // a shared-expert rank presents one local expert on the memory route
    // (reference: src/ep/kernels/tilexr_ep_dispatch_memory_kernel.h:1153, tests/ep/demo/tilexr_ep_dispatch_demo.cpp:632-635)
    const int outLocalExperts = q < shape.sharedRanks ? 1 : static_cast<int>(plan.localExperts);
    const int64_t numSeg = shape.memoryRoute ? static_cast<int64_t>(outLocalExperts) * R : R;
    for (int s = 0; s < R; ++s) {
        if (hipStreamWaitEvent(stream, world->dispatchEvents[static_cast<size_t>(s)].sent, 0) != hipSuccess) {
            return TileXR::TILEXR_ERROR_INTERNAL;
        }
    }
    if (!comm->drainScratch.Reserve(static_cast<size_t>(numSeg + 1) * 4, false)) {
        return TileXR::TILEXR_ERROR_INTERNAL;
    }
    DrainPlanLaunch dp {};
    dp.stage = plan.layout;
    dp.rankSize = R;
    dp.dstRank = q;
    dp.localExperts = localExperts;
    dp.outLocalExperts = outLocalExperts;
    dp.tokenNumsCount = shape.memoryRoute ? outLocalExperts : static_cast<int>(plan.localExperts);
    dp.tp = static_cast<int>(shape.tp);
    dp.memoryRoute = shape.memoryRoute;
    dp.planOffsets = static_cast<int32_t *>(comm->drainScratch.ptr);
    dp.countsOut = p.epRecvCountsOut;
    dp.tpCountsOut = shape.memoryRoute ? nullptr : p.tpRecvCountsOut;
    dp.expertTokenNumsOut = p.expertTokenNumsOut;
    dp.tokenNumsType = static_cast<int>(p.expertTokenNumsType);
    dp.stream = stream;
    int ret = LaunchStatus(LaunchDrainPlan(dp), "drain plan");
    if (ret != kOk) {
        return ret;
    }
    DrainCopyLaunch dc {};
    dc.stage = plan.layout;
    dc.rankSize = R;
    dc.dstRank = q;
    dc.localExperts = localExperts;
    dc.outLocalExperts = outLocalExperts;
    dc.tp = static_cast<int>(shape.tp);
    dc.memoryRoute = shape.memoryRoute;
    dc.planOffsets = dp.planOffsets;
    dc.maxRows = static_cast<int64_t>(R) * shape.bs * plan.perToken;
    dc.rowBytes = plan.rowBytes;
    dc.scaleBytesPerRow = plan.scaleBytesPerRow;
    dc.expandXOut = p.expandXOut;
    dc.assistOut = p.assistInfoForCombineOut;
    dc.scalesOut = p.dynamicScalesOut;
    dc.stream = stream;
    ret = LaunchStatus(LaunchDrainCopy(dc), "drain copy");
    if (ret != kOk) {
        return ret;
    }
    RankEvents &ev = world->dispatchEvents[static_cast<size_t>(q)];
    if (hipEventRecord(ev.drained, stream) != hipSuccess) {
        return TileXR::TILEXR_ERROR_INTERNAL;
    }
    ev.drainedArmed = true;
    return kOk;
}

} // namespace

int RunDispatchMulti(EpComm *comm, const EpDispatchParams &p, bool memoryRoute, int64_t magic)
{
    EpWorld *world = comm->world;
    const int R = world->rankSize;
    const int r = comm->rank;
    const int64_t shared = p.sharedExpertNum;
    const int64_t tp = (!memoryRoute && p.tpWorldSize > 1) ? p.tpWorldSize : 1;
    const int64_t keySpaceBound = static_cast<int64_t>(R / tp) *
        std::max(p.moeExpertNum / (R / tp - p.sharedExpertRankNum), shared);
    if (!WithinKernelLimits(p.bs, p.h, p.topK + shared, std::max(p.moeExpertNum, keySpaceBound), R) || p.extended) {
        return TileXR::TILEXR_ERROR_NOT_SUPPORT;
    }
    hipStream_t stream = static_cast<hipStream_t>(p.stream);
    ExchangeShape shape {};
    shape.bs = p.bs;
    shape.h = p.h;
    shape.topK = p.topK;
    shape.experts = p.moeExpertNum;
    shape.quantMode = p.quantMode;
    shape.sharedNum = shared;
    shape.sharedRanks = p.sharedExpertRankNum;
    shape.tp = tp;
    shape.dtype = static_cast<int>(p.dtype);
    shape.outDtype = static_cast<int>(p.expandXOutDtype);
    shape.memoryRoute = memoryRoute;

    std::lock_guard<std::mutex> lock(world->mu);
    comm->debug.magic = magic;
    for (int s = 0; s < R; ++s) {
        if (world->comms[static_cast<size_t>(s)] == nullptr) {
            return TileXR::TILEXR_ERROR_NOT_INITIALIZED;     // the world is not complete yet
        }
    }
    if (world->pendingDispatch[static_cast<size_t>(r)].present) {
        return TileXR::TILEXR_ERROR_INTERNAL;                // this rank already sent in the exchange in flight
    }
    bool first = true;
    for (const PendingDispatch &pd : world->pendingDispatch) {
        first = first && !pd.present;
    }
    if (first) {
        world->dispatchShape = shape;
    } else if (!(shape == world->dispatchShape)) {
        return TileXR::TILEXR_ERROR_PARA_CHECK_FAIL;         // all ranks of one exchange use the same shape
    }
    StagePlan plan {};
    if (!PlanStage(world, shape, first, &plan)) {
        return TileXR::TILEXR_ERROR_INTERNAL;
    }
    RankEvents &mine = world->dispatchEvents[static_cast<size_t>(r)];
    if (!EnsureEvents(&mine)) {
        return TileXR::TILEXR_ERROR_INTERNAL;
    }
    // the previous exchange's drains read the staging areas this send is about to overwrite
    for (int q = 0; q < R; ++q) {
        const RankEvents &ev = world->dispatchEvents[static_cast<size_t>(q)];
        if (ev.drainedArmed && hipStreamWaitEvent(stream, ev.drained, 0) != hipSuccess) {
            return TileXR::TILEXR_ERROR_INTERNAL;
        }
    }

    // ---- send half: group this rank's rows by destination in its staging area ----
    const int64_t n = p.bs * plan.perToken;
    const CountScratchLayout cs = PlanCountScratch(n, plan.numKeys, plan.keySpace, plan.expertHist);
    const int64_t tableBytes = shared > 0 ? Align256(n * 4) : 0;      // key ids, tuple expert ids, widened mask
    if (!comm->dispatchScratch.Reserve(static_cast<size_t>(cs.totalBytes + 3 * tableBytes), true)) {
        return TileXR::TILEXR_ERROR_INTERNAL;
    }
    const uint8_t *routeMask = reinterpret_cast<const uint8_t *>(p.xActiveMask);
    CountScratch scratch = CarveCountScratch(comm->dispatchScratch.ptr, cs, plan.expertHist);
    const int32_t *routeIds = p.expertIds;
    const int32_t *tupleExperts = nullptr;
    if (shared > 0) {
        int32_t *keyIds = reinterpret_cast<int32_t *>(static_cast<char *>(comm->dispatchScratch.ptr) + cs.totalBytes);
        int32_t *tuples = reinterpret_cast<int32_t *>(static_cast<char *>(comm->dispatchScratch.ptr) + cs.totalBytes +
            tableBytes);
        AugmentLaunch aug {};
        aug.ids = p.expertIds;
        aug.bs = p.bs;
        aug.topK = p.topK;
        aug.moeExpertNum = p.moeExpertNum;
        aug.rankSize = R;
        aug.srcRank = static_cast<int>(r / tp);      // the placement rules see the source's expert rank
        aug.sharedNum = static_cast<int>(shared);
        aug.sharedRanks = static_cast<int>(p.sharedExpertRankNum);
        aug.localExperts = static_cast<int>(plan.localExperts);
        aug.keysPerRank = static_cast<int>(plan.keysPerRank);
        aug.sharedAtExpertId = !memoryRoute;
        aug.keyIdsOut = keyIds;
        aug.tupleExpertsOut = tuples;
        if (memoryRoute && p.xActiveMask != nullptr && p.activeMaskType == TILEXR_EP_ACTIVE_MASK_EXPERT) {
            uint8_t *wide = reinterpret_cast<uint8_t *>(static_cast<char *>(comm->dispatchScratch.ptr) + cs.totalBytes +
                2 * tableBytes);
            aug.routeMask = routeMask;
            aug.routeMaskOut = wide;
            routeMask = wide;
        }
        aug.stream = stream;
        const int ar = LaunchStatus(LaunchAugment(aug), "route tables");
        if (ar != kOk) {
            return ar;
        }
        routeIds = keyIds;
        tupleExperts = tuples;
    }
    int32_t *myCounts = plan.layout.counts + static_cast<int64_t>(r) * plan.layout.countsStride;
    scratch.keyOffset = myCounts;
    scratch.expertTotal = myCounts + plan.layout.expertTotalOffset;
    int32_t *rowOf = reinterpret_cast<int32_t *>(static_cast<char *>(comm->dispatchScratch.ptr) + cs.rowOfOff);
    char *myRows = plan.layout.rows + static_cast<int64_t>(r) * plan.layout.rowsStride;
    char *myAux = plan.layout.aux + static_cast<int64_t>(r) * plan.layout.auxStride;

    RouteCountLaunch count {};
    count.ids = routeIds;
    count.mask = routeMask;
    if (p.xActiveMask == nullptr) {
        count.maskMode = kMaskNone;
    } else if (!memoryRoute) {
        count.maskMode = kMaskPerToken;
    } else {
        count.maskMode = p.activeMaskType == TILEXR_EP_ACTIVE_MASK_EXPERT ? kMaskPerRoute : kMaskTokenPrefix;
    }
    count.bs = p.bs;
    count.topK = plan.perToken;
    count.numExperts = plan.keySpace;
    count.keyDiv = plan.keyDiv;
    count.numKeys = plan.numKeys;
    count.capacity = 0;
    count.scratch = scratch;
    count.tokenNumsType = static_cast<int>(p.expertTokenNumsType);
    count.stream = stream;
    comm->lastKernel[kKernelCount] = "ep_route_count_kernel";
    int ret = Timed(comm, kKernelCount, stream, "route count", [&] { return LaunchRouteCount(count); });
    if (ret != kOk) {
        return ret;
    }
    RoutePlaceLaunch place {};
    place.ids = routeIds;
    place.bs = p.bs;
    place.topK = plan.perToken;
    place.keyDiv = plan.keyDiv;
    place.numKeys = plan.numKeys;
    place.scratch = scratch;
    place.srcRank = r;
    place.expertIdBias = 0;
    place.sharedNum = static_cast<int32_t>(shared);
    place.tupleExperts = tupleExperts;
    place.rowOf = rowOf;
    place.assist = reinterpret_cast<int32_t *>(myAux);
    place.stream = stream;
    ret = Timed(comm, kKernelPlace, stream, "route place", [&] { return LaunchRoutePlace(place); });
    if (ret != kOk) {
        return ret;
    }
    ScatterLaunch scatter {};
    scatter.x = p.x;
    scatter.rowOf = rowOf;
    scatter.bs = p.bs;
    scatter.h = p.h;
    scatter.topK = plan.perToken;
    scatter.quantMode = static_cast<int>(p.quantMode);
    scatter.inputBf16 = memoryRoute && p.dtype == TileXR::TILEXR_DATA_TYPE_BFP16;
    scatter.fp8E5m2 = p.expandXOutDtype == TileXR::TILEXR_DATA_TYPE_FP8E5M2;
    scatter.staticScale = static_cast<const float *>(p.scales);
    scatter.out = myRows;
    scatter.scalesOut = myAux + plan.layout.scalesOffset;
    scatter.stream = stream;
    ret = Timed(comm, kKernelScatter, stream, "scatter", [&] { return LaunchScatter(scatter); });
    if (ret != kOk) {
        return ret;
    }
    if (hipEventRecord(mine.sent, stream) != hipSuccess) {
        return TileXR::TILEXR_ERROR_INTERNAL;
    }
    world->pendingDispatch[static_cast<size_t>(r)].present = true;
    world->pendingDispatch[static_cast<size_t>(r)].params = p;

    // ---- drain halves, once the last rank has sent ----
    for (const PendingDispatch &pd : world->pendingDispatch) {
        if (!pd.present) {
            return kOk;
        }
    }
    int status = kOk;
    for (int q = 0; q < R; ++q) {
        if (!EnsureEvents(&world->dispatchEvents[static_cast<size_t>(q)])) {
            status = TileXR::TILEXR_ERROR_INTERNAL;
            break;
        }
        const int dr = DrainRank(world, q, shape, plan);
        if (dr != kOk) {
            status = dr;
            break;
        }
    }
    for (PendingDispatch &pd : world->pendingDispatch) {
        pd.present = false;
    }
    return status;
}

int RunCombineMulti(EpComm *comm, const EpCombineParams &p, bool memoryRoute, int64_t magic)
{
    (void)magic;
    EpWorld *world = comm->world;
    const int R = world->rankSize;
    const int er = comm->rank;
    // shared-expert rows come back to the slots after the routed ones on the memory route; the MVP route's combine
    // drops them (reference: src/ep/kernels/tilexr_ep_combine_kernel.cpp:94-97)
    const int64_t shared = memoryRoute ? p.sharedExpertNum : 0;
    const int64_t perToken = p.topK + shared;
    if (!WithinKernelLimits(p.bs, p.h, perToken, p.moeExpertNum, R) || p.extended) {
        return TileXR::TILEXR_ERROR_NOT_SUPPORT;
    }
    hipStream_t stream = static_cast<hipStream_t>(p.stream);
    ExchangeShape shape {};
    shape.bs = p.bs;
    shape.h = p.h;
    shape.topK = p.topK;
    shape.experts = p.moeExpertNum;
    shape.quantMode = p.quantMode;
    shape.sharedNum = shared;
    shape.sharedRanks = memoryRoute ? p.sharedExpertRankNum : 0;
    shape.dtype = static_cast<int>(p.dtype);
    shape.memoryRoute = memoryRoute;

    std::lock_guard<std::mutex> lock(world->mu);
    comm->debug.magic = magic;
    for (int s = 0; s < R; ++s) {
        if (world->comms[static_cast<size_t>(s)] == nullptr) {
            return TileXR::TILEXR_ERROR_NOT_INITIALIZED;
        }
    }
    if (world->pendingCombine[static_cast<size_t>(er)].present) {
        return TileXR::TILEXR_ERROR_INTERNAL;
    }
    bool first = true;
    for (const PendingCombine &pc : world->pendingCombine) {
        first = first && !pc.present;
    }
    const int64_t n = p.bs * perToken;
    const int64_t rowBytes = p.h * 2;
    const int64_t slotsStride = Align256(n * rowBytes);
    const int64_t metaStride = (2 * n + 31) / 32 * 32;
    if (first) {
        world->combineShape = shape;
        ++world->combineEpoch;
        if (!world->combineSlots.Reserve(static_cast<size_t>(R * slotsStride), false) ||
            !world->combineMeta.Reserve(static_cast<size_t>(R * metaStride * 8), true)) {
            return TileXR::TILEXR_ERROR_INTERNAL;
        }
    } else if (!(shape == world->combineShape)) {
        return TileXR::TILEXR_ERROR_PARA_CHECK_FAIL;
    }
    RankEvents &mine = world->combineEvents[static_cast<size_t>(er)];
    if (!EnsureEvents(&mine)) {
        return TileXR::TILEXR_ERROR_INTERNAL;
    }
    for (int q = 0; q < R; ++q) {
        const RankEvents &ev = world->combineEvents[static_cast<size_t>(q)];
        if (ev.drainedArmed && hipStreamWaitEvent(stream, ev.drained, 0) != hipSuccess) {
            return TileXR::TILEXR_ERROR_INTERNAL;
        }
    }
    const uint64_t epoch = world->combineEpoch & 0xffffffffull;

    // ---- send half: every row of this expert rank goes back to the slot (token, k) of its source rank ----
    ReturnRowsLaunch back {};
    back.expertOut = p.expertOut;
    back.assist = p.assistInfoForCombine;
    back.counts = p.epRecvCounts;
    // memory route: the rows of this expert rank = last entry of its sendCounts, which has one block of R entries per
    // local expert (a single block on a shared-expert rank)
    const int64_t localExperts = p.moeExpertNum / (R - shape.sharedRanks);
    back.numCounts = memoryRoute ? (er < shape.sharedRanks ? 1 : localExperts) * R : R;
    back.memoryRoute = memoryRoute;
    back.maxCountPerEntry = n;
    back.maxRows = static_cast<int64_t>(R) * n;
    back.rowBytes = rowBytes;
    back.rankSize = R;
    back.expertRank = er;
    back.bs = p.bs;
    back.topK = perToken;
    back.epoch = epoch;
    back.slots = static_cast<char *>(world->combineSlots.ptr);
    back.slotsStride = slotsStride;
    back.meta = static_cast<uint64_t *>(world->combineMeta.ptr);
    back.metaStride = metaStride;
    back.stream = stream;
    int ret = LaunchStatus(LaunchReturnRows(back), "return rows");
    if (ret != kOk) {
        return ret;
    }
    if (hipEventRecord(mine.sent, stream) != hipSuccess) {
        return TileXR::TILEXR_ERROR_INTERNAL;
    }
    world->pendingCombine[static_cast<size_t>(er)].present = true;
    world->pendingCombine[static_cast<size_t>(er)].params = p;
    for (const PendingCombine &pc : world->pendingCombine) {
        if (!pc.present) {
            return kOk;
        }
    }

    // ---- reduce halves ----
    int status = kOk;
    for (int r = 0; r < R && status == kOk; ++r) {
        const EpCombineParams &rp = world->pendingCombine[static_cast<size_t>(r)].params;
        EpComm *rc = world->comms[static_cast<size_t>(r)];
        hipStream_t rs = static_cast<hipStream_t>(rp.stream);
        RankEvents &ev = world->combineEvents[static_cast<size_t>(r)];
        if (!EnsureEvents(&ev)) {
            status = TileXR::TILEXR_ERROR_INTERNAL;
            break;
        }
        for (int s = 0; s < R; ++s) {
            if (hipStreamWaitEvent(rs, world->combineEvents[static_cast<size_t>(s)].sent, 0) != hipSuccess) {
                status = TileXR::TILEXR_ERROR_INTERNAL;
            }
        }
        uint64_t *meta = static_cast<uint64_t *>(world->combineMeta.ptr) + static_cast<int64_t>(r) * metaStride;
        ReduceLaunch red {};
        red.expertOut = static_cast<char *>(world->combineSlots.ptr) + static_cast<int64_t>(r) * slotsStride;
        red.rowBytes = rowBytes;
        red.inverseTagged = meta;
        red.epoch = epoch;
        red.orderKeys = memoryRoute ? nullptr : meta + n;
        red.expertScales = memoryRoute ? rp.expertScales : nullptr;
        red.tokenMask = memoryRoute ? reinterpret_cast<const uint8_t *>(rp.xActiveMask) : nullptr;
        red.sharedExpertX = memoryRoute ? rp.sharedExpertX : nullptr;
        red.reduceKind = memoryRoute ? kReduceFp32 : kReducePerAdd;
        red.commQuant = memoryRoute ? static_cast<int>(rp.quantMode) : 0;
        red.bf16 = rp.dtype == TileXR::TILEXR_DATA_TYPE_BFP16;
        red.bs = rp.bs;
        red.h = rp.h;
        red.topK = rp.topK;
        red.sharedSlots = shared;
        red.y = rp.yOut;
        red.numComputeUnits = world->numComputeUnits;
        red.stream = rs;
        if (status == kOk) {
            status = Timed(rc, kKernelReduce, rs, "reduce", [&] { return LaunchReduce(red); });
        }
        if (status == kOk) {
            if (hipEventRecord(ev.drained, rs) != hipSuccess) {
                status = TileXR::TILEXR_ERROR_INTERNAL;
            }
            ev.drainedArmed = true;
        }
    }
    for (PendingCombine &pc : world->pendingCombine) {
        pc.present = false;
    }
    return status;
}

} // namespace TileXREp
