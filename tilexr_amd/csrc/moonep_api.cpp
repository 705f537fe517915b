// Host side of the plan-driven (MoonEP) Dispatch and Combine stages: the C entry points, argument validation in the
// reference's order, and the ordering of the exchange among the logical ranks that share the device.
//
// The reference runs one process per rank and lets its kernels meet at magic-tagged barriers in each other's peer
// windows (src/moonep/dispatch/kernels/tilexr_moonep_dispatch_kernel.cpp:108-147).  With every rank in one process on
// one device the host orders the exchange instead: a call records what its rank asked for; when the last rank of the
// world has called, the kernels -- each launched once for all ranks -- are enqueued on the world's own stream behind an
// event of every rank's stream, and every rank's stream then waits for the end of the exchange.  A rank's outputs are
// therefore complete once every rank has made the call and the rank's stream has been synchronised.  A world of one
// rank runs directly on the caller's stream.
#include <cstddef>
#include <limits>
#include <mutex>
#include <vector>

#include <hip/hip_runtime_api.h>

#include "ep_context.h"
#include "ep_run_common.h"
#include "moonep_host.h"
#include "moonep_stage.h"
#include "tilexr_moonep.h"

namespace TileXRMoon {

using TileXREp::EpComm;
using TileXREp::EpWorld;

namespace {

constexpr int kOk = TILEXR_MOONEP_SUCCESS;
constexpr int kInvalid = TILEXR_MOONEP_ERROR_INVALID_ARGUMENT;

bool CheckedMul(uint64_t a, uint64_t b, uint64_t *out)
{
    if (a != 0 && b > std::numeric_limits<uint64_t>::max() / a) {
        return false;
    }
    *out = a * b;
    return true;
}

// reference: src/moonep/common/moonep_stage_layout.h:51-72
bool TensorHeaderValid(const TileXRMoonEpTensorV1 *t)
{
    if (t == nullptr || t->structSize < sizeof(*t) || t->abiVersion != TILEXR_MOONEP_ABI_VERSION_V1 || t->data == nullptr ||
        t->rank == 0 || t->rank > TILEXR_MOONEP_MAX_TENSOR_RANK || t->elementCount == 0) {
        return false;
    }
    uint64_t elements = 1;
    for (uint32_t d = 0; d < TILEXR_MOONEP_MAX_TENSOR_RANK; ++d) {
        if (d < t->rank) {
            if (t->shape[d] <= 0 || !CheckedMul(elements, static_cast<uint64_t>(t->shape[d]), &elements)) {
                return false;
            }
        } else if (t->shape[d] != 0) {
            return false;
        }
    }
    return elements == t->elementCount;
}

// reference: src/moonep/common/moonep_stage_layout.h:74-99
bool PlanValid(int64_t commRank, int64_t commWorld, const TileXRMoonEpPlanV1 *p, int64_t *s)
{
    if (p == nullptr || p->structSize < sizeof(*p) || p->abiVersion != TILEXR_MOONEP_ABI_VERSION_V1 || commWorld <= 0 ||
        commWorld > 128 || commRank < 0 || commRank >= commWorld || p->n <= 0 || p->r != commWorld || p->e <= 0 ||
        p->b <= 0 || p->nvS < p->n || p->k <= 0 || p->k > kMaxTopK || p->n % p->k != 0 || p->e % p->r != 0 ||
        p->b > p->e / p->r || p->dst == nullptr || p->e > std::numeric_limits<int64_t>::max() - p->b ||
        p->expertsToCopy == nullptr || p->zeroFillRanges == nullptr || p->remoteStats == nullptr ||
        p->dupGroups == nullptr || p->dupLoffs == nullptr || p->dupCounts == nullptr || p->status == nullptr) {
        return false;
    }
    uint64_t encodedCapacity = 0;
    if (!CheckedMul(static_cast<uint64_t>(p->r), static_cast<uint64_t>(p->nvS), &encodedCapacity) ||
        encodedCapacity > static_cast<uint64_t>(std::numeric_limits<int32_t>::max()) + 1u) {
        return false;
    }
    *s = p->n / p->k;
    return *s > 0;
}

// reference: src/moonep/dispatch/host/dispatch_layout.cpp:12-23, src/moonep/combine/host/combine_layout.cpp:13-23
bool HiddenPairValid(const TileXRMoonEpTensorV1 *in, const TileXRMoonEpTensorV1 *out, int64_t inRows, int64_t outRows)
{
    return TensorHeaderValid(in) && TensorHeaderValid(out) && in->dtype == TILEXR_MOONEP_DTYPE_BFLOAT16 &&
        out->dtype == TILEXR_MOONEP_DTYPE_BFLOAT16 && in->rank == 2 && out->rank == 2 && in->shape[0] == inRows &&
        in->shape[1] > 0 && out->shape[0] == outRows && out->shape[1] == in->shape[1] &&
        in->shape[1] <= std::numeric_limits<int32_t>::max() / 2;
}

// reference: dispatch_layout.cpp:25-36 (sk -> nvs) and combine_layout.cpp:25-37 (nvs -> sk)
bool WeightsPairValid(const TileXRMoonEpTensorV1 *sk, const TileXRMoonEpTensorV1 *nvs, int64_t s, int64_t k, int64_t nvS)
{
    if (sk == nullptr || nvs == nullptr) {
        return sk == nullptr && nvs == nullptr;
    }
    return TensorHeaderValid(sk) && TensorHeaderValid(nvs) && sk->dtype == TILEXR_MOONEP_DTYPE_FLOAT32 &&
        nvs->dtype == TILEXR_MOONEP_DTYPE_FLOAT32 && sk->rank == 2 && sk->shape[0] == s && sk->shape[1] == k &&
        nvs->rank == 1 && nvs->shape[0] == nvS;
}

// reference: src/moonep/common/moonep_stage_host.h:14-21
bool LocalityValid(const TileXR::CommArgs &a)
{
    return a.rankSize > 0 && a.rankSize <= TileXR::TILEXR_MAX_RANK_SIZE && a.rank >= 0 && a.rank < a.rankSize &&
        a.localRankSize > 0 && a.localRankSize <= a.rankSize && a.rankSize % a.localRankSize == 0 && a.localRank >= 0 &&
        a.localRank < a.localRankSize;
}

void FillCommon(StageCall *call, const TileXRMoonEpPlanV1 *plan, int64_t s, int64_t h, uint64_t flags, hipStream_t stream)
{
    call->present = true;
    call->stream = stream;
    call->s = s;
    call->k = plan->k;
    call->h = h;
    call->nvS = plan->nvS;
    call->flags = flags;
    call->dst = static_cast<const int32_t *>(plan->dst);
    call->dupGroups = static_cast<int32_t *>(plan->dupGroups);
    call->dupLoffs = static_cast<int32_t *>(plan->dupLoffs);
    call->dupCounts = static_cast<int32_t *>(plan->dupCounts);
    call->status = static_cast<int32_t *>(plan->status);
}

bool EnsureEvent(hipEvent_t *e)
{
    return *e != nullptr || hipEventCreateWithFlags(e, hipEventDisableTiming) == hipSuccess;
}

int Internal(hipError_t err, const char *what)
{
    if (err == hipSuccess) {
        return kOk;
    }
    std::fprintf(stderr, "tilexr-moonep: %s failed: %s\n", what, hipGetErrorString(err));
    return TILEXR_MOONEP_ERROR_INTERNAL;
}

#define MOON_TRY(expr, what)                      \
    do {                                          \
        const int moonTryRet = Internal((expr), (what)); \
        if (moonTryRet != kOk) {                  \
            return moonTryRet;                    \
        }                                         \
    } while (0)

// Sizes the world's per-row tables for this shape and returns views into them.  Entries carry their epoch, so a
// change of layout needs no clearing: whatever an older call left behind has an older epoch.
bool PrepareTables(WorldState *st, int world, int64_t nvS, int64_t n, WorldTables *out)
{
    const int64_t rows = nvS > n ? nvS : n;
    const int64_t stride = (rows + kTableAlign - 1) / kTableAlign * kTableAlign;
    const int64_t groups = (rows + kChunkRows - 1) / kChunkRows;
    const int64_t perRank8 = stride * 8;
    // six 8-byte tables, two 4-byte tables, then the per-rank words
    const int64_t bytes = world * (6 * perRank8 + 2 * stride * 4 + stride) + world * 8 + world * groups * 8 + 256;
    if (!st->tables.Reserve(static_cast<size_t>(bytes), true)) {
        return false;
    }
    char *p = static_cast<char *>(st->tables.ptr);
    auto take = [&p](int64_t size) {
        char *at = p;
        p += size;
        return at;
    };
    out->rowTag = reinterpret_cast<uint64_t *>(take(world * perRank8));
    out->parentTag = reinterpret_cast<uint64_t *>(take(world * perRank8));
    out->groupStart = reinterpret_cast<uint64_t *>(take(world * perRank8));
    out->slotSrc = reinterpret_cast<uint64_t *>(take(world * perRank8));
    out->slotDup = reinterpret_cast<uint64_t *>(take(world * perRank8));
    out->slotGroup = reinterpret_cast<uint64_t *>(take(world * perRank8));
    out->fail = reinterpret_cast<uint64_t *>(take(world * 8));
    out->sibling = reinterpret_cast<uint32_t *>(take(world * stride * 4));
    out->slotCount = reinterpret_cast<int32_t *>(take(world * stride * 4));
    out->chunkTotals = reinterpret_cast<int32_t *>(take(world * groups * 8));
    out->direct = reinterpret_cast<uint8_t *>(take(world * stride));
    out->stride = stride;
    out->groupStride = groups;
    return true;
}

// One epoch per exchange.  The tag is 32 bits wide: when the counter's low word comes round to zero the tables are
// cleared once, so a tag of 2^32 calls ago can never be taken for a fresh one.
bool NextEpoch(WorldState *st, uint64_t *epoch)
{
    ++st->epochCounter;
    if ((st->epochCounter & 0xffffffffull) == 0) {
        if (st->tables.ptr != nullptr &&
            (hipDeviceSynchronize() != hipSuccess || hipMemset(st->tables.ptr, 0, st->tables.bytes) != hipSuccess ||
                hipDeviceSynchronize() != hipSuccess)) {
            return false;
        }
        ++st->epochCounter;
    }
    *epoch = st->epochCounter & 0xffffffffull;
    return true;
}

WorldState *StateOf(EpWorld *world)
{
    if (world->moon == nullptr) {
        WorldState *st = new WorldState();
        st->dispatch.resize(static_cast<size_t>(world->rankSize));
        st->combine.resize(static_cast<size_t>(world->rankSize));
        st->events.resize(static_cast<size_t>(world->rankSize));
        world->moon = st;
    }
    return world->moon;
}

bool AllPresent(const std::vector<StageCall> &calls)
{
    for (const StageCall &c : calls) {
        if (!c.present) {
            return false;
        }
    }
    return true;
}

bool SameShape(const StageCall &a, const StageCall &b)
{
    return a.s == b.s && a.k == b.k && a.h == b.h && a.nvS == b.nvS && a.flags == b.flags &&
        (a.weightsSk != nullptr) == (b.weightsSk != nullptr);
}

// The stream the exchange runs on, and what it has to wait for first.  A one-rank world runs on the caller's stream.  A
// larger world runs on a stream of its own that waits until every rank's stream has reached its call (`arrived`): the
// kernels read and write all ranks' tensors.  Either way the stream also waits for the previous exchange of the world,
// whose kernels may still be reading the shared tables.
int BeginExchange(EpWorld *world, WorldState *st, const std::vector<StageCall> &calls, hipStream_t *stream)
{
    const int R = world->rankSize;
    if (R == 1) {
        *stream = calls[0].stream;
    } else {
        if (st->stream == nullptr) {
            MOON_TRY(hipStreamCreateWithFlags(&st->stream, hipStreamNonBlocking), "creating the world's stream");
        }
        *stream = st->stream;
        for (int r = 0; r < R; ++r) {
            MOON_TRY(hipStreamWaitEvent(*stream, st->events[static_cast<size_t>(r)].arrived, 0), "waiting for a rank's call");
        }
    }
    if (st->doneArmed) {
        MOON_TRY(hipStreamWaitEvent(*stream, st->done, 0), "waiting for the previous exchange");
    }
    return kOk;
}

// Marks the end of the exchange and makes every rank's stream wait for it.
int EndExchange(EpWorld *world, WorldState *st, const std::vector<StageCall> &calls, hipStream_t stream)
{
    if (st->done == nullptr) {
        MOON_TRY(hipEventCreateWithFlags(&st->done, hipEventDisableTiming), "creating an event");
    }
    MOON_TRY(hipEventRecord(st->done, stream), "recording an event");
    st->doneArmed = true;
    if (world->rankSize > 1) {
        for (const StageCall &c : calls) {
            MOON_TRY(hipStreamWaitEvent(c.stream, st->done, 0), "waiting for the exchange");
        }
    }
    return kOk;
}

// Timing events and kernel names are a measurement aid of rank 0's communicator (TileXREpSetKernelTimingEvents): the
// launch they bracket covers every rank of the world.
LaunchTiming TimingOf(EpWorld *world, int kernel)
{
    EpComm *c = world->comms[0];
    std::lock_guard<std::mutex> lock(c->mu);
    LaunchTiming t;
    t.start = c->timing[kernel][0];
    t.stop = c->timing[kernel][1];
    return t;
}

void NoteKernel(EpWorld *world, int kernel, const char *name)
{
    for (EpComm *c : world->comms) {
        std::lock_guard<std::mutex> lock(c->mu);
        c->lastKernel[kernel] = name;
    }
}

int LaunchDispatchWorld(EpWorld *world, WorldState *st)
{
    const int R = world->rankSize;
    const std::vector<StageCall> &calls = st->dispatch;
    const StageCall &shape = calls[0];
    DispatchWorld w {};
    if (!PrepareTables(st, R, shape.nvS, shape.s * shape.k, &w.tables) || !NextEpoch(st, &w.epoch)) {
        return TILEXR_MOONEP_ERROR_INTERNAL;
    }
    w.world = R;
    w.s = shape.s;
    w.k = shape.k;
    w.h = shape.h;
    w.nvS = shape.nvS;
    w.fresh = (shape.flags & TILEXR_MOONEP_FLAG_BUILD_DEDUP) != 0;
    for (int r = 0; r < R; ++r) {
        const StageCall &c = calls[static_cast<size_t>(r)];
        w.dst[r] = c.dst;
        w.hiddenSh[r] = c.hiddenSh;
        w.weightsSk[r] = c.weightsSk;
        w.hiddenNvsh[r] = c.hiddenNvsh;
        w.weightsNvs[r] = c.weightsNvs;
        w.dupGroups[r] = c.dupGroups;
        w.dupLoffs[r] = c.dupLoffs;
        w.dupCounts[r] = c.dupCounts;
        w.status[r] = c.status;
    }
    hipStream_t stream = nullptr;
    int ret = BeginExchange(world, st, calls, &stream);
    if (ret != kOk) {
        return ret;
    }
    MOON_TRY(LaunchMoonDispatch(w, stream, TimingOf(world, TileXREp::kKernelScatter)), "launching the dispatch kernels");
    NoteKernel(world, TileXREp::kKernelScatter, MoonScatterKernelName());
    return EndExchange(world, st, calls, stream);
}

int LaunchCombineWorld(EpWorld *world, WorldState *st)
{
    const int R = world->rankSize;
    const std::vector<StageCall> &calls = st->combine;
    const StageCall &shape = calls[0];
    CombineWorld w {};
    if (!PrepareTables(st, R, shape.nvS, shape.s * shape.k, &w.tables) || !NextEpoch(st, &w.epoch)) {
        return TILEXR_MOONEP_ERROR_INTERNAL;
    }
    w.world = R;
    w.s = shape.s;
    w.k = shape.k;
    w.h = shape.h;
    w.nvS = shape.nvS;
    for (int r = 0; r < R; ++r) {
        const StageCall &c = calls[static_cast<size_t>(r)];
        w.dstLocal[r] = c.dstLocal;
        w.hiddenNvsh[r] = c.hiddenNvsh;
        w.weightsNvs[r] = c.weightsNvs;
        w.dupGroups[r] = c.dupGroups;
        w.dupLoffs[r] = c.dupLoffs;
        w.dupCounts[r] = c.dupCounts;
        w.hiddenSh[r] = c.hiddenShOut;
        w.weightsSk[r] = c.weightsSkOut;
        w.status[r] = c.status;
    }
    hipStream_t stream = nullptr;
    int ret = BeginExchange(world, st, calls, &stream);
    if (ret != kOk) {
        return ret;
    }
    MOON_TRY(LaunchMoonCombine(w, stream, TimingOf(world, TileXREp::kKernelReduce)), "launching the combine kernels");
    NoteKernel(world, TileXREp::kKernelReduce, MoonReduceKernelName());
    return EndExchange(world, st, calls, stream);
}

// Files one rank's call; the last rank of the world to arrive enqueues the whole exchange.
int Arrive(EpComm *comm, const StageCall &call, bool combine)
{
    EpWorld *world = comm->world;
    if (!world->deviceReady) {
        return TILEXR_MOONEP_ERROR_INTERNAL;    // no peer windows (reference: moonep_stage_host.h:55-58)
    }
    if (world->rankSize > kMaxWorld) {
        return TILEXR_MOONEP_ERROR_NOT_SUPPORTED;
    }
    std::lock_guard<std::mutex> lock(world->mu);
    for (int r = 0; r < world->rankSize; ++r) {
        if (world->comms[static_cast<size_t>(r)] == nullptr) {
            return TileXR::TILEXR_ERROR_NOT_INITIALIZED;
        }
    }
    WorldState *st = StateOf(world);
    std::vector<StageCall> &calls = combine ? st->combine : st->dispatch;
    StageCall &mine = calls[static_cast<size_t>(comm->rank)];
    if (mine.present) {
        return TILEXR_MOONEP_ERROR_INTERNAL;    // this rank already has a call of this stage waiting for its peers
    }
    for (const StageCall &c : calls) {
        if (c.present && !SameShape(c, call)) {
            // The world cannot run this exchange.  The calls already filed for it are dropped, each with this rank
            // named in its device status as the peer that failed (what a peer's bad plan leaves there in the
            // reference: src/moonep/dispatch/kernels/tilexr_moonep_dispatch_kernel.cpp:512,
            // src/moonep/combine/kernels/tilexr_moonep_combine_kernel.cpp:423), so that the world is usable again.
            const int32_t failure = (combine ? kCombineRemoteFailureBase : kDispatchRemoteFailureBase) + comm->rank;
            for (StageCall &waiting : calls) {
                if (waiting.present && waiting.status != nullptr) {
                    (void)LaunchMoonStatus(waiting.status, failure, waiting.stream);
                }
                waiting.present = false;
            }
            return kInvalid;
        }
    }
    RankEvents &ev = st->events[static_cast<size_t>(comm->rank)];
    if (!EnsureEvent(&ev.arrived)) {
        return TILEXR_MOONEP_ERROR_INTERNAL;
    }
    (void)comm->nextMagic.fetch_add(1);         // one magic per launch, as in the reference (moonep_stage_host.h:75-83)
    if (world->rankSize > 1) {
        MOON_TRY(hipEventRecord(ev.arrived, call.stream), "recording an event");
    }
    mine = call;
    if (!AllPresent(calls)) {
        return kOk;
    }
    const int ret = combine ? LaunchCombineWorld(world, st) : LaunchDispatchWorld(world, st);
    for (StageCall &c : calls) {
        c.present = false;
    }
    return ret;
}

} // namespace

void ReleaseWorldState(WorldState *st)
{
    if (st == nullptr) {
        return;
    }
    st->tables.Release();
    for (RankEvents &e : st->events) {
        if (e.arrived != nullptr) {
            (void)hipEventDestroy(e.arrived);
        }
    }
    if (st->done != nullptr) {
        (void)hipEventDestroy(st->done);
    }
    if (st->stream != nullptr) {
        (void)hipStreamDestroy(st->stream);
    }
    delete st;
}

// reference: src/moonep/host/tilexr_moonep.cpp:300-320, src/moonep/dispatch/host/dispatch_host.cpp:9-60,
// src/moonep/dispatch/host/dispatch_layout.cpp:45-76
int ValidateDispatch(const TileXRMoonEpDispatchArgsV1 *args, aclrtStream stream, EpComm **commOut, StageCall *call)
{
    const size_t legacyBytes = offsetof(TileXRMoonEpDispatchArgsV1, registeredWorkspace);
    const size_t workspaceBytes = offsetof(TileXRMoonEpDispatchArgsV1, trace);
    if (args != nullptr && args->structSize >= workspaceBytes &&
        (args->registeredWorkspace != nullptr || args->registeredWorkspaceBytes != 0)) {
        return TILEXR_MOONEP_ERROR_NOT_SUPPORTED;     // the registered-workspace variant needs a second device
    }
    if (args != nullptr && args->structSize >= sizeof(*args) && args->trace != nullptr) {
        return kInvalid;
    }
    if (args == nullptr || args->structSize < legacyBytes || args->abiVersion != TILEXR_MOONEP_ABI_VERSION_V1 ||
        args->comm == nullptr || args->plan == nullptr || args->hiddenSh == nullptr || args->hiddenNvsh == nullptr ||
        stream == nullptr) {
        return kInvalid;
    }
    if ((args->flags & TILEXR_MOONEP_FLAG_ZERO_COPY) != 0) {
        return TILEXR_MOONEP_ERROR_NOT_SUPPORTED;
    }
    EpComm *comm = TileXREp::LookupComm(args->comm);
    if (comm == nullptr) {
        return TileXR::TILEXR_ERROR_NOT_INITIALIZED;
    }
    if (!LocalityValid(comm->host)) {
        return kInvalid;
    }
    const uint64_t allowed = TILEXR_MOONEP_FLAG_BUILD_DEDUP | TILEXR_MOONEP_FLAG_SKIP_INTER_RANK_SYNC;
    int64_t s = 0;
    if ((args->flags & ~allowed) != 0 || !PlanValid(comm->host.rank, comm->host.rankSize, args->plan, &s) ||
        !HiddenPairValid(args->hiddenSh, args->hiddenNvsh, s, args->plan->nvS) ||
        !WeightsPairValid(args->routeWeightsSk, args->routeWeightsNvs, s, args->plan->k, args->plan->nvS)) {
        return kInvalid;
    }
    FillCommon(call, args->plan, s, args->hiddenSh->shape[1], args->flags & TILEXR_MOONEP_FLAG_BUILD_DEDUP,
        static_cast<hipStream_t>(stream));
    call->hiddenSh = args->hiddenSh->data;
    call->weightsSk = args->routeWeightsSk == nullptr ? nullptr : static_cast<const float *>(args->routeWeightsSk->data);
    call->hiddenNvsh = args->hiddenNvsh->data;
    call->weightsNvs = args->routeWeightsNvs == nullptr ? nullptr : static_cast<float *>(args->routeWeightsNvs->data);
    *commOut = comm;
    return kOk;
}

// reference: src/moonep/combine/host/combine_host.cpp:7-58, src/moonep/combine/host/combine_layout.cpp:101-120
int ValidateCombine(const TileXRMoonEpCombineArgsV1 *args, aclrtStream stream, EpComm **commOut, StageCall *call)
{
    if (args == nullptr || args->structSize < sizeof(*args) || args->abiVersion != TILEXR_MOONEP_ABI_VERSION_V1 ||
        args->comm == nullptr || args->plan == nullptr || args->dstLocal == nullptr || args->hiddenNvsh == nullptr ||
        args->hiddenSh == nullptr || stream == nullptr) {
        return kInvalid;
    }
    if ((args->flags & TILEXR_MOONEP_FLAG_ZERO_COPY) != 0) {
        return TILEXR_MOONEP_ERROR_NOT_SUPPORTED;
    }
    EpComm *comm = TileXREp::LookupComm(args->comm);
    if (comm == nullptr) {
        return TileXR::TILEXR_ERROR_NOT_INITIALIZED;
    }
    if (!LocalityValid(comm->host)) {
        return kInvalid;
    }
    int64_t s = 0;
    if (args->flags != TILEXR_MOONEP_FLAG_NONE || !PlanValid(comm->host.rank, comm->host.rankSize, args->plan, &s) ||
        !HiddenPairValid(args->hiddenNvsh, args->hiddenSh, args->plan->nvS, s) ||
        !WeightsPairValid(args->routeWeightsSk, args->routeWeightsNvs, s, args->plan->k, args->plan->nvS)) {
        return kInvalid;
    }
    FillCommon(call, args->plan, s, args->hiddenNvsh->shape[1], 0, static_cast<hipStream_t>(stream));
    call->dstLocal = args->dstLocal;
    call->hiddenNvsh = args->hiddenNvsh->data;
    call->weightsNvs = args->routeWeightsNvs == nullptr ? nullptr : static_cast<float *>(args->routeWeightsNvs->data);
    call->weightsSk = call->weightsNvs;      // only its presence is compared between ranks
    call->hiddenShOut = args->hiddenSh->data;
    call->weightsSkOut = args->routeWeightsSk == nullptr ? nullptr : static_cast<float *>(args->routeWeightsSk->data);
    *commOut = comm;
    return kOk;
}

} // namespace TileXRMoon

extern "C" {

uint32_t TileXRMoonEpGetAbiVersion(void)
{
    return TILEXR_MOONEP_ABI_VERSION_V2;
}

int TileXRMoonEpGetCapabilitiesV1(uint64_t *nativeStages, uint64_t *stubStages)
{
    if (nativeStages == nullptr || stubStages == nullptr) {
        return TILEXR_MOONEP_ERROR_INVALID_ARGUMENT;
    }
    *nativeStages = static_cast<uint64_t>(TILEXR_MOONEP_STAGE_DISPATCH) | static_cast<uint64_t>(TILEXR_MOONEP_STAGE_COMBINE);
    *stubStages = 0;
    return TILEXR_MOONEP_SUCCESS;
}

int TileXRMoonEpGetCapabilitiesV2(uint64_t *nativeStages, uint64_t *stubStages)
{
    return TileXRMoonEpGetCapabilitiesV1(nativeStages, stubStages);
}

int64_t TileXRMoonEpSetCachedRowBytes(int64_t bytes)
{
    return TileXRMoon::SetCachedRowBytes(bytes);
}

int TileXRMoonEpDispatchV1(const TileXRMoonEpDispatchArgsV1 *args, aclrtStream stream)
{
    TileXREp::EpComm *comm = nullptr;
    TileXRMoon::StageCall call {};
    const int ret = TileXRMoon::ValidateDispatch(args, stream, &comm, &call);
    if (ret != TILEXR_MOONEP_SUCCESS) {
        return ret;
    }
    return TileXRMoon::Arrive(comm, call, false);
}

int TileXRMoonEpCombineV1(const TileXRMoonEpCombineArgsV1 *args, aclrtStream stream)
{
    TileXREp::EpComm *comm = nullptr;
    TileXRMoon::StageCall call {};
    const int ret = TileXRMoon::ValidateCombine(args, stream, &comm, &call);
    if (ret != TILEXR_MOONEP_SUCCESS) {
        return ret;
    }
    return TileXRMoon::Arrive(comm, call, true);
}

}
