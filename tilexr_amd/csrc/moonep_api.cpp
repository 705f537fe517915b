// Host side of the plan-driven (MoonEP) Dispatch and Combine stages: the C entry points, argument validation in the
// reference's order, and the ordering of the kernels of all logical ranks that share the device.
//
// The reference runs one process per rank and lets its kernels meet at magic-tagged barriers in each other's peer
// windows (src/moonep/dispatch/kernels/tilexr_moonep_dispatch_kernel.cpp:108-147).  With every rank in one process on
// one device the host orders the exchange instead: a call records what its rank asked for; when the last rank of the
// world has called, every rank's kernels are enqueued on that rank's own stream, with events where one rank's kernels
// read or write what another rank's kernels produced.  A rank's outputs are therefore complete once every rank has
// made the call and the rank's stream has been synchronised.
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
    const int64_t stride = (rows + kRowsPerGroup - 1) / kRowsPerGroup * kRowsPerGroup;
    const int64_t groups = stride / kRowsPerGroup;
    const int64_t perRank8 = stride * 8;
    // six 8-byte tables, two 4-byte tables, then the per-rank words
    const int64_t bytes = world * (6 * perRank8 + 2 * stride * 4) + world * 8 + world * groups * 4 + 256;
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
    out->dupMask = reinterpret_cast<uint64_t *>(take(world * perRank8));
    out->groupOf = reinterpret_cast<uint64_t *>(take(world * perRank8));
    out->slotSrc = reinterpret_cast<uint64_t *>(take(world * perRank8));
    out->fail = reinterpret_cast<uint64_t *>(take(world * 8));
    out->sibling = reinterpret_cast<uint32_t *>(take(world * stride * 4));
    out->workList = reinterpret_cast<int32_t *>(take(world * stride * 4));
    out->workCount = reinterpret_cast<int32_t *>(take(world * groups * 4));
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

// Every stream first waits for what the previous exchange left running on any stream of the world: the tables are
// shared, and a kernel of this exchange must not overwrite an entry a kernel of the last one has yet to read.
int WaitForPreviousExchange(WorldState *st, const std::vector<StageCall> &calls)
{
    for (const StageCall &c : calls) {
        for (RankEvents &e : st->events) {
            if (e.doneArmed) {
                MOON_TRY(hipStreamWaitEvent(c.stream, e.done, 0), "waiting for the previous exchange");
            }
        }
    }
    return kOk;
}

int LaunchDispatchWorld(EpWorld *world, WorldState *st)
{
    const int R = world->rankSize;
    const std::vector<StageCall> &calls = st->dispatch;
    const StageCall &shape = calls[0];
    WorldTables tables {};
    uint64_t epoch = 0;
    if (!PrepareTables(st, R, shape.nvS, shape.s * shape.k, &tables) || !NextEpoch(st, &epoch)) {
        return TILEXR_MOONEP_ERROR_INTERNAL;
    }
    int ret = WaitForPreviousExchange(st, calls);
    if (ret != kOk) {
        return ret;
    }
    const bool fresh = (shape.flags & TILEXR_MOONEP_FLAG_BUILD_DEDUP) != 0;
    ReceiveTable out {};
    for (int q = 0; q < R; ++q) {
        out.hidden[q] = calls[static_cast<size_t>(q)].hiddenNvsh;
        out.weights[q] = calls[static_cast<size_t>(q)].weightsNvs;
    }
    for (int s = 0; s < R; ++s) {
        const StageCall &c = calls[static_cast<size_t>(s)];
        // rows go straight into the other ranks' receive tensors: not before those ranks' streams have reached the call
        for (int q = 0; q < R; ++q) {
            if (q != s) {
                MOON_TRY(hipStreamWaitEvent(c.stream, st->events[static_cast<size_t>(q)].arrived, 0), "waiting for a peer's call");
            }
        }
        ScatterLaunch l {};
        l.dst = c.dst;
        l.hiddenSh = c.hiddenSh;
        l.weightsSk = c.weightsSk;
        l.s = c.s;
        l.k = c.k;
        l.h = c.h;
        l.nvS = c.nvS;
        l.world = R;
        l.srcRank = s;
        l.fresh = fresh;
        l.out = out;
        l.tables = tables;
        l.epoch = epoch;
        l.stream = c.stream;
        MOON_TRY(LaunchMoonScatter(l), "launching the scatter kernel");
        MOON_TRY(hipEventRecord(st->events[static_cast<size_t>(s)].sent, c.stream), "recording an event");
    }
    for (int q = 0; q < R; ++q) {
        const StageCall &c = calls[static_cast<size_t>(q)];
        for (int s = 0; s < R; ++s) {
            if (s != q) {
                MOON_TRY(hipStreamWaitEvent(c.stream, st->events[static_cast<size_t>(s)].sent, 0), "waiting for a peer's rows");
            }
        }
        if (fresh) {
            DedupBuildLaunch b {};
            b.nvS = c.nvS;
            b.rank = q;
            b.tables = tables;
            b.epoch = epoch;
            b.dupGroups = c.dupGroups;
            b.dupLoffs = c.dupLoffs;
            b.dupCounts = c.dupCounts;
            b.stream = c.stream;
            MOON_TRY(LaunchMoonDedupBuild(b), "launching the duplicate-plan kernel");
        } else {
            GroupWalkLaunch w {};
            w.nvS = c.nvS;
            w.rank = q;
            w.combine = false;
            w.dupGroups = c.dupGroups;
            w.dupLoffs = c.dupLoffs;
            w.dupCounts = c.dupCounts;
            w.tables = tables;
            w.epoch = epoch;
            w.stream = c.stream;
            MOON_TRY(LaunchMoonGroupWalk(w), "launching the group-walk kernel");
        }
        FillLaunch f {};
        f.nvS = c.nvS;
        f.h = c.h;
        f.world = R;
        f.rank = q;
        f.expand = !fresh;
        f.hiddenNvsh = c.hiddenNvsh;
        f.weightsNvs = c.weightsNvs;
        f.tables = tables;
        f.epoch = epoch;
        f.status = c.status;
        f.stream = c.stream;
        MOON_TRY(LaunchMoonFill(f), "launching the fill kernels");
        MOON_TRY(hipEventRecord(st->events[static_cast<size_t>(q)].done, c.stream), "recording an event");
        st->events[static_cast<size_t>(q)].doneArmed = true;
    }
    return kOk;
}

int LaunchCombineWorld(EpWorld *world, WorldState *st)
{
    const int R = world->rankSize;
    const std::vector<StageCall> &calls = st->combine;
    const StageCall &shape = calls[0];
    WorldTables tables {};
    uint64_t epoch = 0;
    if (!PrepareTables(st, R, shape.nvS, shape.s * shape.k, &tables) || !NextEpoch(st, &epoch)) {
        return TILEXR_MOONEP_ERROR_INTERNAL;
    }
    int ret = WaitForPreviousExchange(st, calls);
    if (ret != kOk) {
        return ret;
    }
    SourceTable src {};
    for (int q = 0; q < R; ++q) {
        const StageCall &c = calls[static_cast<size_t>(q)];
        src.hidden[q] = c.hiddenNvsh;
        src.weights[q] = c.weightsNvs;
        src.dupGroups[q] = c.dupGroups;
        src.dupLoffs[q] = c.dupLoffs;
    }
    for (int q = 0; q < R; ++q) {
        const StageCall &c = calls[static_cast<size_t>(q)];
        GroupWalkLaunch w {};
        w.nvS = c.nvS;
        w.rank = q;
        w.combine = true;
        w.dupGroups = c.dupGroups;
        w.dupLoffs = c.dupLoffs;
        w.dupCounts = c.dupCounts;
        w.tables = tables;
        w.epoch = epoch;
        w.stream = c.stream;
        MOON_TRY(LaunchMoonGroupWalk(w), "launching the group-walk kernel");
        ReverseLaunch r {};
        r.dstLocal = c.dstLocal;
        r.nvS = c.nvS;
        r.n = c.s * c.k;
        r.world = R;
        r.rank = q;
        r.tables = tables;
        r.epoch = epoch;
        r.stream = c.stream;
        MOON_TRY(LaunchMoonReverse(r), "launching the reverse-route kernel");
        MOON_TRY(hipEventRecord(st->events[static_cast<size_t>(q)].sent, c.stream), "recording an event");
    }
    for (int p = 0; p < R; ++p) {
        const StageCall &c = calls[static_cast<size_t>(p)];
        // covers both the slot table and the expert ranks' tensors: `sent` follows the expert rank's call on its stream
        for (int q = 0; q < R; ++q) {
            if (q != p) {
                MOON_TRY(hipStreamWaitEvent(c.stream, st->events[static_cast<size_t>(q)].sent, 0), "waiting for a peer's slots");
            }
        }
        MoonReduceLaunch l {};
        l.s = c.s;
        l.k = c.k;
        l.h = c.h;
        l.nvS = c.nvS;
        l.world = R;
        l.rank = p;
        l.src = src;
        l.tables = tables;
        l.epoch = epoch;
        l.hiddenSh = c.hiddenShOut;
        l.weightsSk = c.weightsSkOut;
        l.status = c.status;
        l.numComputeUnits = world->numComputeUnits;
        l.stream = c.stream;
        MOON_TRY(LaunchMoonReduce(l), "launching the reduce kernel");
        MOON_TRY(hipEventRecord(st->events[static_cast<size_t>(p)].done, c.stream), "recording an event");
        st->events[static_cast<size_t>(p)].doneArmed = true;
    }
    return kOk;
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
            return kInvalid;
        }
    }
    RankEvents &ev = st->events[static_cast<size_t>(comm->rank)];
    if (!EnsureEvent(&ev.arrived) || !EnsureEvent(&ev.sent) || !EnsureEvent(&ev.done)) {
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
        for (hipEvent_t ev : {e.arrived, e.sent, e.done}) {
            if (ev != nullptr) {
                (void)hipEventDestroy(ev);
            }
        }
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
