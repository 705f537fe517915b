// Plain-C access to the host-side arithmetic and rules, for callers (tests, sizing tools) that cannot include the
// C++ headers.  Every hook forwards to the function of the same purpose in ep_host.h; nothing here touches the GPU.
#include <cstring>

#include "ep_host.h"
#include "hooks.h"

#include <algorithm>
#include <atomic>
#include <random>
#include <thread>
#include <vector>

#include "ep_tile_publish.h"

using namespace TileXREp;

namespace {

void *Fake(bool present, uintptr_t where)
{
    return present ? reinterpret_cast<void *>(where) : nullptr;
}

TileXR::CommArgs MakeComm(const TileXREpHookComm &c)
{
    TileXR::CommArgs args {};
    args.rank = c.rank;
    args.localRank = c.rank;
    args.rankSize = c.rankSize;
    args.localRankSize = c.localRankSize;
    args.extraFlag = c.extraFlag;
    for (int r = 0; r < c.rankSize && r < TileXR::TILEXR_MAX_RANK_SIZE; ++r) {
        args.peerMems[r] = r == c.nullPeer ? nullptr : reinterpret_cast<GM_ADDR>(0x10000000ull + 0x1000000ull * r);
    }
    if (c.hasUdma) {
        args.udmaInfoPtr = reinterpret_cast<GM_ADDR>(0x30000000ull);
        args.udmaRegistryPtr = reinterpret_cast<GM_ADDR>(0x40000000ull);
    }
    return args;
}

EpDispatchParams MakeDispatch(const TileXREpHookDispatch &d)
{
    EpDispatchParams p {};
    p.x = Fake(d.has & TILEXR_HOOK_X, 0x1000);
    p.expertIds = static_cast<int32_t *>(Fake(d.has & TILEXR_HOOK_EXPERT_IDS, 0x2000));
    p.scales = Fake(d.has & TILEXR_HOOK_SCALES, 0x3000);
    p.xActiveMask = static_cast<bool *>(Fake(d.has & TILEXR_HOOK_ACTIVE_MASK, 0x4000));
    p.expertScales = Fake(d.has & TILEXR_HOOK_EXPERT_SCALES, 0x5000);
    p.comm = Fake(d.has & TILEXR_HOOK_COMM, 0x6000);
    p.expandXOut = Fake(d.has & TILEXR_HOOK_EXPAND_X, 0x7000);
    p.dynamicScalesOut = Fake(d.has & TILEXR_HOOK_DYNAMIC_SCALES, 0x8000);
    p.assistInfoForCombineOut = static_cast<int32_t *>(Fake(d.has & TILEXR_HOOK_ASSIST, 0x9000));
    p.expertTokenNumsOut = static_cast<int64_t *>(Fake(d.has & TILEXR_HOOK_TOKEN_NUMS, 0xa000));
    p.epRecvCountsOut = static_cast<int32_t *>(Fake(d.has & TILEXR_HOOK_COUNTS, 0xb000));
    p.tpRecvCountsOut = static_cast<int32_t *>(Fake(d.has & TILEXR_HOOK_TP_COUNTS, 0xc000));
    p.expandScalesOut = Fake(d.has & TILEXR_HOOK_EXPAND_SCALES, 0xd000);
    p.workspace = Fake(d.has & TILEXR_HOOK_WORKSPACE, 0xe000);
    p.stream = Fake(d.has & TILEXR_HOOK_STREAM, 0xf000);
    p.activeMaskType = d.activeMaskType;
    p.bs = d.bs;
    p.h = d.h;
    p.topK = d.topK;
    p.moeExpertNum = d.moeExpertNum;
    p.epWorldSize = d.epWorldSize;
    p.epRankId = d.epRankId;
    p.tpWorldSize = d.tpWorldSize;
    p.tpRankId = d.tpRankId;
    p.expertShardType = d.expertShardType;
    p.sharedExpertNum = d.sharedExpertNum;
    p.sharedExpertRankNum = d.sharedExpertRankNum;
    p.quantMode = d.quantMode;
    p.globalBs = d.globalBs;
    p.expertTokenNumsType = d.expertTokenNumsType;
    p.dtype = static_cast<TileXR::TileXRDataType>(d.dtype);
    p.expandXOutDtype = static_cast<TileXR::TileXRDataType>(d.expandXOutDtype);
    return p;
}

EpCombineParams MakeCombine(const TileXREpHookCombine &c)
{
    EpCombineParams p {};
    p.expertOut = Fake(c.has & TILEXR_HOOK_X, 0x1000);
    p.assistInfoForCombine = static_cast<int32_t *>(Fake(c.has & TILEXR_HOOK_ASSIST, 0x9000));
    p.epRecvCounts = static_cast<int32_t *>(Fake(c.has & TILEXR_HOOK_COUNTS, 0xb000));
    p.expertScales = static_cast<float *>(Fake(c.has & TILEXR_HOOK_EXPERT_SCALES, 0x5000));
    p.xActiveMask = static_cast<bool *>(Fake(c.has & TILEXR_HOOK_ACTIVE_MASK, 0x4000));
    p.sharedExpertX = Fake(c.has & TILEXR_HOOK_SCALES, 0x3000);
    p.comm = Fake(c.has & TILEXR_HOOK_COMM, 0x6000);
    p.yOut = Fake(c.has & TILEXR_HOOK_EXPAND_X, 0x7000);
    p.workspace = Fake(c.has & TILEXR_HOOK_WORKSPACE, 0xe000);
    p.stream = Fake(c.has & TILEXR_HOOK_STREAM, 0xf000);
    p.activeMaskType = c.activeMaskType;
    p.bs = c.bs;
    p.h = c.h;
    p.topK = c.topK;
    p.moeExpertNum = c.moeExpertNum;
    p.epWorldSize = c.epWorldSize;
    p.epRankId = c.epRankId;
    p.tpWorldSize = c.tpWorldSize;
    p.tpRankId = c.tpRankId;
    p.expertShardType = c.expertShardType;
    p.sharedExpertNum = c.sharedExpertNum;
    p.sharedExpertRankNum = c.sharedExpertRankNum;
    p.quantMode = c.quantMode;
    p.globalBs = c.globalBs;
    p.dtype = static_cast<TileXR::TileXRDataType>(c.dtype);
    return p;
}

} // namespace

extern "C" {

int TileXREpHookValidateDispatch(int which, const TileXREpHookDispatch *dispatch, const TileXREpHookComm *comm)
{
    if (dispatch == nullptr) {
        return TileXR::TILEXR_ERROR_PARA_CHECK_FAIL;
    }
    const EpDispatchParams p = MakeDispatch(*dispatch);
    if (which == TILEXR_HOOK_RULE_BASIC) {
        return TileXREpValidateBasicDispatchParams(p);
    }
    if (comm == nullptr) {
        return TileXR::TILEXR_ERROR_PARA_CHECK_FAIL;
    }
    const TileXR::CommArgs args = MakeComm(*comm);
    EpWindowConfig window {};
    EpMemoryDispatchReferenceConfig memory {};
    switch (which) {
        case TILEXR_HOOK_RULE_V2:
            return TileXREpValidateDispatchV2Config(p, args);
        case TILEXR_HOOK_RULE_MVP:
            return TileXREpValidateDispatchConfig(p, args, &window);
        case TILEXR_HOOK_RULE_MEMORY:
            return TileXREpValidateDispatchMemoryConfig(p, args, comm->blockDim, &memory, true);
        case TILEXR_HOOK_RULE_MEMORY_UNCAPPED:
            return TileXREpValidateDispatchMemoryConfig(p, args, comm->blockDim, &memory, false);
        default:
            return TileXR::TILEXR_ERROR_PARA_CHECK_FAIL;
    }
}

int TileXREpHookValidateCombine(int which, const TileXREpHookCombine *combine, const TileXREpHookComm *comm)
{
    if (combine == nullptr) {
        return TileXR::TILEXR_ERROR_PARA_CHECK_FAIL;
    }
    const EpCombineParams p = MakeCombine(*combine);
    if (which == TILEXR_HOOK_RULE_BASIC) {
        return TileXREpValidateBasicCombineParams(p);
    }
    if (comm == nullptr) {
        return TileXR::TILEXR_ERROR_PARA_CHECK_FAIL;
    }
    const TileXR::CommArgs args = MakeComm(*comm);
    EpWindowConfig window {};
    EpMemoryCombineReferenceConfig memory {};
    switch (which) {
        case TILEXR_HOOK_RULE_MVP:
            return TileXREpValidateCombineConfig(p, args, &window, true);
        case TILEXR_HOOK_RULE_MEMORY:
            return TileXREpValidateCombineMemoryConfig(p, args, comm->blockDim, &memory, true);
        case TILEXR_HOOK_RULE_MEMORY_UNCAPPED:
            return TileXREpValidateCombineMemoryConfig(p, args, comm->blockDim, &memory, false);
        default:
            return TileXR::TILEXR_ERROR_PARA_CHECK_FAIL;
    }
}

int TileXREpHookWindowConfig(int64_t rankSize, int64_t expertRankSize, int64_t bs, int64_t h, int64_t topK,
    int64_t moeExpertNum, int64_t sharedExpertNum, int64_t sharedExpertRankNum, int dtype, int64_t payloadExtraBytes,
    int64_t *out9)
{
    EpWindowConfig cfg {};
    const int ret = TileXREpBuildDispatchWindowConfigForExpertRanks(rankSize, expertRankSize, bs, h, topK,
        moeExpertNum, sharedExpertNum, sharedExpertRankNum, static_cast<TileXR::TileXRDataType>(dtype),
        payloadExtraBytes, out9 == nullptr ? nullptr : &cfg);
    if (ret == 0) {
        const int64_t v[9] = {cfg.localExpertNum, cfg.dtypeBytes, cfg.maxRoutesPerSrc, cfg.rowBytes,
            cfg.payloadRowBytes, cfg.payloadBytesPerSlot, cfg.assistBytesPerSlot, cfg.slotBytes, cfg.totalBytes};
        std::memcpy(out9, v, sizeof(v));
    }
    return ret;
}

int TileXREpHookMemoryDispatchConfig(int64_t rankSize, int64_t rank, int64_t bs, int64_t h, int64_t topK,
    int64_t moeExpertNum, int64_t sharedExpertNum, int64_t sharedExpertRankNum, int64_t globalBs, int dtype,
    int expandXOutDtype, int64_t quantMode, uint32_t blockDim, int64_t *out19)
{
    EpMemoryDispatchReferenceConfig cfg {};
    const int ret = TileXREpBuildMemoryDispatchReferenceConfig(rankSize, rank, bs, h, topK, moeExpertNum,
        sharedExpertNum, sharedExpertRankNum, globalBs, static_cast<TileXR::TileXRDataType>(dtype),
        static_cast<TileXR::TileXRDataType>(expandXOutDtype), quantMode, blockDim, out19 == nullptr ? nullptr : &cfg);
    if (ret == 0) {
        const int64_t v[19] = {cfg.localExpertNum, cfg.rscvStatusNum, cfg.blockDim, cfg.aivUsedCumSum,
            cfg.aivUsedAllToAll, cfg.sharedUsedAivNum, cfg.moeUsedAivNum, cfg.hCommuSize, cfg.hOutSize,
            cfg.scaleOutBytes, cfg.tokenQuantAlignBytes, cfg.expertPerSizeOnWin, cfg.combineReserveBytes,
            cfg.workspaceBytes, cfg.totalWinSize, cfg.dispatchHalfBytes, cfg.maxSizeForUbBuffer, cfg.totalUbSize,
            cfg.allToAllUbBytes};
        std::memcpy(out19, v, sizeof(v));
    }
    return ret;
}

int TileXREpHookMemoryCombineConfig(int64_t rankSize, int64_t rank, int64_t bs, int64_t h, int64_t topK,
    int64_t moeExpertNum, int64_t sharedExpertNum, int64_t sharedExpertRankNum, int64_t globalBs, int dtype,
    int64_t quantMode, uint32_t blockDim, int64_t *out10)
{
    EpMemoryCombineReferenceConfig cfg {};
    const int ret = TileXREpBuildMemoryCombineReferenceConfig(rankSize, rank, bs, h, topK, moeExpertNum,
        sharedExpertNum, sharedExpertRankNum, globalBs, static_cast<TileXR::TileXRDataType>(dtype), quantMode,
        blockDim, out10 == nullptr ? nullptr : &cfg);
    if (ret == 0) {
        const int64_t v[10] = {cfg.moeExpertNumPerRank, cfg.blockDim, cfg.blockCntPerToken, cfg.packedRowBytes,
            cfg.combineReserveBytes, cfg.workspaceBytes, cfg.totalWinSize, cfg.combineHalfBytes, cfg.receiveUbBytes,
            cfg.sendUbBytes};
        std::memcpy(out10, v, sizeof(v));
    }
    return ret;
}

uint32_t TileXREpHookMemoryCountCoreNum(int64_t totalExpertNum, int64_t rscvStatusNum, uint32_t blockDim)
{
    return TileXREpMemoryCountCoreNum(totalExpertNum, rscvStatusNum, blockDim);
}

int TileXREpHookDstRank(int32_t expertId, int64_t localExpertNum)
{
    return TileXREpDstRank(expertId, localExpertNum);
}

int TileXREpHookLocalExpert(int32_t expertId, int64_t localExpertNum)
{
    return TileXREpLocalExpert(expertId, localExpertNum);
}

int64_t TileXREpHookDataTypeSize(int dtype)
{
    return TileXREpDataTypeSize(static_cast<TileXR::TileXRDataType>(dtype));
}

int64_t TileXREpHookAlignUp(int64_t value, int64_t alignment)
{
    return TileXREpAlignUp(value, alignment);
}

int64_t TileXREpHookUdmaOperationBytes(int64_t totalBytes, int64_t rankSize, int64_t slotBytes)
{
    return TileXREpUdmaOperationBytes(totalBytes, rankSize, slotBytes);
}

int64_t TileXREpHookUdmaWorkspaceBytes(int64_t totalBytes, int64_t rankSize, int64_t slotBytes)
{
    return TileXREpUdmaRequiredWorkspaceBytes(totalBytes, rankSize, slotBytes);
}

int TileXREpHookTilePublishStress(int totalRows, int maxRows, int tileRows, int parts, int threads, int rounds,
    uint32_t seed, int fault)
{
    if (totalRows < 0 || maxRows < totalRows || tileRows <= 0 || parts <= 0 || threads <= 0 || rounds <= 0) {
        return -100;
    }
    const int maxTiles = (maxRows + tileRows - 1) / tileRows;
    const int tiles = (totalRows + tileRows - 1) / tileRows;
    std::vector<uint32_t> counters(static_cast<size_t>(TileXREp::TileCounterWords(maxRows, tileRows)), 0u);
    std::vector<uint64_t> flags(static_cast<size_t>(maxTiles > 0 ? maxTiles : 1), 0ull);
    std::vector<std::atomic<int>> landed(static_cast<size_t>(totalRows > 0 ? totalRows : 1));
    std::vector<std::atomic<int>> stores(static_cast<size_t>(maxTiles > 0 ? maxTiles : 1));
    std::atomic<int> violation {0};

    // host flavour of the three memory operations; a store of a readiness word checks the protocol's promise
    struct HostOps {
        TileXREp::TilePublishArgs *args;
        std::vector<uint64_t> *flags;
        std::vector<std::atomic<int>> *landed;
        std::vector<std::atomic<int>> *stores;
        std::atomic<int> *violation;
        int parts;
        uint32_t FetchAdd(uint32_t *p) { return __atomic_fetch_add(p, 1u, __ATOMIC_ACQ_REL); }
        void Store(uint32_t *p, uint32_t v) { __atomic_store_n(p, v, __ATOMIC_RELEASE); }
        void Store(uint64_t *p, uint64_t v)
        {
            const int tile = static_cast<int>(p - flags->data());
            const int begin = tile * args->tileRows;
            const int end = begin + args->tileRows < args->totalRows ? begin + args->tileRows : args->totalRows;
            for (int r = begin; r < end; ++r) {
                if ((*landed)[static_cast<size_t>(r)].load(std::memory_order_acquire) != parts) {
                    violation->store(-1);      // published before every part of every row had landed
                }
            }
            if ((*stores)[static_cast<size_t>(tile)].fetch_add(1) != 0) {
                violation->store(-2);          // published twice in one dispatch
            }
            __atomic_store_n(p, v, __ATOMIC_RELEASE);
        }
    };

    std::mt19937 rng(seed);
    for (int round = 0; round < rounds; ++round) {
        TileXREp::TilePublishArgs args {};
        args.flags = flags.data();
        args.counters = counters.data();
        args.tileRows = tileRows;
        args.maxTiles = maxTiles;
        args.totalRows = totalRows;
        args.epoch = static_cast<uint64_t>(round + 1);
        for (auto &l : landed) {
            l.store(0);
        }
        for (auto &st : stores) {
            st.store(0);
        }
        // every (row, part) event once, shuffled, dealt to the threads round-robin
        std::vector<int> events(static_cast<size_t>(totalRows) * parts);
        for (size_t i = 0; i < events.size(); ++i) {
            events[i] = static_cast<int>(i);
        }
        std::shuffle(events.begin(), events.end(), rng);
        std::vector<std::thread> pool;
        for (int t = 0; t < threads; ++t) {
            pool.emplace_back([&, t] {
                HostOps ops {&args, &flags, &landed, &stores, &violation, parts};
                for (size_t i = static_cast<size_t>(t); i < events.size(); i += static_cast<size_t>(threads)) {
                    const int row = events[i] / parts;
                    if (fault == 1) {
                        TileXREp::PublishLanded(ops, args, row, parts);
                        std::this_thread::yield();
                        landed[static_cast<size_t>(row)].fetch_add(1, std::memory_order_release);
                        continue;
                    }
                    landed[static_cast<size_t>(row)].fetch_add(1, std::memory_order_release);   // "the part is in memory"
                    TileXREp::PublishLanded(ops, args, row, parts);
                    if (fault == 2 && i == static_cast<size_t>(t)) {
                        TileXREp::PublishLanded(ops, args, row, parts);
                    }
                }
            });
        }
        for (auto &th : pool) {
            th.join();
        }
        if (violation.load() != 0) {
            return violation.load();
        }
        for (int tile = 0; tile < tiles; ++tile) {
            const int left = totalRows - tile * tileRows;
            const uint64_t want = (args.epoch << 32) | static_cast<uint32_t>(left < tileRows ? left : tileRows);
            if (flags[static_cast<size_t>(tile)] != want) {
                return -3;                     // a tile was never published, or with the wrong word
            }
        }
        for (uint32_t c : counters) {
            if (c != 0u) {
                return -4;                     // a counter did not return to zero
            }
        }
    }
    return 0;
}

}
