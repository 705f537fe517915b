// Memory-route reference window arithmetic.
//
// The reference stages every dispatched / combined row in a peer window as 512-byte blocks (480 payload + 32 flag
// bytes, src/include/tilexr_data_as_flag.h:22-30) and budgets its 190 KiB unified buffer per vector core; the
// numbers below restate src/ep/host/ep_memory_layout.cpp so callers that size buffers by them, and the reference's
// own known-answer tests, get identical values.  The HIP kernels need neither the window nor the buffer budget:
// `enforceCapacity == false` keeps every argument rule and overflow check but skips the rejections that only
// express those two capacities.
#include <algorithm>

#include "checked_math.h"
#include "ep_host.h"

namespace TileXREp {
namespace {

constexpr int64_t kAlign = kEpMemoryWindowAlignmentBytes;
constexpr int64_t kBlock = kEpMemorySplitBlockBytes;
constexpr int64_t kPayload = kEpMemorySplitPayloadBytes;

bool IsFloat16Like(TileXR::TileXRDataType dtype)
{
    return dtype == TileXR::TILEXR_DATA_TYPE_FP16 || dtype == TileXR::TILEXR_DATA_TYPE_BFP16;
}

// Rules shared by both configs (reference: ep_memory_layout.cpp:78-90, 318-330).
bool SharedRulesOk(int64_t rankSize, int64_t rank, int64_t bs, int64_t h, int64_t topK, int64_t moeExpertNum,
    int64_t sharedExpertNum, int64_t sharedExpertRankNum, int64_t globalBs, TileXR::TileXRDataType dtype)
{
    const int64_t moeRankNum = rankSize - sharedExpertRankNum;
    return rankSize > 0 && rankSize <= TileXR::TILEXR_MAX_RANK_SIZE && rank >= 0 && rank < rankSize && bs > 0 &&
        h > 0 && topK > 0 && moeExpertNum > 0 && sharedExpertNum >= 0 && sharedExpertRankNum >= 0 && globalBs > 0 &&
        globalBs % rankSize == 0 && IsFloat16Like(dtype) &&
        ((sharedExpertNum == 0) == (sharedExpertRankNum == 0)) && sharedExpertRankNum < rankSize &&
        (sharedExpertNum == 0 || sharedExpertRankNum % sharedExpertNum == 0) && moeRankNum > 0 &&
        moeExpertNum % moeRankNum == 0;
}

// Workspace the reference carves from the end of the peer window: one int32 per (core, source rank, local expert).
Nat WorkspaceBytes(int64_t rankSize, int64_t expertsPerRank, uint32_t blockDim)
{
    return (Nat(static_cast<int64_t>(blockDim)) * (Nat(rankSize) * Nat(expertsPerRank)) *
            Nat(static_cast<int64_t>(sizeof(int32_t)))).alignUp(kAlign);
}

} // namespace

uint32_t TileXREpMemoryCountCoreNum(int64_t totalExpertNum, int64_t rscvStatusNum, uint32_t blockDim)
{
    // reference: ep_memory_layout.cpp:54-65 and tilexr_ep_dispatch_memory_kernel.h:388-392:
    // clamp(totalExperts / 16, 1, min(blockDim / 2, 8, receive states))
    if (totalExpertNum <= 0 || rscvStatusNum <= 0 || blockDim < 2) {
        return 0;
    }
    uint64_t cores = std::max<uint64_t>(static_cast<uint64_t>(totalExpertNum / 16), 1);
    cores = std::min<uint64_t>({cores, blockDim / 2, kEpMemoryMaxCountCoreNum, static_cast<uint64_t>(rscvStatusNum)});
    return static_cast<uint32_t>(cores);
}

static int BuildMemoryDispatch(int64_t rankSize, int64_t rank, int64_t bs, int64_t h, int64_t topK,
    int64_t moeExpertNum, int64_t sharedExpertNum, int64_t sharedExpertRankNum, int64_t globalBs,
    TileXR::TileXRDataType dtype, TileXR::TileXRDataType expandXOutDtype, int64_t quantMode, uint32_t blockDim,
    bool enforceCapacity, EpMemoryDispatchReferenceConfig *out)
{
    constexpr int kReject = TileXR::TILEXR_ERROR_PARA_CHECK_FAIL;
    const bool mx = quantMode == TILEXR_EP_QUANT_MXFP8;
    const bool outTypeOk = mx ? (expandXOutDtype == TileXR::TILEXR_DATA_TYPE_FP8E4M3 ||
                                    expandXOutDtype == TileXR::TILEXR_DATA_TYPE_FP8E5M2)
                              : expandXOutDtype == dtype;
    if (out == nullptr || blockDim < 2 || blockDim > kEpMemoryMaxVectorCoreNum ||
        (quantMode != TILEXR_EP_QUANT_NONE && !mx) || !outTypeOk ||
        !SharedRulesOk(rankSize, rank, bs, h, topK, moeExpertNum, sharedExpertNum, sharedExpertRankNum, globalBs,
            dtype)) {
        return kReject;
    }

    EpMemoryDispatchReferenceConfig cfg {};
    cfg.blockDim = blockDim;
    const int64_t expertsPerRank = moeExpertNum / (rankSize - sharedExpertRankNum);
    const bool sharedRank = rank < sharedExpertRankNum;
    cfg.localExpertNum = sharedRank ? 1 : expertsPerRank;
    cfg.rscvStatusNum = sharedRank ? rankSize : rankSize * expertsPerRank;

    // core split between counting and sending (reference: :103-126)
    const Nat totalExperts = Nat(sharedExpertRankNum) + Nat(moeExpertNum);
    if (!totalExperts.ok()) {
        return kReject;
    }
    cfg.aivUsedCumSum = TileXREpMemoryCountCoreNum(totalExperts.get(), cfg.rscvStatusNum, blockDim);
    if (cfg.aivUsedCumSum == 0 || cfg.aivUsedCumSum >= blockDim) {
        return kReject;
    }
    cfg.aivUsedAllToAll = blockDim - cfg.aivUsedCumSum;
    if (sharedExpertRankNum > 0) {
        const uint64_t share = static_cast<uint64_t>(cfg.aivUsedAllToAll) * static_cast<uint64_t>(sharedExpertNum) /
            static_cast<uint64_t>(topK + sharedExpertNum);
        cfg.sharedUsedAivNum = share == 0 ? 1u : static_cast<uint32_t>(share);
    }
    if (cfg.sharedUsedAivNum >= cfg.aivUsedAllToAll) {
        return kReject;
    }
    cfg.moeUsedAivNum = cfg.aivUsedAllToAll - cfg.sharedUsedAivNum;

    // one staged row: payload (+ E8M0 scales) + 32-byte {rank, token, k} triple, cut into 480-byte pieces (:128-152)
    const int64_t elemBytes = TileXREpDataTypeSize(dtype);
    const Nat inputBytes = Nat(h) * Nat(elemBytes);
    const Nat outBytes = Nat(h) * Nat(mx ? 1 : elemBytes);
    const Nat scaleBytes = mx ? Nat(h).ceilDiv(32).alignUp(2) : Nat(0);
    const Nat tripleOffset = (outBytes.alignUp(mx ? 256 : kAlign) + scaleBytes).alignUp(kAlign);
    const Nat blocks = (tripleOffset + Nat(kAlign)).ceilDiv(kPayload);
    const Nat packedPayload = blocks * Nat(kPayload);
    const Nat rowOnWindow = blocks * Nat(kBlock);
    const int64_t tokensPerRank = globalBs / rankSize;
    const Nat expertSegment = Nat(tokensPerRank) * rowOnWindow;

    // space the combine of the same layer keeps in the same half (:160-174)
    const Nat combineRow = inputBytes.ceilDiv(kPayload) * Nat(kBlock);
    const Nat combineReserve = Nat(tokensPerRank) * (Nat(topK) + Nat(sharedExpertNum)) * combineRow;

    const Nat workspace = WorkspaceBytes(rankSize, expertsPerRank, blockDim);
    if (!tripleOffset.ok() || !rowOnWindow.ok() || !expertSegment.ok() || !combineReserve.ok() || !workspace.ok()) {
        return kReject;
    }
    cfg.scaleOutBytes = scaleBytes.get();
    cfg.tokenQuantAlignBytes = tripleOffset.get();
    cfg.hCommuSize = rowOnWindow.get();
    cfg.hOutSize = outBytes.get();
    cfg.expertPerSizeOnWin = expertSegment.get();
    cfg.combineReserveBytes = combineReserve.get();
    cfg.workspaceBytes = workspace.get();
    cfg.totalWinSize = TileXR::IPC_BUFF_MAX_SIZE - kEpMemoryStateWindowBytes - cfg.workspaceBytes;
    if (cfg.totalWinSize <= 0) {
        return kReject;
    }
    cfg.dispatchHalfBytes = cfg.totalWinSize / 2;

    const Nat halfNeeded = combineReserve + Nat(cfg.rscvStatusNum) * expertSegment;
    if (!halfNeeded.ok() || (enforceCapacity && halfNeeded.get() > cfg.dispatchHalfBytes)) {
        return kReject;
    }

    // unified-buffer budgets (:197-303)
    const Nat idsBytes = Nat(bs) * Nat(topK) * Nat(static_cast<int64_t>(sizeof(int32_t)));
    const Nat idsAligned = idsBytes.alignUp(kAlign);
    const Nat maskAsHalf = Nat(bs) * Nat(topK).alignUp(kAlign) * Nat(static_cast<int64_t>(sizeof(uint16_t)));
    Nat scratch = Max(idsAligned, maskAsHalf);
    if (mx) {
        const Nat quantWork = (scaleBytes.alignUp(32) * Nat(static_cast<int64_t>(sizeof(float))) +
                               scaleBytes * Nat(static_cast<int64_t>(sizeof(uint16_t)))).alignUp(kAlign);
        scratch = Max(scratch, quantWork);
    }
    if (!scratch.ok()) {
        return kReject;
    }
    cfg.maxSizeForUbBuffer = scratch.get();
    cfg.totalUbSize = kEpMemoryFullUbBytes;
    if (enforceCapacity && (cfg.maxSizeForUbBuffer <= 0 || cfg.maxSizeForUbBuffer >= cfg.totalUbSize)) {
        return kReject;
    }

    const Nat rowAligned = inputBytes.alignUp(mx ? 128 : kAlign);
    const Nat idsVec = idsBytes.alignUp(256);
    const Nat sendUb = Nat(2 * kAlign) + Nat(2) * ((mx ? rowAligned : packedPayload) + rowAligned) +
        Nat(2) * idsVec + Nat(2) * scratch + idsAligned + (mx ? packedPayload : Nat(0)) + rowOnWindow;
    if (!sendUb.ok() || (enforceCapacity && sendUb.get() > cfg.totalUbSize)) {
        return kReject;
    }
    cfg.allToAllUbBytes = sendUb.get();

    const Nat statesPerCountCore = Nat(cfg.rscvStatusNum).ceilDiv(cfg.aivUsedCumSum);
    const Nat countUb = Nat(kAlign) + Nat(2) * scratch + Nat(2) * idsVec + totalExperts.alignUp(8) * Nat(kAlign) +
        (statesPerCountCore * Nat(kAlign)).alignUp(256) +
        (statesPerCountCore * Nat(static_cast<int64_t>(sizeof(float)))).alignUp(kAlign) +
        statesPerCountCore * Nat(kAlign) + Nat(2 * static_cast<int64_t>(blockDim)) * Nat(kAlign) +
        (Nat(static_cast<int64_t>(blockDim)) * Nat(static_cast<int64_t>(sizeof(float)))).alignUp(kAlign) +
        Nat(3 * kAlign) + Nat(cfg.rscvStatusNum) * Nat(kAlign) +
        (Nat(expertsPerRank) * Nat(static_cast<int64_t>(sizeof(int64_t)))).alignUp(kAlign) +
        (Nat(rankSize) * Nat(static_cast<int64_t>(sizeof(float)))).alignUp(kAlign);
    if (!countUb.ok() || (enforceCapacity && countUb.get() > cfg.totalUbSize)) {
        return kReject;
    }

    const Nat statesPerCore = Nat(cfg.rscvStatusNum).ceilDiv(blockDim);
    const Nat copyFixed = Nat(kAlign) + (Nat(cfg.rscvStatusNum) * Nat(static_cast<int64_t>(sizeof(int32_t)))).alignUp(kAlign) +
        Nat(2 * static_cast<int64_t>(cfg.aivUsedCumSum)) * Nat(kAlign) +
        Nat(3) * (statesPerCore * Nat(static_cast<int64_t>(sizeof(uint32_t)))).alignUp(kAlign) + Nat(2 * kAlign) +
        blocks * Nat(kAlign);
    if (!copyFixed.ok() || (enforceCapacity && (copyFixed.get() >= cfg.totalUbSize ||
                                                   cfg.totalUbSize - copyFixed.get() < cfg.hCommuSize))) {
        return kReject;
    }

    *out = cfg;
    return TileXR::TILEXR_SUCCESS;
}

int TileXREpBuildMemoryDispatchReferenceConfig(int64_t rankSize, int64_t rank, int64_t bs, int64_t h, int64_t topK,
    int64_t moeExpertNum, int64_t sharedExpertNum, int64_t sharedExpertRankNum, int64_t globalBs,
    TileXR::TileXRDataType dtype, TileXR::TileXRDataType expandXOutDtype, int64_t quantMode, uint32_t blockDim,
    EpMemoryDispatchReferenceConfig *out)
{
    return BuildMemoryDispatch(rankSize, rank, bs, h, topK, moeExpertNum, sharedExpertNum, sharedExpertRankNum,
        globalBs, dtype, expandXOutDtype, quantMode, blockDim, true, out);
}

static int BuildMemoryCombine(int64_t rankSize, int64_t rank, int64_t bs, int64_t h, int64_t topK,
    int64_t moeExpertNum, int64_t sharedExpertNum, int64_t sharedExpertRankNum, int64_t globalBs,
    TileXR::TileXRDataType dtype, int64_t quantMode, uint32_t blockDim, bool enforceCapacity,
    EpMemoryCombineReferenceConfig *out)
{
    constexpr int kReject = TileXR::TILEXR_ERROR_PARA_CHECK_FAIL;
    const bool mx = quantMode == TILEXR_EP_QUANT_COMM_MXFP8_E5M2 || quantMode == TILEXR_EP_QUANT_MXFP8;
    if (out == nullptr || blockDim == 0 || blockDim > kEpMemoryMaxVectorCoreNum ||
        (quantMode != TILEXR_EP_QUANT_NONE && !mx) ||
        !SharedRulesOk(rankSize, rank, bs, h, topK, moeExpertNum, sharedExpertNum, sharedExpertRankNum, globalBs,
            dtype)) {
        return kReject;
    }

    EpMemoryCombineReferenceConfig cfg {};
    cfg.blockDim = blockDim;
    cfg.moeExpertNumPerRank = moeExpertNum / (rankSize - sharedExpertRankNum);

    // one combined row on the wire (reference: :334-360)
    const int64_t elemBytes = TileXREpDataTypeSize(dtype);
    const Nat rowBytes = Nat(h) * Nat(elemBytes);
    const Nat scaleCount = mx ? Nat(h).ceilDiv(32).alignUp(2) : Nat(0);
    const Nat wireBytes = mx ? Nat(h).alignUp(256) + scaleCount : rowBytes;
    const Nat rowAligned = mx ? Nat(h).alignUp(128) * Nat(elemBytes) : rowBytes.alignUp(kAlign);
    const Nat blocks = wireBytes.ceilDiv(kPayload);
    const Nat packedRow = blocks * Nat(kBlock);
    const Nat routesPerToken = Nat(topK) + Nat(sharedExpertNum);
    const Nat reserve = Nat(globalBs / rankSize) * routesPerToken * packedRow;
    const Nat workspace = WorkspaceBytes(rankSize, cfg.moeExpertNumPerRank, blockDim);
    if (!blocks.ok() || !packedRow.ok() || !reserve.ok() || !workspace.ok()) {
        return kReject;
    }
    cfg.blockCntPerToken = blocks.get();
    cfg.packedRowBytes = packedRow.get();
    cfg.combineReserveBytes = reserve.get();
    cfg.workspaceBytes = workspace.get();
    cfg.totalWinSize = TileXR::IPC_BUFF_MAX_SIZE - kEpMemoryStateWindowBytes - cfg.workspaceBytes;
    cfg.combineHalfBytes = cfg.totalWinSize / 2;
    if (cfg.totalWinSize <= 0 || (enforceCapacity && cfg.combineReserveBytes > cfg.combineHalfBytes)) {
        return kReject;
    }

    // unified-buffer budgets of the receive and send phases (:378-455)
    const Nat flagFloats = (routesPerToken * blocks * Nat(kAlign / static_cast<int64_t>(sizeof(float)))).alignUp(64);
    const Nat flagCheck = flagFloats * Nat(static_cast<int64_t>(sizeof(float))) + flagFloats.alignUp(256);
    const Nat compact = blocks * Nat(kPayload);
    const Nat floatRow = (Nat(h) * Nat(static_cast<int64_t>(sizeof(float)))).alignUp(mx ? 512 : kAlign);
    const Nat outRow = rowBytes.alignUp(kAlign);
    Nat receive = Nat(4 * kAlign) + flagCheck + Max(compact, outRow) + Nat(3) * floatRow + outRow +
        (Nat(topK) * Nat(static_cast<int64_t>(sizeof(float)))).alignUp(kAlign) + Nat(bs).alignUp(kAlign) +
        blocks * Nat(kAlign);
    Nat send = Nat(kAlign) + (mx ? rowAligned : Max(rowAligned, compact)) + packedRow;
    if (mx) {
        receive = receive + scaleCount.alignUp(128) * Nat(2 * static_cast<int64_t>(sizeof(float)));
        send = send + compact + (scaleCount.alignUp(32) * Nat(static_cast<int64_t>(sizeof(float))) +
                                 scaleCount * Nat(static_cast<int64_t>(sizeof(uint16_t)))).alignUp(kAlign);
    }
    if (!receive.ok() || !send.ok()) {
        return kReject;
    }
    cfg.receiveUbBytes = receive.get();
    cfg.sendUbBytes = send.get();
    if (enforceCapacity && (cfg.sendUbBytes > kEpMemoryFullUbBytes || cfg.receiveUbBytes > kEpMemoryFullUbBytes)) {
        return kReject;
    }

    *out = cfg;
    return TileXR::TILEXR_SUCCESS;
}

int TileXREpBuildMemoryCombineReferenceConfig(int64_t rankSize, int64_t rank, int64_t bs, int64_t h, int64_t topK,
    int64_t moeExpertNum, int64_t sharedExpertNum, int64_t sharedExpertRankNum, int64_t globalBs,
    TileXR::TileXRDataType dtype, int64_t quantMode, uint32_t blockDim, EpMemoryCombineReferenceConfig *out)
{
    return BuildMemoryCombine(rankSize, rank, bs, h, topK, moeExpertNum, sharedExpertNum, sharedExpertRankNum,
        globalBs, dtype, quantMode, blockDim, true, out);
}

// Used by the validators: same rules, optionally without the staged-window / unified-buffer capacities.
int TileXREpBuildMemoryDispatchConfigFor(bool enforceCapacity, int64_t rankSize, int64_t rank, int64_t bs, int64_t h,
    int64_t topK, int64_t moeExpertNum, int64_t sharedExpertNum, int64_t sharedExpertRankNum, int64_t globalBs,
    TileXR::TileXRDataType dtype, TileXR::TileXRDataType expandXOutDtype, int64_t quantMode, uint32_t blockDim,
    EpMemoryDispatchReferenceConfig *out)
{
    return BuildMemoryDispatch(rankSize, rank, bs, h, topK, moeExpertNum, sharedExpertNum, sharedExpertRankNum,
        globalBs, dtype, expandXOutDtype, quantMode, blockDim, enforceCapacity, out);
}

int TileXREpBuildMemoryCombineConfigFor(bool enforceCapacity, int64_t rankSize, int64_t rank, int64_t bs, int64_t h,
    int64_t topK, int64_t moeExpertNum, int64_t sharedExpertNum, int64_t sharedExpertRankNum, int64_t globalBs,
    TileXR::TileXRDataType dtype, int64_t quantMode, uint32_t blockDim, EpMemoryCombineReferenceConfig *out)
{
    return BuildMemoryCombine(rankSize, rank, bs, h, topK, moeExpertNum, sharedExpertNum, sharedExpertRankNum,
        globalBs, dtype, quantMode, blockDim, enforceCapacity, out);
}

} // namespace TileXREp
