// MVP-route window arithmetic and expert placement.
//
// Restates the numbers of the reference's src/ep/host/ep_layout.cpp: a per-destination window made of a 64-byte
// header and one slot per source rank; a slot is a 64-byte header, `bs*(topK+shared)` payload rows (plus optional
// per-row extra bytes, e.g. a float scale), then 16-byte assist tuples, each part rounded up to 32 bytes.  On one
// device rows never pass through such a window, but callers size buffers by these values and the reference's
// known-answer tests pin them, so they are kept exact.
#include "checked_math.h"
#include "ep_host.h"

namespace TileXREp {

int64_t TileXREpAlignUp(int64_t value, int64_t alignment)
{
    // reference: ep_layout.cpp:41-55
    return Nat(value).alignUp(alignment).get();
}

int64_t TileXREpDataTypeSize(TileXR::TileXRDataType dtype)
{
    // reference: ep_layout.cpp:57-66
    switch (dtype) {
        case TileXR::TILEXR_DATA_TYPE_INT8:
            return 1;
        case TileXR::TILEXR_DATA_TYPE_FP16:
        case TileXR::TILEXR_DATA_TYPE_BFP16:
            return 2;
        default:
            return TileXR::TILEXR_INVALID_VALUE;
    }
}

bool TileXREpIsSupportedDataType(TileXR::TileXRDataType dtype)
{
    return TileXREpDataTypeSize(dtype) > 0;
}

int64_t TileXREpUdmaOperationBytes(int64_t totalBytes, int64_t rankSize, int64_t slotBytes)
{
    // reference: ep_layout.cpp:73-113.  Two window copies, a ready word per rank, R*R relay slots and a second
    // set of ready words, every part starting on a cache line.
    if (totalBytes <= 0 || rankSize <= 0 || rankSize > TileXR::TILEXR_MAX_RANK_SIZE || slotBytes <= 0) {
        return TileXR::TILEXR_INVALID_VALUE;
    }
    const Nat ready = Nat(rankSize) * Nat(static_cast<int64_t>(sizeof(uint64_t)));
    const Nat relaySlots = (Nat(totalBytes).alignUp(kEpWindowAlignmentBytes) * Nat(2) + ready)
                               .alignUp(kEpUdmaCacheLineBytes);
    const Nat relayReady = (relaySlots + Nat(rankSize) * Nat(rankSize) * Nat(slotBytes))
                               .alignUp(kEpUdmaCacheLineBytes);
    return (relayReady + ready).alignUp(kEpUdmaCacheLineBytes).get();
}

int64_t TileXREpUdmaRequiredWorkspaceBytes(int64_t totalBytes, int64_t rankSize, int64_t slotBytes)
{
    // reference: ep_layout.cpp:115-128: two operations and a status word
    const int64_t op = TileXREpUdmaOperationBytes(totalBytes, rankSize, slotBytes);
    if (op == TileXR::TILEXR_INVALID_VALUE) {
        return TileXR::TILEXR_INVALID_VALUE;
    }
    return (Nat(op) * Nat(2) + Nat(static_cast<int64_t>(sizeof(uint64_t)))).alignUp(kEpUdmaCacheLineBytes).get();
}

int TileXREpBuildWindowConfig(int64_t rankSize, int64_t bs, int64_t h, int64_t topK, int64_t moeExpertNum,
    TileXR::TileXRDataType dtype, EpWindowConfig *out)
{
    // reference: ep_layout.cpp:130-134
    return TileXREpBuildDispatchWindowConfigForExpertRanks(rankSize, rankSize, bs, h, topK, moeExpertNum, 0, 0,
        dtype, 0, out);
}

int TileXREpBuildDispatchWindowConfigForExpertRanks(int64_t rankSize, int64_t expertRankSize, int64_t bs,
    int64_t h, int64_t topK, int64_t moeExpertNum, int64_t sharedExpertNum, int64_t sharedExpertRankNum,
    TileXR::TileXRDataType dtype, int64_t payloadExtraBytes, EpWindowConfig *out)
{
    return TileXREpBuildDispatchWindowConfigBounded(rankSize, expertRankSize, bs, h, topK, moeExpertNum,
        sharedExpertNum, sharedExpertRankNum, dtype, payloadExtraBytes, TileXR::IPC_BUFF_MAX_SIZE, out);
}

int TileXREpBuildDispatchWindowConfigBounded(int64_t rankSize, int64_t expertRankSize, int64_t bs,
    int64_t h, int64_t topK, int64_t moeExpertNum, int64_t sharedExpertNum, int64_t sharedExpertRankNum,
    TileXR::TileXRDataType dtype, int64_t payloadExtraBytes, int64_t maxTotalBytes, EpWindowConfig *out)
{
    // reference: ep_layout.cpp:152-226 (there maxTotalBytes is always the 512 MiB peer-window size)
    const int64_t moeRankNum = expertRankSize - sharedExpertRankNum;
    const bool shapeOk = out != nullptr && rankSize > 0 && rankSize <= TileXR::TILEXR_MAX_RANK_SIZE &&
        expertRankSize > 0 && expertRankSize <= rankSize && bs > 0 && h > 0 && topK > 0 && moeExpertNum > 0 &&
        sharedExpertNum >= 0 && sharedExpertRankNum >= 0 && sharedExpertRankNum <= expertRankSize &&
        moeRankNum > 0 && moeExpertNum % moeRankNum == 0 && payloadExtraBytes >= 0 &&
        TileXREpIsSupportedDataType(dtype);
    if (!shapeOk) {
        return TileXR::TILEXR_ERROR_PARA_CHECK_FAIL;
    }

    EpWindowConfig cfg {};
    cfg.rankSize = rankSize;
    cfg.bs = bs;
    cfg.h = h;
    cfg.topK = topK;
    cfg.moeExpertNum = moeExpertNum;
    cfg.localExpertNum = sharedExpertRankNum > 0 ? moeExpertNum / moeRankNum : moeExpertNum / expertRankSize;
    cfg.dtypeBytes = TileXREpDataTypeSize(dtype);

    const Nat routes = Nat(bs) * (Nat(topK) + Nat(sharedExpertNum));
    const Nat rowBytes = Nat(h) * Nat(cfg.dtypeBytes);
    const Nat payload = (routes * rowBytes + routes * Nat(payloadExtraBytes)).alignUp(kEpWindowAlignmentBytes);
    const Nat assist = (routes * Nat(kEpAssistTupleInts * static_cast<int64_t>(sizeof(int32_t))))
                           .alignUp(kEpWindowAlignmentBytes);
    const Nat slot = (Nat(kEpSrcSlotHeaderBytes) + payload + assist).alignUp(kEpWindowAlignmentBytes);
    const Nat total = Nat(kEpWindowHeaderBytes) + Nat(rankSize) * slot;
    if (!total.ok() || total.get() > maxTotalBytes) {
        return TileXR::TILEXR_ERROR_PARA_CHECK_FAIL;
    }

    cfg.maxRoutesPerSrc = routes.get();
    cfg.rowBytes = rowBytes.get();
    cfg.payloadRowBytes = cfg.rowBytes;
    cfg.payloadBytesPerSlot = payload.get();
    cfg.assistBytesPerSlot = assist.get();
    cfg.slotBytes = slot.get();
    cfg.totalBytes = total.get();
    *out = cfg;
    return TileXR::TILEXR_SUCCESS;
}

int TileXREpDstRank(int32_t expertId, int64_t localExpertNum)
{
    // reference: ep_layout.cpp:228-234
    if (expertId < 0 || localExpertNum <= 0) {
        return static_cast<int>(TileXR::TILEXR_INVALID_VALUE);
    }
    return static_cast<int>(expertId / localExpertNum);
}

int TileXREpLocalExpert(int32_t expertId, int64_t localExpertNum)
{
    // reference: ep_layout.cpp:236-242
    if (expertId < 0 || localExpertNum <= 0) {
        return static_cast<int>(TileXR::TILEXR_INVALID_VALUE);
    }
    return static_cast<int>(expertId % localExpertNum);
}

} // namespace TileXREp
