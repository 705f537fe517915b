// Argument and configuration rules of the EP entry points.
//
// Each function returns the status the reference returns for the same arguments:
//   basic parameter checks     src/ep/host/ep_dispatch_host.cpp:28-37, 155-163
//   MVP V2 capability rules    src/ep/host/ep_dispatch_host.cpp:39-111
//   MVP window / comm rules    src/ep/host/ep_dispatch_host.cpp:113-153, 165-186
//   memory-route dispatch      src/ep/host/ep_dispatch_memory_host.cpp:51-106
//   memory-route combine       src/ep/host/ep_combine_memory_host.cpp:43-82
// The order of the checks is kept, because the first failing rule decides between -1, -3 and -6.
#include <limits>

#include "ep_host.h"

namespace TileXREp {

int TileXREpBuildMemoryDispatchConfigFor(bool enforceCapacity, int64_t rankSize, int64_t rank, int64_t bs, int64_t h,
    int64_t topK, int64_t moeExpertNum, int64_t sharedExpertNum, int64_t sharedExpertRankNum, int64_t globalBs,
    TileXR::TileXRDataType dtype, TileXR::TileXRDataType expandXOutDtype, int64_t quantMode, uint32_t blockDim,
    EpMemoryDispatchReferenceConfig *out);
int TileXREpBuildMemoryCombineConfigFor(bool enforceCapacity, int64_t rankSize, int64_t rank, int64_t bs, int64_t h,
    int64_t topK, int64_t moeExpertNum, int64_t sharedExpertNum, int64_t sharedExpertRankNum, int64_t globalBs,
    TileXR::TileXRDataType dtype, int64_t quantMode, uint32_t blockDim, EpMemoryCombineReferenceConfig *out);

namespace {

using TileXR::CommArgs;
constexpr int kOk = TileXR::TILEXR_SUCCESS;
constexpr int kBadParam = TileXR::TILEXR_ERROR_PARA_CHECK_FAIL;
constexpr int kNoInit = TileXR::TILEXR_ERROR_NOT_INITIALIZED;
constexpr int kNoSupport = TileXR::TILEXR_ERROR_NOT_SUPPORT;

int64_t TpSize(int64_t tpWorldSize)
{
    return tpWorldSize == 0 ? 1 : tpWorldSize;
}

int64_t ExpertRanks(const CommArgs &comm, int64_t tpWorldSize)
{
    const int64_t tp = TpSize(tpWorldSize);
    return tp <= 0 ? 0 : comm.rankSize / tp;
}

bool SpansNodes(const CommArgs &comm)
{
    return comm.localRankSize > 0 && comm.localRankSize < comm.rankSize;
}

bool RankFieldsOk(const CommArgs &comm)
{
    return comm.rankSize > 0 && comm.rankSize <= TileXR::TILEXR_MAX_RANK_SIZE && comm.rank >= 0 &&
        comm.rank < comm.rankSize;
}

bool AllPeersMapped(const CommArgs &comm)
{
    for (int r = 0; r < comm.rankSize; ++r) {
        if (comm.peerMems[r] == nullptr) {
            return false;
        }
    }
    return true;
}

bool CrossNodeReady(const CommArgs &comm, const void *workspace)
{
    return workspace != nullptr && (comm.extraFlag & TileXR::ExtraFlag::UDMA) != 0 && comm.udmaInfoPtr != nullptr &&
        comm.udmaRegistryPtr != nullptr;
}

// globalBs must be 0 or bs * rankSize (reference: ep_dispatch_memory_host.cpp:23-35)
bool ResolveGlobalBs(int64_t bs, int64_t requested, const CommArgs &comm, int64_t *globalBs)
{
    if (bs <= 0 || comm.rankSize <= 0 || bs > std::numeric_limits<int64_t>::max() / comm.rankSize) {
        return false;
    }
    const int64_t expected = bs * comm.rankSize;
    if (requested != 0 && requested != expected) {
        return false;
    }
    *globalBs = expected;
    return true;
}

} // namespace

int TileXREpValidateBasicDispatchParams(const EpDispatchParams &p)
{
    const bool ok = p.x != nullptr && p.expertIds != nullptr && p.comm != nullptr && p.expandXOut != nullptr &&
        p.expertTokenNumsOut != nullptr && p.epRecvCountsOut != nullptr && p.assistInfoForCombineOut != nullptr &&
        p.stream != nullptr && p.bs > 0 && p.h > 0 && p.topK > 0 && p.moeExpertNum > 0 &&
        TileXREpIsSupportedDataType(p.dtype);
    return ok ? kOk : kBadParam;
}

int TileXREpValidateDispatchV2Config(const EpDispatchParams &p, const CommArgs &comm)
{
    if (p.expertShardType != 0) {
        return kNoSupport;
    }
    if (p.quantMode != TILEXR_EP_QUANT_NONE && p.quantMode != TILEXR_EP_QUANT_STATIC_INT8 &&
        p.quantMode != TILEXR_EP_QUANT_TOKEN_INT8) {
        return kNoSupport;
    }
    const bool int8Out = p.dtype == TileXR::TILEXR_DATA_TYPE_INT8;
    if (p.quantMode == TILEXR_EP_QUANT_STATIC_INT8 &&
        (p.scales == nullptr || !int8Out || p.dynamicScalesOut != nullptr || p.expandScalesOut != nullptr)) {
        return kBadParam;
    }
    if (p.quantMode == TILEXR_EP_QUANT_TOKEN_INT8 &&
        (p.scales != nullptr || !int8Out || p.dynamicScalesOut == nullptr || p.expandScalesOut != nullptr)) {
        return kBadParam;
    }
    if (p.quantMode == TILEXR_EP_QUANT_NONE && !TileXREpIsSupportedDataType(p.dtype)) {
        return kBadParam;
    }

    const int64_t tp = TpSize(p.tpWorldSize);
    if (p.tpRankId < 0 || p.tpRankId >= tp || (tp == 1 && p.tpRankId != 0)) {
        return kBadParam;
    }
    if (tp > 1) {
        if (p.tpRecvCountsOut == nullptr || comm.rankSize % tp != 0 || comm.rank % tp != p.tpRankId) {
            return kBadParam;
        }
        const int64_t groupBegin = (comm.rank / tp) * tp;
        const int64_t groupEnd = groupBegin + tp;
        if (groupBegin < 0 || groupEnd > comm.rankSize || comm.localRankSize <= 1) {
            return kNoSupport;
        }
        for (int64_t peer = groupBegin; peer < groupEnd; ++peer) {
            if (comm.rank / comm.localRankSize != peer / comm.localRankSize) {
                return kNoSupport;      // a tensor-parallel group must not span nodes
            }
        }
    }

    if (p.sharedExpertNum < 0 || p.sharedExpertRankNum < 0) {
        return kBadParam;
    }
    if ((p.sharedExpertNum == 0) != (p.sharedExpertRankNum == 0) || p.sharedExpertNum != p.sharedExpertRankNum) {
        return kNoSupport;
    }
    const int64_t expertRanks = ExpertRanks(comm, p.tpWorldSize);
    if (p.sharedExpertRankNum > expertRanks) {
        return kBadParam;
    }
    const int64_t moeRanks = expertRanks - p.sharedExpertRankNum;
    if (moeRanks <= 0 || p.moeExpertNum % moeRanks != 0) {
        return kBadParam;
    }
    if (p.expertTokenNumsType != kEpExpertTokenNumsTypePrefixSum &&
        p.expertTokenNumsType != kEpExpertTokenNumsTypeCount) {
        return kNoSupport;
    }
    const int64_t myEpRank = tp == 1 ? comm.rank : comm.rank / tp;
    if ((p.epWorldSize != 0 && p.epWorldSize != expertRanks) || (p.epRankId != 0 && p.epRankId != myEpRank) ||
        (p.globalBs != 0 && p.globalBs != p.bs * comm.rankSize)) {
        return kBadParam;
    }
    return kOk;
}

static int ValidateDispatchConfigBounded(const EpDispatchParams &p, const CommArgs &comm, EpWindowConfig *window,
    int64_t maxWindowBytes)
{
    if (window == nullptr || !RankFieldsOk(comm)) {
        return kBadParam;
    }
    if (!AllPeersMapped(comm)) {
        return kNoInit;
    }
    if (SpansNodes(comm) && !CrossNodeReady(comm, p.workspace)) {
        return kNoInit;
    }
    int ret = TileXREpValidateDispatchV2Config(p, comm);
    if (ret != kOk) {
        return ret;
    }
    const int64_t scaleBytesPerRow = p.quantMode == TILEXR_EP_QUANT_TOKEN_INT8 ? static_cast<int64_t>(sizeof(float)) : 0;
    ret = TileXREpBuildDispatchWindowConfigBounded(comm.rankSize, ExpertRanks(comm, p.tpWorldSize), p.bs, p.h, p.topK,
        p.moeExpertNum, p.sharedExpertNum, p.sharedExpertRankNum, p.dtype, scaleBytesPerRow, maxWindowBytes, window);
    if (ret != kOk) {
        return ret;
    }
    const int64_t tp = TpSize(p.tpWorldSize);
    if (tp > 1 && maxWindowBytes == TileXR::IPC_BUFF_MAX_SIZE &&
        TileXREpAlignUp(window->totalBytes, kEpWindowAlignmentBytes) * (tp + 2) > TileXR::IPC_BUFF_MAX_SIZE) {
        return kBadParam;
    }
    return kOk;
}

int TileXREpValidateDispatchConfig(const EpDispatchParams &p, const CommArgs &comm, EpWindowConfig *window)
{
    return ValidateDispatchConfigBounded(p, comm, window, TileXR::IPC_BUFF_MAX_SIZE);
}

int TileXREpValidateDispatchConfigUncapped(const EpDispatchParams &p, const CommArgs &comm, EpWindowConfig *window)
{
    return ValidateDispatchConfigBounded(p, comm, window, std::numeric_limits<int64_t>::max());
}

int TileXREpValidateDispatchMemoryConfig(const EpDispatchParams &p, const CommArgs &comm, uint32_t blockDim,
    EpMemoryDispatchReferenceConfig *config, bool enforceWindowCapacity)
{
    if (config == nullptr || !RankFieldsOk(comm)) {
        return kBadParam;
    }
    if (!AllPeersMapped(comm)) {
        return kNoInit;
    }
    if (TpSize(p.tpWorldSize) != 1 || p.tpRankId != 0 || p.tpRecvCountsOut != nullptr || p.scales != nullptr ||
        p.expertScales != nullptr || p.expandScalesOut != nullptr) {
        return kNoSupport;
    }
    const TileXR::TileXRDataType outType =
        p.expandXOutDtype == TileXR::TILEXR_DATA_TYPE_RESERVED ? p.dtype : p.expandXOutDtype;
    if (p.quantMode == TILEXR_EP_QUANT_NONE) {
        if (p.dynamicScalesOut != nullptr || outType != p.dtype) {
            return kBadParam;
        }
    } else if (p.quantMode == TILEXR_EP_QUANT_MXFP8) {
        if (p.dynamicScalesOut == nullptr || (outType != TileXR::TILEXR_DATA_TYPE_FP8E4M3 &&
                                                 outType != TileXR::TILEXR_DATA_TYPE_FP8E5M2)) {
            return kBadParam;
        }
    } else {
        return kNoSupport;
    }
    if (p.expertShardType != 0 || p.expertTokenNumsType < kEpExpertTokenNumsTypePrefixSum ||
        p.expertTokenNumsType > kEpExpertTokenNumsTypeCount ||
        (p.epWorldSize != 0 && p.epWorldSize != comm.rankSize) || (p.epRankId != 0 && p.epRankId != comm.rank)) {
        return kBadParam;
    }
    // mask type and pointer must agree (reference: ep_dispatch_memory_host.cpp:37-47)
    if (p.activeMaskType == TILEXR_EP_ACTIVE_MASK_NONE) {
        if (p.xActiveMask != nullptr) {
            return kBadParam;
        }
    } else if (p.activeMaskType == TILEXR_EP_ACTIVE_MASK_TOKEN || p.activeMaskType == TILEXR_EP_ACTIVE_MASK_EXPERT) {
        if (p.xActiveMask == nullptr) {
            return kBadParam;
        }
    } else {
        return kBadParam;
    }
    int64_t globalBs = 0;
    if (!ResolveGlobalBs(p.bs, p.globalBs, comm, &globalBs)) {
        return kBadParam;
    }
    return TileXREpBuildMemoryDispatchConfigFor(enforceWindowCapacity, comm.rankSize, comm.rank, p.bs, p.h, p.topK,
        p.moeExpertNum, p.sharedExpertNum, p.sharedExpertRankNum, globalBs, p.dtype, outType, p.quantMode, blockDim,
        config);
}

int TileXREpValidateBasicCombineParams(const EpCombineParams &p)
{
    const bool ok = p.expertOut != nullptr && p.assistInfoForCombine != nullptr && p.epRecvCounts != nullptr &&
        p.comm != nullptr && p.yOut != nullptr && p.stream != nullptr && p.bs > 0 && p.h > 0 && p.topK > 0 &&
        p.moeExpertNum > 0 && TileXREpIsSupportedDataType(p.dtype);
    return ok ? kOk : kBadParam;
}

int TileXREpValidateCombineConfig(const EpCombineParams &p, const CommArgs &comm, EpWindowConfig *window,
    bool enforceWindowCapacity)
{
    if (window == nullptr || !RankFieldsOk(comm)) {
        return kBadParam;
    }
    if (SpansNodes(comm) && !CrossNodeReady(comm, p.workspace)) {
        return kNoInit;
    }
    if (!AllPeersMapped(comm)) {
        return kNoInit;
    }
    return TileXREpBuildDispatchWindowConfigBounded(comm.rankSize, comm.rankSize, p.bs, p.h, p.topK, p.moeExpertNum,
        0, 0, p.dtype, 0, enforceWindowCapacity ? TileXR::IPC_BUFF_MAX_SIZE : std::numeric_limits<int64_t>::max(),
        window);
}

int TileXREpValidateCombineMemoryConfig(const EpCombineParams &p, const CommArgs &comm, uint32_t blockDim,
    EpMemoryCombineReferenceConfig *config, bool enforceWindowCapacity)
{
    if (config == nullptr || !RankFieldsOk(comm)) {
        return kBadParam;
    }
    if (!AllPeersMapped(comm)) {
        return kNoInit;
    }
    const bool mx = p.quantMode == TILEXR_EP_QUANT_COMM_MXFP8_E5M2 || p.quantMode == TILEXR_EP_QUANT_MXFP8;
    if (TpSize(p.tpWorldSize) != 1 || p.tpRankId != 0 || (p.quantMode != TILEXR_EP_QUANT_NONE && !mx)) {
        return kNoSupport;
    }
    if (mx && p.expertScales == nullptr) {
        return kBadParam;
    }
    if (p.expertShardType != 0 || (p.epWorldSize != 0 && p.epWorldSize != comm.rankSize) ||
        (p.epRankId != 0 && p.epRankId != comm.rank)) {
        return kBadParam;
    }
    // reference: ep_combine_memory_host.cpp:27-39 -- the [bs, topK] mask is a dispatch-only feature
    if (p.activeMaskType == TILEXR_EP_ACTIVE_MASK_NONE) {
        if (p.xActiveMask != nullptr) {
            return kBadParam;
        }
    } else if (p.activeMaskType == TILEXR_EP_ACTIVE_MASK_TOKEN) {
        if (p.xActiveMask == nullptr) {
            return kBadParam;
        }
    } else if (p.activeMaskType == TILEXR_EP_ACTIVE_MASK_EXPERT) {
        return kNoSupport;
    } else {
        return kBadParam;
    }
    int64_t globalBs = 0;
    if (!ResolveGlobalBs(p.bs, p.globalBs, comm, &globalBs)) {
        return kBadParam;
    }
    return TileXREpBuildMemoryCombineConfigFor(enforceWindowCapacity, comm.rankSize, comm.rank, p.bs, p.h, p.topK,
        p.moeExpertNum, p.sharedExpertNum, p.sharedExpertRankNum, globalBs, p.dtype, p.quantMode, blockDim, config);
}

} // namespace TileXREp
