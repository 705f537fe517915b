// Host-side interface of libtilexr-ep (internal header).
//
// Mirrors the reference's host layer so its tests and callers map one-to-one:
//   parameter bundles      src/ep/host/ep_host.h:17-78
//   window arithmetic      src/ep/host/ep_layout.h:11-49, ep_memory_layout.h:10-64
//   validation             src/ep/host/ep_host.h:86-101
// Only the arithmetic and the rules are shared with the reference; launching is HIP-specific (ep_launch.h).
#ifndef TILEXR_AMD_EP_HOST_H
#define TILEXR_AMD_EP_HOST_H

#include <cstdint>

#include "comm_args.h"
#include "tilexr_api.h"
#include "tilexr_ep.h"
#include "tilexr_types.h"

namespace TileXREp {

constexpr int64_t kEpExpertTokenNumsTypePrefixSum = 0;
constexpr int64_t kEpExpertTokenNumsTypeCount = 1;

// MVP window format constants (reference: src/ep/common/ep_window.h:8-22)
constexpr int64_t kEpWindowAlignmentBytes = 32;
constexpr int64_t kEpAssistTupleInts = 4;
constexpr int64_t kEpWindowHeaderBytes = 64;
constexpr int64_t kEpSrcSlotHeaderBytes = 64;

// Memory-route packing constants (reference: src/ep/host/ep_memory_layout.h:10-16,
// src/include/tilexr_data_as_flag.h:22-30)
constexpr int64_t kEpMemoryStateWindowBytes = 1024 * 1024;
constexpr int64_t kEpMemoryWindowAlignmentBytes = 32;
constexpr int64_t kEpMemorySplitBlockBytes = 512;
constexpr int64_t kEpMemorySplitPayloadBytes = 480;
constexpr int64_t kEpMemoryFullUbBytes = 190 * 1024;
constexpr uint32_t kEpMemoryMaxCountCoreNum = 8;
constexpr uint32_t kEpMemoryMaxVectorCoreNum = 200;

// UDMA cache line used by the cross-node workspace arithmetic (reference: src/include/tilexr_udma_types.h)
constexpr int64_t kEpUdmaCacheLineBytes = 64;

struct EpDispatchParams {
    void *x = nullptr;
    int32_t *expertIds = nullptr;
    void *scales = nullptr;
    bool *xActiveMask = nullptr;
    int64_t activeMaskType = TILEXR_EP_ACTIVE_MASK_NONE;
    void *expertScales = nullptr;
    TileXRCommPtr comm = nullptr;
    int64_t bs = 0;
    int64_t h = 0;
    int64_t topK = 0;
    int64_t moeExpertNum = 0;
    int64_t epWorldSize = 0;
    int64_t epRankId = 0;
    int64_t tpWorldSize = 0;
    int64_t tpRankId = 0;
    int64_t expertShardType = 0;
    int64_t sharedExpertNum = 0;
    int64_t sharedExpertRankNum = 0;
    int64_t quantMode = 0;
    int64_t globalBs = 0;
    int64_t expertTokenNumsType = 0;
    void *expandXOut = nullptr;
    void *dynamicScalesOut = nullptr;
    int32_t *assistInfoForCombineOut = nullptr;
    int64_t *expertTokenNumsOut = nullptr;
    int32_t *epRecvCountsOut = nullptr;
    int32_t *tpRecvCountsOut = nullptr;
    void *expandScalesOut = nullptr;
    void *workspace = nullptr;
    TileXR::TileXRDataType dtype = TileXR::TILEXR_DATA_TYPE_RESERVED;
    TileXR::TileXRDataType expandXOutDtype = TileXR::TILEXR_DATA_TYPE_RESERVED;
    aclrtStream stream = nullptr;
    // additions of TileXRMoeEpDispatchMemoryEx (no reference counterpart)
    int64_t expertCapacity = 0;
    int32_t *rowIndexMapOut = nullptr;
    uint64_t *tileFlagsOut = nullptr;
    int64_t tileRows = 0;
    int64_t *epochOut = nullptr;
    void *metaReadyEvent = nullptr;
    bool extended = false;
    // TileXRMoeEpDispatchMemoryNoAlloc: the kernels' scratch is the per-GPU static array, nothing is allocated
    bool noAlloc = false;
};

struct EpCombineParams {
    void *expertOut = nullptr;
    int32_t *assistInfoForCombine = nullptr;
    int32_t *epRecvCounts = nullptr;
    float *expertScales = nullptr;
    bool *xActiveMask = nullptr;
    int64_t activeMaskType = TILEXR_EP_ACTIVE_MASK_NONE;
    void *sharedExpertX = nullptr;
    TileXRCommPtr comm = nullptr;
    int64_t bs = 0;
    int64_t h = 0;
    int64_t topK = 0;
    int64_t moeExpertNum = 0;
    int64_t epWorldSize = 0;
    int64_t epRankId = 0;
    int64_t tpWorldSize = 0;
    int64_t tpRankId = 0;
    int64_t expertShardType = 0;
    int64_t sharedExpertNum = 0;
    int64_t sharedExpertRankNum = 0;
    int64_t quantMode = 0;
    int64_t globalBs = 0;
    void *yOut = nullptr;
    void *workspace = nullptr;
    TileXR::TileXRDataType dtype = TileXR::TILEXR_DATA_TYPE_RESERVED;
    aclrtStream stream = nullptr;
    // additions of TileXRMoeEpCombineMemoryEx (no reference counterpart)
    int64_t expertOutQuantMode = 0;
    void *expertOutScales = nullptr;
    const int32_t *rowIndexMap = nullptr;
    const uint64_t *tileFlags = nullptr;
    int64_t tileRows = 0;
    int64_t flagEpoch = 0;
    int64_t waitTimeoutUs = 0;
    int32_t *deviceStatusOut = nullptr;
    bool extended = false;
};

// ---- MVP window arithmetic (reference: src/ep/host/ep_layout.cpp) ----
struct EpWindowConfig {
    int64_t rankSize = 0;
    int64_t bs = 0;
    int64_t h = 0;
    int64_t topK = 0;
    int64_t moeExpertNum = 0;
    int64_t localExpertNum = 0;
    int64_t dtypeBytes = 0;
    int64_t maxRoutesPerSrc = 0;
    int64_t rowBytes = 0;
    int64_t payloadRowBytes = 0;
    int64_t payloadBytesPerSlot = 0;
    int64_t assistBytesPerSlot = 0;
    int64_t slotBytes = 0;
    int64_t totalBytes = 0;
};

int64_t TileXREpAlignUp(int64_t value, int64_t alignment);
int64_t TileXREpDataTypeSize(TileXR::TileXRDataType dtype);
bool TileXREpIsSupportedDataType(TileXR::TileXRDataType dtype);
int64_t TileXREpUdmaOperationBytes(int64_t totalBytes, int64_t rankSize, int64_t slotBytes);
int64_t TileXREpUdmaRequiredWorkspaceBytes(int64_t totalBytes, int64_t rankSize, int64_t slotBytes);
int TileXREpBuildWindowConfig(int64_t rankSize, int64_t bs, int64_t h, int64_t topK, int64_t moeExpertNum,
    TileXR::TileXRDataType dtype, EpWindowConfig *out);
int TileXREpBuildDispatchWindowConfigForExpertRanks(int64_t rankSize, int64_t expertRankSize, int64_t bs,
    int64_t h, int64_t topK, int64_t moeExpertNum, int64_t sharedExpertNum, int64_t sharedExpertRankNum,
    TileXR::TileXRDataType dtype, int64_t payloadExtraBytes, EpWindowConfig *out);
// Same arithmetic with a caller-chosen size limit (the entry points pass INT64_MAX: nothing is staged in a
// 512 MiB peer window on one device).
int TileXREpBuildDispatchWindowConfigBounded(int64_t rankSize, int64_t expertRankSize, int64_t bs,
    int64_t h, int64_t topK, int64_t moeExpertNum, int64_t sharedExpertNum, int64_t sharedExpertRankNum,
    TileXR::TileXRDataType dtype, int64_t payloadExtraBytes, int64_t maxTotalBytes, EpWindowConfig *out);
int TileXREpDstRank(int32_t expertId, int64_t localExpertNum);
int TileXREpLocalExpert(int32_t expertId, int64_t localExpertNum);

// ---- memory-route reference window arithmetic (reference: src/ep/host/ep_memory_layout.cpp) ----
// These numbers describe the reference's staged peer window (480+32 byte blocks, UB budgets).  The HIP path moves
// rows without that window, so they are kept for callers and tests that size buffers by them; launches on one
// device are not gated on the window capacity.
struct EpMemoryDispatchReferenceConfig {
    int64_t localExpertNum = 0;
    int64_t rscvStatusNum = 0;
    uint32_t blockDim = 0;
    uint32_t aivUsedCumSum = 0;
    uint32_t aivUsedAllToAll = 0;
    uint32_t sharedUsedAivNum = 0;
    uint32_t moeUsedAivNum = 0;
    int64_t hCommuSize = 0;
    int64_t hOutSize = 0;
    int64_t scaleOutBytes = 0;
    int64_t tokenQuantAlignBytes = 0;
    int64_t expertPerSizeOnWin = 0;
    int64_t combineReserveBytes = 0;
    int64_t workspaceBytes = 0;
    int64_t totalWinSize = 0;
    int64_t dispatchHalfBytes = 0;
    int64_t maxSizeForUbBuffer = 0;
    int64_t totalUbSize = 0;
    int64_t allToAllUbBytes = 0;
};

struct EpMemoryCombineReferenceConfig {
    int64_t moeExpertNumPerRank = 0;
    uint32_t blockDim = 0;
    int64_t blockCntPerToken = 0;
    int64_t packedRowBytes = 0;
    int64_t combineReserveBytes = 0;
    int64_t workspaceBytes = 0;
    int64_t totalWinSize = 0;
    int64_t combineHalfBytes = 0;
    int64_t receiveUbBytes = 0;
    int64_t sendUbBytes = 0;
};

uint32_t TileXREpMemoryCountCoreNum(int64_t totalExpertNum, int64_t rscvStatusNum, uint32_t blockDim);
int TileXREpBuildMemoryDispatchReferenceConfig(int64_t rankSize, int64_t rank, int64_t bs, int64_t h, int64_t topK,
    int64_t moeExpertNum, int64_t sharedExpertNum, int64_t sharedExpertRankNum, int64_t globalBs,
    TileXR::TileXRDataType dtype, TileXR::TileXRDataType expandXOutDtype, int64_t quantMode, uint32_t blockDim,
    EpMemoryDispatchReferenceConfig *out);
int TileXREpBuildMemoryCombineReferenceConfig(int64_t rankSize, int64_t rank, int64_t bs, int64_t h, int64_t topK,
    int64_t moeExpertNum, int64_t sharedExpertNum, int64_t sharedExpertRankNum, int64_t globalBs,
    TileXR::TileXRDataType dtype, int64_t quantMode, uint32_t blockDim, EpMemoryCombineReferenceConfig *out);

// ---- validation (reference: src/ep/host/ep_dispatch_host.cpp, ep_dispatch_memory_host.cpp,
//      ep_combine_memory_host.cpp) ----
int TileXREpValidateBasicDispatchParams(const EpDispatchParams &params);
int TileXREpValidateDispatchV2Config(const EpDispatchParams &params, const TileXR::CommArgs &commArgs);
int TileXREpValidateDispatchConfig(const EpDispatchParams &params, const TileXR::CommArgs &commArgs,
    EpWindowConfig *window);
// `enforceWindowCapacity` reproduces the reference's 512 MiB staged-window limit (its unit tests rely on it); the
// entry points pass false because rows never pass through such a window here.
int TileXREpValidateDispatchMemoryConfig(const EpDispatchParams &params, const TileXR::CommArgs &commArgs,
    uint32_t blockDim, EpMemoryDispatchReferenceConfig *config, bool enforceWindowCapacity = true);
int TileXREpValidateBasicCombineParams(const EpCombineParams &params);
int TileXREpValidateCombineConfig(const EpCombineParams &params, const TileXR::CommArgs &commArgs,
    EpWindowConfig *window, bool enforceWindowCapacity = true);
int TileXREpValidateCombineMemoryConfig(const EpCombineParams &params, const TileXR::CommArgs &commArgs,
    uint32_t blockDim, EpMemoryCombineReferenceConfig *config, bool enforceWindowCapacity = true);

// MVP dispatch rules without the 512 MiB staged-window limit (what the entry points use).
int TileXREpValidateDispatchConfigUncapped(const EpDispatchParams &params, const TileXR::CommArgs &commArgs,
    EpWindowConfig *window);

// Block count the reference-window arithmetic is evaluated with when the entry points validate (the reference
// passes its vector-core count, src/ep/host/ep_kernel_launch.cpp:297-305; the numbers only feed -3 checks).
constexpr uint32_t kEpReferenceBlockDim = 48;

} // namespace TileXREp

#endif // TILEXR_AMD_EP_HOST_H
