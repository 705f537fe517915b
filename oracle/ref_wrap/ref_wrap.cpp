// C-ABI shims over the reference's own host sources, compiled where they lie.
//
// Test infrastructure only.  This file is built by oracle/Makefile together with the reference's
// ep_layout.cpp, ep_memory_layout.cpp, its header-only MXFP8 golden model and its no-NPU checker
// core, into oracle/_ref/libtilexr_ep_ref.so.  It exists so the tests can compare this repository's
// host arithmetic and CPU oracle against the reference's compiled answers.  It is never linked into
// the product library.
#include <cstdint>
#include <cstring>
#include <vector>

#include "ep_layout.h"
#include "ep_memory_layout.h"
#include "mxfp8_golden.h"
#include "tilexr/checker/case.h"
#include "tilexr/checker/executor.h"
#include "tilexr/checker/oracle.h"
#include "tilexr/checker/world.h"
#include "tilexr_types.h"

extern "C" {

// out[13]: fields of EpWindowConfig in declaration order (after rankSize..moeExpertNum):
// localExpertNum, dtypeBytes, maxRoutesPerSrc, rowBytes, payloadRowBytes, payloadBytesPerSlot,
// assistBytesPerSlot, slotBytes, totalBytes
int ref_window_config(int64_t rankSize, int64_t expertRankSize, int64_t bs, int64_t h, int64_t topK,
    int64_t moeExpertNum, int64_t sharedExpertNum, int64_t sharedExpertRankNum, int dtype,
    int64_t payloadExtraBytes, int64_t *out)
{
    TileXREp::EpWindowConfig cfg {};
    const int ret = TileXREp::TileXREpBuildDispatchWindowConfigForExpertRanks(rankSize, expertRankSize, bs, h,
        topK, moeExpertNum, sharedExpertNum, sharedExpertRankNum, static_cast<TileXR::TileXRDataType>(dtype),
        payloadExtraBytes, &cfg);
    if (ret == 0 && out != nullptr) {
        out[0] = cfg.localExpertNum;
        out[1] = cfg.dtypeBytes;
        out[2] = cfg.maxRoutesPerSrc;
        out[3] = cfg.rowBytes;
        out[4] = cfg.payloadRowBytes;
        out[5] = cfg.payloadBytesPerSlot;
        out[6] = cfg.assistBytesPerSlot;
        out[7] = cfg.slotBytes;
        out[8] = cfg.totalBytes;
    }
    return ret;
}

int64_t ref_udma_operation_bytes(int64_t totalBytes, int64_t rankSize, int64_t slotBytes)
{
    return TileXREp::TileXREpUdmaOperationBytes(totalBytes, rankSize, slotBytes);
}

int64_t ref_udma_workspace_bytes(int64_t totalBytes, int64_t rankSize, int64_t slotBytes)
{
    return TileXREp::TileXREpUdmaRequiredWorkspaceBytes(totalBytes, rankSize, slotBytes);
}

uint32_t ref_memory_count_core_num(int64_t totalExpertNum, int64_t rscvStatusNum, uint32_t blockDim)
{
    return TileXREp::TileXREpMemoryCountCoreNum(totalExpertNum, rscvStatusNum, blockDim);
}

// out[19] in EpMemoryDispatchReferenceConfig declaration order.
int ref_memory_dispatch_config(int64_t rankSize, int64_t rank, int64_t bs, int64_t h, int64_t topK,
    int64_t moeExpertNum, int64_t sharedExpertNum, int64_t sharedExpertRankNum, int64_t globalBs, int dtype,
    int outDtype, int64_t quantMode, uint32_t blockDim, int64_t *out)
{
    TileXREp::EpMemoryDispatchReferenceConfig cfg {};
    const int ret = TileXREp::TileXREpBuildMemoryDispatchReferenceConfig(rankSize, rank, bs, h, topK, moeExpertNum,
        sharedExpertNum, sharedExpertRankNum, globalBs, static_cast<TileXR::TileXRDataType>(dtype),
        static_cast<TileXR::TileXRDataType>(outDtype), quantMode, blockDim, &cfg);
    if (ret == 0 && out != nullptr) {
        const int64_t values[19] = {cfg.localExpertNum, cfg.rscvStatusNum, cfg.blockDim, cfg.aivUsedCumSum,
            cfg.aivUsedAllToAll, cfg.sharedUsedAivNum, cfg.moeUsedAivNum, cfg.hCommuSize, cfg.hOutSize,
            cfg.scaleOutBytes, cfg.tokenQuantAlignBytes, cfg.expertPerSizeOnWin, cfg.combineReserveBytes,
            cfg.workspaceBytes, cfg.totalWinSize, cfg.dispatchHalfBytes, cfg.maxSizeForUbBuffer, cfg.totalUbSize,
            cfg.allToAllUbBytes};
        std::memcpy(out, values, sizeof(values));
    }
    return ret;
}

// out[10] in EpMemoryCombineReferenceConfig declaration order.
int ref_memory_combine_config(int64_t rankSize, int64_t rank, int64_t bs, int64_t h, int64_t topK,
    int64_t moeExpertNum, int64_t sharedExpertNum, int64_t sharedExpertRankNum, int64_t globalBs, int dtype,
    int64_t quantMode, uint32_t blockDim, int64_t *out)
{
    TileXREp::EpMemoryCombineReferenceConfig cfg {};
    const int ret = TileXREp::TileXREpBuildMemoryCombineReferenceConfig(rankSize, rank, bs, h, topK, moeExpertNum,
        sharedExpertNum, sharedExpertRankNum, globalBs, static_cast<TileXR::TileXRDataType>(dtype), quantMode,
        blockDim, &cfg);
    if (ret == 0 && out != nullptr) {
        const int64_t values[10] = {cfg.moeExpertNumPerRank, cfg.blockDim, cfg.blockCntPerToken, cfg.packedRowBytes,
            cfg.combineReserveBytes, cfg.workspaceBytes, cfg.totalWinSize, cfg.combineHalfBytes,
            cfg.receiveUbBytes, cfg.sendUbBytes};
        std::memcpy(out, values, sizeof(values));
    }
    return ret;
}

int ref_dst_rank(int32_t expertId, int64_t localExpertNum)
{
    return TileXREp::TileXREpDstRank(expertId, localExpertNum);
}

int ref_local_expert(int32_t expertId, int64_t localExpertNum)
{
    return TileXREp::TileXREpLocalExpert(expertId, localExpertNum);
}

// ---- MXFP8 golden model (tests/ep/demo/mxfp8_golden.h) ----
static TileXREpDemo::Mxfp8Format Format(int e5m2)
{
    return e5m2 ? TileXREpDemo::Mxfp8Format::E5M2 : TileXREpDemo::Mxfp8Format::E4M3;
}

int64_t ref_mxfp8_scale_count(int64_t h)
{
    return static_cast<int64_t>(TileXREpDemo::Mxfp8ScaleCountPerRow(static_cast<std::size_t>(h)));
}

void ref_mxfp8_quant_row(const float *input, int64_t h, int e5m2, uint8_t *elements, uint8_t *scales)
{
    TileXREpDemo::QuantizeMxfp8Row(input, static_cast<std::size_t>(h), Format(e5m2), elements, scales);
}

uint8_t ref_fp8_encode(float value, int e5m2)
{
    return TileXREpDemo::EncodeFp8(value, Format(e5m2));
}

float ref_fp8_decode(uint8_t value, int e5m2)
{
    return TileXREpDemo::DecodeFp8(value, Format(e5m2));
}

// ---- no-NPU checker (tools/checker) ----
static tilexr::checker::CheckerCase MakeCase(int op, int rankSize, int64_t bs, int64_t h, int64_t topK,
    int64_t moeExpertNum, int dtype)
{
    tilexr::checker::CheckerCase c;
    c.op = op == 0 ? tilexr::checker::CollectiveOp::kEpDispatch : tilexr::checker::CollectiveOp::kEpCombine;
    c.rank_size = rankSize;
    c.server_count = 1;
    c.bs = bs;
    c.h = h;
    c.top_k = topK;
    c.moe_expert_num = moeExpertNum;
    c.data_type = static_cast<TileXR::TileXRDataType>(dtype);
    return c;
}

int64_t ref_checker_default_ids(int rankSize, int64_t bs, int64_t topK, int64_t moeExpertNum, int32_t *out)
{
    const auto c = MakeCase(0, rankSize, bs, 8, topK, moeExpertNum, TileXR::TILEXR_DATA_TYPE_FP16);
    const std::vector<int32_t> ids = tilexr::checker::DefaultEpDispatchExpertIds(c);
    if (out != nullptr) {
        std::memcpy(out, ids.data(), ids.size() * sizeof(int32_t));
    }
    return static_cast<int64_t>(ids.size());
}

// Routes a destination rank expects for arbitrary ids (all source ranks use the same id table).
// out = n x {src, token, k, expert}; returns n (call with out == nullptr to size).
int64_t ref_checker_routes(int rankSize, int64_t bs, int64_t topK, int64_t moeExpertNum, const int32_t *ids,
    int dstRank, int32_t *out)
{
    const auto c = MakeCase(0, rankSize, bs, 8, topK, moeExpertNum, TileXR::TILEXR_DATA_TYPE_FP16);
    const std::vector<int32_t> table(ids, ids + bs * topK);
    const auto routes = tilexr::checker::ExpectedEpDispatchRoutes(c, table, dstRank);
    if (out != nullptr) {
        for (std::size_t i = 0; i < routes.size(); ++i) {
            out[i * 4 + 0] = routes[i].src_rank;
            out[i * 4 + 1] = routes[i].token_id;
            out[i * 4 + 2] = routes[i].top_k_id;
            out[i * 4 + 3] = routes[i].expert_id;
        }
    }
    return static_cast<int64_t>(routes.size());
}

uint16_t ref_checker_input_value(int rank, int64_t token, int64_t hIndex)
{
    return tilexr::checker::EpDispatchInputValue(rank, token, hIndex);
}

int64_t ref_checker_output_bytes(int op, int rankSize, int64_t bs, int64_t h, int64_t topK, int64_t moeExpertNum,
    int dtype)
{
    const auto c = MakeCase(op, rankSize, bs, h, topK, moeExpertNum, dtype);
    return static_cast<int64_t>(op == 0 ? tilexr::checker::EpDispatchOutputBytes(c) :
                                           tilexr::checker::EpCombineOutputBytes(c));
}

// Runs the checker's ep_dispatch (op 0) or ep_combine (op 1) executor with its default inputs and copies every
// rank's flat output blob into out[rank * outputBytes ...].  Returns 0 when the checker passes with no mismatches.
int ref_checker_run(int op, int rankSize, int64_t bs, int64_t h, int64_t topK, int64_t moeExpertNum, int dtype,
    uint8_t *out, int64_t *eventCount)
{
    using namespace tilexr::checker;
    const CheckerCase c = MakeCase(op, rankSize, bs, h, topK, moeExpertNum, dtype);
    std::size_t inputBytes = 0;
    std::size_t outputBytes = 0;
    if (op == 0) {
        inputBytes = static_cast<std::size_t>(bs * h) * ElementSize(c.data_type);
        outputBytes = EpDispatchOutputBytes(c);
    } else {
        inputBytes = EpCombineInputBytes(c);
        outputBytes = EpCombineOutputBytes(c);
    }
    RankWorld world = RankWorld::Create(rankSize, inputBytes, outputBytes, op == 0 ? outputBytes : inputBytes);
    world.ConfigureServers(1);
    CollectiveExecutor executor;
    const RunResult result = executor.Run(&world, c);
    if (eventCount != nullptr) {
        *eventCount = static_cast<int64_t>(result.event_count);
    }
    if (!result.status.ok() || !result.mismatches.empty()) {
        return 1;
    }
    if (out != nullptr) {
        for (int rank = 0; rank < rankSize; ++rank) {
            const CheckerStatus st = world.UserOutput(rank).ReadBytes(0, out + rank * outputBytes, outputBytes);
            if (!st.ok()) {
                return 2;
            }
        }
    }
    return 0;
}

} // extern "C"
