// Launch interface of the exchange kernels used when several logical ranks share the device (rankSize > 1).
//
// A multi-rank dispatch is two halves.  The source rank's call groups its rows by destination into a staging area
// (the same count / place / scatter kernels as the single-rank path, writing to staging instead of expandXOut).
// Once every rank has sent, each destination rank's outputs are assembled ("drained") from all staging areas:
//   plan   per-segment counts -> count outputs + exclusive offsets, one workgroup
//   copy   one workgroup per output row: locate its segment, copy row, assist tuple and scales
// A multi-rank combine is the transpose: every expert rank returns its rows to per-(token, k) slots of the source
// ranks ("return"), then each source rank runs the ordinary reduce kernel over its slots.
#ifndef TILEXR_AMD_EP_EXCHANGE_H
#define TILEXR_AMD_EP_EXCHANGE_H

#include <cstdint>

#include <hip/hip_runtime_api.h>

namespace TileXREp {

// Staging of one world: every per-source area has the same size, so kernels address areas arithmetically.
struct StageLayout {
    char *rows;              // [R] x rowsStride bytes: payload rows grouped by key
    int64_t rowsStride;
    char *aux;               // [R] x auxStride bytes: assist tuples [n,4] int32, then per-row scales
    int64_t auxStride;
    int64_t scalesOffset;    // offset of the scales inside an aux area
    int32_t *counts;         // [R] x countsStride ints: keyOffset[numKeys+1], expertTotal[E]
    int64_t countsStride;
    int64_t expertTotalOffset;   // in ints
};

// Builds the per-source route tables of a dispatch with shared experts: for every token its sharedNum shared routes
// followed by its topK routed ones, as positions in the world's key space (rank * keysPerRank + local index).
struct AugmentLaunch {
    const int32_t *ids;      // [bs, topK]
    int64_t bs;
    int64_t topK;
    int64_t moeExpertNum;
    int rankSize;
    int srcRank;
    int sharedNum;
    int sharedRanks;
    int localExperts;        // routed experts per non-shared rank
    int keysPerRank;
    bool sharedAtExpertId;   // local index of shared route s on its rank: s (MVP route) or 0 (memory route)
    int32_t *keyIdsOut;      // [bs, sharedNum + topK]; -1 = not routed
    int32_t *tupleExpertsOut;// [bs, sharedNum + topK]
    const uint8_t *routeMask;    // optional [bs, topK] expert mask ...
    uint8_t *routeMaskOut;       // ... widened to [bs, sharedNum + topK]: a token's shared routes are live when the
                                 // token keeps at least one routed expert
    hipStream_t stream;
};

struct DrainPlanLaunch {
    StageLayout stage;
    int rankSize;
    int dstRank;
    int localExperts;        // keys per rank in the staging areas' key space
    int outLocalExperts;     // memory route: segments per source on this rank (1 on a shared-expert rank)
    int tokenNumsCount;      // entries of expertTokenNumsOut
    int tp;                  // MVP route: lanes per tensor-parallel group (<= 1: none)
    bool memoryRoute;        // segments (localExpert, src) with inclusive-sum counts, else (src) with plain counts
    int32_t *planOffsets;    // [numSeg + 1] exclusive offsets (scratch of the destination rank)
    int32_t *countsOut;
    int32_t *tpCountsOut;    // optional mirror of countsOut (MVP route)
    int64_t *expertTokenNumsOut;
    int tokenNumsType;
    hipStream_t stream;
};

struct DrainCopyLaunch {
    StageLayout stage;
    int rankSize;
    int dstRank;
    int localExperts;
    int outLocalExperts;
    int tp;
    bool memoryRoute;
    const int32_t *planOffsets;
    int64_t maxRows;
    int64_t rowBytes;
    int64_t scaleBytesPerRow;
    void *expandXOut;
    int32_t *assistOut;
    void *scalesOut;
    hipStream_t stream;
};

struct ReturnRowsLaunch {
    const void *expertOut;
    const int32_t *assist;
    const int32_t *counts;
    int64_t numCounts;
    bool memoryRoute;
    int64_t maxCountPerEntry;
    int64_t maxRows;
    int64_t rowBytes;
    int rankSize;
    int expertRank;          // the calling rank
    int64_t bs;
    int64_t topK;            // slots per token: rows whose topKId is not below it are skipped
    uint64_t epoch;
    char *slots;             // [R] x slotsStride: rows at slot token*topK + k of the source rank
    int64_t slotsStride;
    uint64_t *meta;          // [R] x metaStride words: inverse (epoch << 32 | slot), then order keys
    int64_t metaStride;      // in words
    hipStream_t stream;
};

hipError_t LaunchAugment(const AugmentLaunch &l);
hipError_t LaunchDrainPlan(const DrainPlanLaunch &l);
hipError_t LaunchDrainCopy(const DrainCopyLaunch &l);
hipError_t LaunchReturnRows(const ReturnRowsLaunch &l);

} // namespace TileXREp

#endif // TILEXR_AMD_EP_EXCHANGE_H
