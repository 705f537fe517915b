// Launch interface of the plan-driven (MoonEP) dispatch / combine kernels (internal header).
//
// The reference moves rows through per-rank peer windows with magic-tagged barriers between "window cleared", "data
// ready" and "window drained" (src/moonep/dispatch/kernels/tilexr_moonep_dispatch_kernel.cpp:108-147,
// src/moonep/combine/kernels/tilexr_moonep_combine_kernel.cpp:117-177).  Here every rank of the world lives on one
// device, so a source rank writes straight into the destination rank's receive tensor and the only shared state is a
// set of small per-row tables in library scratch.  Every table entry carries the epoch of the call that wrote it in
// its upper 32 bits, so nothing is ever cleared between calls.
//
//   dispatch  scatter   (per source rank)       rows, weights, row tags, parent / sibling records of duplicates
//             build     (per destination rank)  fresh plans: dupGroups / dupLoffs / dupCounts from the parent records
//             walk      (per destination rank)  saved plans: parent records from dupGroups / dupLoffs
//             classify + fill (per destination) rows nobody named -> zero, duplicate rows of a saved plan -> copy of
//                                               their primary row; device status
//   combine   walk      (per expert rank)       duplicate mask and group-of-primary table
//             reverse   (per expert rank)       dstLocal -> slot table of the origin ranks
//             reduce    (per origin rank)       K slots per token, duplicate groups pre-summed, fp32 -> bf16
#ifndef TILEXR_AMD_MOONEP_STAGE_H
#define TILEXR_AMD_MOONEP_STAGE_H

#include <cstdint>

#include <hip/hip_runtime_api.h>

namespace TileXRMoon {

constexpr int kMaxWorld = 16;       // ranks of a world this library runs the stages for
constexpr int kMaxTopK = 32;        // reference: src/moonep/common/moonep_stage_layout.h:78
constexpr int kRowsPerGroup = 256;  // rows one classify workgroup looks at
constexpr int kFillSplit = 16;      // fill workgroups per classify group

// Device status values (reference: src/moonep/common/moonep_peer_window.h:36-43).
constexpr int32_t kDispatchOk = 2000;
constexpr int32_t kDispatchInvalidRoute = 2001;
constexpr int32_t kDispatchRemoteFailureBase = 2100;
constexpr int32_t kCombineOk = 0;
constexpr int32_t kCombineInvalidRoute = 3001;
constexpr int32_t kCombineRemoteFailureBase = 3100;

// Per-row tables of one world, each [world][nvS] unless noted; `stride` = entries per rank.
struct WorldTables {
    uint64_t *rowTag;        // dispatch: epoch << 32 | 2 (a route names the row) | 1 (a route wrote its hidden values)
    uint64_t *parentTag;     // dispatch: epoch << 32 | primary row + 1 when the row is a duplicate
    uint32_t *sibling;       // dispatch, fresh plans: rank among the duplicates of its primary | count << 16
    uint64_t *groupStart;    // dispatch, fresh plans: epoch << 32 | first dupLoffs index of the primary's group
    uint64_t *dupMask;       // combine: epoch << 32 | 1 when the row is a duplicate
    uint64_t *groupOf;       // combine: epoch << 32 | group index + 1 when the row is a primary with duplicates
    uint64_t *slotSrc;       // combine: [world][n] epoch << 32 | duplicate << 31 | expert rank * nvS + row
    uint64_t *fail;          // [world] epoch << 32 | device status of the rank's own failure
    int32_t *workList;       // dispatch: [world][nvS] rows the fill kernel has to write, grouped by classify group
    int32_t *workCount;      // dispatch: [world][groups]
    int64_t stride;          // >= nvS and >= n
    int64_t groupStride;     // classify groups per rank
};

struct ReceiveTable {
    void *hidden[kMaxWorld];       // hiddenNvsh of every rank
    float *weights[kMaxWorld];     // routeWeightsNvs of every rank (all null when weights are not exchanged)
};

struct ScatterLaunch {
    const int32_t *dst;            // [s * k]
    const void *hiddenSh;          // [s, h] bf16
    const float *weightsSk;        // [s * k] or null
    int64_t s, k, h, nvS;
    int world;
    int srcRank;
    bool fresh;                    // the duplicate plan is being built: duplicates are written here, with records
    ReceiveTable out;
    WorldTables tables;
    uint64_t epoch;
    hipStream_t stream;
};

struct DedupBuildLaunch {
    int64_t nvS;
    int rank;
    WorldTables tables;
    uint64_t epoch;
    int32_t *dupGroups;            // out [nvS, 3]
    int32_t *dupLoffs;             // out [nvS]
    int32_t *dupCounts;            // out [2]
    hipStream_t stream;
};

struct GroupWalkLaunch {
    int64_t nvS;
    int rank;
    bool combine;                  // fills dupMask / groupOf and rejects duplicate == primary; else fills parentTag
    const int32_t *dupGroups;
    const int32_t *dupLoffs;
    const int32_t *dupCounts;
    WorldTables tables;
    uint64_t epoch;
    hipStream_t stream;
};

struct FillLaunch {
    int64_t nvS, h;
    int world;
    int rank;
    bool expand;                   // saved plan: duplicate rows take a copy of their primary row
    void *hiddenNvsh;
    float *weightsNvs;             // or null
    WorldTables tables;
    uint64_t epoch;
    int32_t *status;               // plan->status
    hipStream_t stream;
};

struct ReverseLaunch {
    const int32_t *dstLocal;       // [nvS]
    int64_t nvS, n;
    int world;
    int rank;
    WorldTables tables;
    uint64_t epoch;
    hipStream_t stream;
};

struct SourceTable {
    const void *hidden[kMaxWorld];         // hiddenNvsh of every expert rank
    const float *weights[kMaxWorld];       // routeWeightsNvs of every expert rank, or null
    const int32_t *dupGroups[kMaxWorld];
    const int32_t *dupLoffs[kMaxWorld];
};

struct MoonReduceLaunch {
    int64_t s, k, h, nvS;
    int world;
    int rank;
    SourceTable src;
    WorldTables tables;
    uint64_t epoch;
    void *hiddenSh;                // out [s, h] bf16
    float *weightsSk;              // out [s * k] or null
    int32_t *status;
    int numComputeUnits;
    hipStream_t stream;
};

hipError_t LaunchMoonScatter(const ScatterLaunch &l);
hipError_t LaunchMoonDedupBuild(const DedupBuildLaunch &l);
hipError_t LaunchMoonGroupWalk(const GroupWalkLaunch &l);
hipError_t LaunchMoonFill(const FillLaunch &l);
hipError_t LaunchMoonReverse(const ReverseLaunch &l);
hipError_t LaunchMoonReduce(const MoonReduceLaunch &l);

// Names of the kernel templates the last scatter / reduce launch used (for the benchmark's roofline line).
const char *MoonScatterKernelName();
const char *MoonReduceKernelName();

} // namespace TileXRMoon

#endif // TILEXR_AMD_MOONEP_STAGE_H
