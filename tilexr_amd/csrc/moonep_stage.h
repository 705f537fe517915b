// Launch interface of the plan-driven (MoonEP) dispatch / combine kernels (internal header).
//
// The reference moves rows through per-rank peer windows with magic-tagged barriers between "window cleared", "data
// ready" and "window drained" (src/moonep/dispatch/kernels/tilexr_moonep_dispatch_kernel.cpp:108-147,
// src/moonep/combine/kernels/tilexr_moonep_combine_kernel.cpp:117-177).  Here every rank of the world lives on one
// device, so a source rank writes straight into the destination rank's receive tensor, and one launch of each kernel
// covers every rank of the world (grid dimension y = rank).  The only shared state is a set of small per-row tables in
// library scratch; every table entry carries the epoch of the call that wrote it in its upper 32 bits, so nothing is
// ever cleared between calls.
//
//   dispatch  walk      saved plans: parent records from dupGroups / dupLoffs
//             agree     saved plans: per duplicate route, whether the plan's primary is the token's own primary row
//             records   fresh plans of smaller worlds: what the routes record (below), ahead of the scatter, in the
//                       launch that reads the token rows ahead; the plan is then built by extra workgroups of the
//                       scatter launch instead of by launches after it
//             scatter   rows, weights, row tags; fresh plans: parent / sibling records of duplicates
//             build     fresh plans: dupGroups / dupCounts from the parent records
//             finish    per row: what is left to write (zeros, or a copy of the primary of a saved plan) and writing it;
//                       dupLoffs of a fresh plan; weights of unnamed rows; device status
//   combine   prepare   dstLocal and the duplicate plan -> per-slot tables of the origins (which row, duplicate or not,
//                       its duplicate group)
//             reduce    K slots per token, duplicate groups pre-summed, fp32 -> bf16; device status
#ifndef TILEXR_AMD_MOONEP_STAGE_H
#define TILEXR_AMD_MOONEP_STAGE_H

#include <cstdint>

#include <hip/hip_runtime_api.h>

namespace TileXRMoon {

constexpr int kMaxWorld = 16;       // ranks of a world this library runs the stages for
constexpr int kMaxTopK = 32;        // reference: src/moonep/common/moonep_stage_layout.h:78
constexpr int kTableAlign = 256;    // per-rank table strides are a multiple of this many entries
constexpr int kChunkRows = 2048;    // rows per workgroup of the duplicate-plan build

// Device status values (reference: src/moonep/common/moonep_peer_window.h:36-43).
constexpr int32_t kDispatchOk = 2000;
constexpr int32_t kDispatchInvalidRoute = 2001;
constexpr int32_t kDispatchRemoteFailureBase = 2100;
constexpr int32_t kCombineOk = 0;
constexpr int32_t kCombineInvalidRoute = 3001;
constexpr int32_t kCombineRemoteFailureBase = 3100;

// Per-row tables of one world, each [world][stride] unless noted.
struct WorldTables {
    uint64_t *rowTag;        // dispatch: epoch << 32 | bits: a route names the row, a route wrote its hidden values,
                             //           the source wrote it as a duplicate the saved plan agrees with
    uint64_t *parentTag;     // dispatch: epoch << 32 | primary row + 1 when the row is a duplicate
    uint32_t *sibling;       // dispatch, fresh plans: rank among the duplicates of its primary | count << 16
    uint64_t *groupStart;    // dispatch, fresh plans: epoch << 32 | first dupLoffs index of the primary's group
    uint64_t *slotSrc;       // combine: per origin slot, epoch << 32 | expert rank * nvS + row of the row returned to it
    uint64_t *slotDup;       // combine: per origin slot, epoch << 32 | 1 when that row is a duplicate (it does not travel)
    uint64_t *slotGroup;     // combine: per origin slot, epoch << 32 | first dupLoffs index when that row has duplicates
    int32_t *slotCount;      // combine: per origin slot, number of those duplicates (valid with slotGroup)
    uint8_t *direct;         // dispatch, saved plans: per source route, 1 when the source writes the duplicate's row itself
                             //           (rewritten for every route by every saved-plan dispatch)
    uint64_t *fail;          // [world] epoch << 32 | device status of the rank's own failure
    int32_t *chunkTotals;    // dispatch, fresh plans: [world][groupStride][2] group-opening rows and duplicates per chunk
    int64_t stride;          // >= nvS and >= n, a multiple of kTableAlign
    int64_t groupStride;     // chunks per rank
};

// One Dispatch of every rank of a world.
struct DispatchWorld {
    int world;
    int64_t s, k, h, nvS;
    bool fresh;                                // the duplicate plan is built by this call
    uint64_t epoch;
    WorldTables tables;
    const int32_t *dst[kMaxWorld];             // [s * k] route words
    const void *hiddenSh[kMaxWorld];           // [s, h] bf16
    const float *weightsSk[kMaxWorld];         // [s * k], or all null
    void *hiddenNvsh[kMaxWorld];               // out [nvS, h] bf16
    float *weightsNvs[kMaxWorld];              // out [nvS]
    int32_t *dupGroups[kMaxWorld];             // [nvS, 3]  out when fresh, else in
    int32_t *dupLoffs[kMaxWorld];              // [nvS]
    int32_t *dupCounts[kMaxWorld];             // [2]
    int32_t *status[kMaxWorld];
};

// One Combine of every rank of a world.
struct CombineWorld {
    int world;
    int64_t s, k, h, nvS;
    uint64_t epoch;
    WorldTables tables;
    const int32_t *dstLocal[kMaxWorld];        // [nvS]
    const void *hiddenNvsh[kMaxWorld];         // [nvS, h] bf16
    const float *weightsNvs[kMaxWorld];        // [nvS], or all null
    const int32_t *dupGroups[kMaxWorld];
    const int32_t *dupLoffs[kMaxWorld];
    const int32_t *dupCounts[kMaxWorld];
    void *hiddenSh[kMaxWorld];                 // out [s, h] bf16
    float *weightsSk[kMaxWorld];               // out [s * k]
    int32_t *status[kMaxWorld];
};

// Optional (start, stop) events recorded around the scatter / reduce launch.
struct LaunchTiming {
    hipEvent_t start = nullptr;
    hipEvent_t stop = nullptr;
};

hipError_t LaunchMoonDispatch(const DispatchWorld &w, hipStream_t stream, const LaunchTiming &scatterTiming);
hipError_t LaunchMoonCombine(const CombineWorld &w, hipStream_t stream, const LaunchTiming &reduceTiming);

// Stores one device status word in stream order.
hipError_t LaunchMoonStatus(int32_t *status, int32_t value, hipStream_t stream);

// Bytes of token rows (all ranks of a world together) up to which the scatter assumes that they are still in the
// device's memory-side cache when it runs; returns the previous value.  Default 256 MiB.
int64_t SetCachedRowBytes(int64_t bytes);

// Names of the kernel templates the last scatter / reduce launch used (for the benchmark's roofline line).
const char *MoonScatterKernelName();
const char *MoonReduceKernelName();

} // namespace TileXRMoon

#endif // TILEXR_AMD_MOONEP_STAGE_H
