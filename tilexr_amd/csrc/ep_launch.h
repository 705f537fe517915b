// Kernel launch interface between the host orchestration (api.cpp, multi_rank.cpp) and the HIP kernels (ep_count.hip,
// ep_scatter.hip, ep_reduce.hip).
//
// The data path of one dispatch is three launches on the caller's stream:
//   count   per-chunk stable rank of every route within its key + per-chunk key histogram; the last workgroup
//           to finish scans the histograms into per-chunk bases, per-key offsets and the count outputs
//   place   destination row of every route, assist tuples, inverse row map (folded into the scatter launch when
//           nothing has to be complete before the scatter starts)
//   scatter token rows read once and written to their topK destination rows (optionally quantised)
// and of one combine two launches:
//   invert  (skipped when the caller supplies the row map) row -> (token, k) inverse from the assist tuples
//   reduce  per token: gather rows, dequantise, weighted fp32 sum in k order, one rounding to the output type
// A "key" is what rows are grouped by: the expert (memory route), the destination rank (MVP route across logical
// ranks) or nothing (MVP route on one rank: plain compaction of live routes).
#ifndef TILEXR_AMD_EP_LAUNCH_H
#define TILEXR_AMD_EP_LAUNCH_H

#include <cstdint>

#include <hip/hip_runtime_api.h>

#include "ep_tile_publish.h"

namespace TileXREp {

constexpr int kMinChunkShift = 10;      // a counting workgroup handles 2^shift routes: 1024 ...
constexpr int kMaxChunkShift = 13;      // ... up to 8192, chosen so that about kTargetChunks workgroups run
constexpr int kTargetChunks = 128;      // (the last one to finish scans one histogram row per chunk: 64 from 1024 keys
                                        // on, where that scan is the longer part; 131 072 routes x 128 experts: count
                                        // launch 11.3 us with 64 chunks, 9.9 us with 128)
constexpr int kMaxKeys = 2048;          // keys (experts) the counting kernel's LDS tables hold
constexpr int kMaxTopK = 64;

enum MaskMode : int {
    kMaskNone = 0,
    kMaskPerToken = 1,      // route live iff mask[token]           (MVP route, combine)
    kMaskPerRoute = 2,      // route live iff mask[token, k]        (memory route, expert mask)
    kMaskTokenPrefix = 3,   // route live iff token < sum(mask)     (memory route, token mask)
};

struct CountScratch {
    int chunkShift;         // log2 of the routes per counting workgroup
    uint32_t *ticket;       // 1 word, zero between launches
    int32_t *localRank;     // [n]  rank of the route within (chunk, key); -1 when the route is not live
    int32_t *chunkHist;     // [chunks, numKeys] in: counts; out: exclusive sum over earlier chunks
    int32_t *chunkExpHist;  // [chunks, experts] only when keys are coarser than experts, else nullptr
    int32_t *keyOffset;     // [numKeys + 1] exclusive sum of kept rows per key
    int32_t *keyKept;       // [numKeys] rows kept per key (after capacity)
    int32_t *expertTotal;   // [experts] live routes per expert (before capacity when keys are coarser)
};

struct RouteCountLaunch {
    const int32_t *ids;
    const uint8_t *mask;
    int maskMode;
    int64_t bs;
    int64_t topK;
    int64_t numExperts;
    int64_t keyDiv;          // key = expert / keyDiv
    int64_t numKeys;
    int64_t capacity;        // rows kept per key, 0 = all
    CountScratch scratch;
    // outputs written by the last workgroup when non-null (single-rank fast path)
    int32_t *sendCountsOut;      // [numKeys] inclusive sum of kept rows
    int32_t *recvCountOut;       // [1] total kept rows
    int64_t *expertTokenNumsOut; // [experts]
    int tokenNumsType;
    // Token rows the scatter that follows will read: extra workgroups of this launch read them once while the counting
    // workgroups wait on their own small loads, which leaves the rows in the memory-side cache.  Null or 0: none.
    const void *warmRows;
    int64_t warmBytes;
    hipStream_t stream;
};

// Memory route, one rank, keys = experts, no mask, no capacity limit: rows and assist tuples of all routes in one launch
// (ep_rows.hip), for id tables small enough that every workgroup reads the whole table itself.
constexpr int kRowsTableRoutes = 262144;
struct RouteRowsLaunch {
    const int32_t *ids;
    int64_t bs;
    int64_t topK;
    int64_t numKeys;
    int32_t srcRank;
    int32_t expertIdBias;
    int32_t *rowOf;              // [n] out: row of each route, -1 = none
    int32_t *assist;             // [rows, 4] out
    int32_t *totalRowsOut;       // [1] out: rows kept
    int32_t *sendCountsOut;      // optional [numKeys] inclusive sum of kept rows
    int64_t *expertTokenNumsOut; // optional [numKeys]
    int tokenNumsType;
    const void *warmRows;        // as RouteCountLaunch
    int64_t warmBytes;
    hipStream_t stream;
};
bool RouteRowsPays(int64_t routes, int64_t numKeys, bool rowsAhead, bool readsRowsAhead);
bool RouteRowsFits(const int32_t *ids, int64_t routes, int64_t numKeys, int maskMode, int64_t capacity);
hipError_t LaunchRouteRows(const RouteRowsLaunch &l);

struct RoutePlaceLaunch {
    const int32_t *ids;
    int64_t bs;
    int64_t topK;
    int64_t keyDiv;
    int64_t numKeys;
    int64_t capacity;
    CountScratch scratch;
    int32_t srcRank;
    int32_t expertIdBias;        // added to the id stored in the assist tuple (shared experts shift ids)
    // Shared experts (logical multi-rank worlds): a token's routes are its `sharedNum` shared routes followed by
    // its routed ones, `topK` counts both, `ids` holds positions in the world's key space and `tupleExperts`
    // the expert id each route reports in its assist tuple.  The tuple's topKId is topK - sharedNum + s for
    // shared route s and the routed index otherwise.
    int32_t sharedNum;
    const int32_t *tupleExperts; // [n] or nullptr (the tuple then reports ids[i] + expertIdBias)
    int32_t *rowOf;              // [n] out
    int32_t *assist;             // [rows, 4] out
    hipStream_t stream;
};

struct ScatterLaunch {
    const void *x;
    const int32_t *rowOf;            // rows resolved by an earlier place launch, unless ...
    const RoutePlaceLaunch *fusedPlace;  // ... this is set: the scatter resolves them itself (rowOf output optional)
    int64_t bs;
    int64_t h;
    int64_t topK;
    int quantMode;               // TileXREpQuantMode
    bool inputBf16;              // decode of x when quantising
    bool fp8E5m2;
    const float *staticScale;
    void *out;                   // rows of h*2 bytes (mode 0) or h bytes
    void *scalesOut;             // fp32 [rows] (2), u8 [rows, mxScaleCount] (4), fp32 [rows, ceil(h/128)] (5)
    // Optional readiness words, one per `tileRows` rows: (epoch << 32) | rows in the tile, stored once, by whoever
    // lands the tile's last row, after every row of the tile is complete in memory.  Landed rows are counted in
    // `tileCounters` (library scratch, all zero between launches), never in the words consumers poll: a poll of a
    // word that atomics are hitting holds those atomics up (measured: 20 000 polls slow the scatter from 95 to
    // 215 us), a poll of a word that is stored once costs the producer nothing.
    uint64_t *tileFlags;
    uint32_t *tileCounters;      // TileCounterWords(bs * topK, tileRows) words
    int64_t tileRows;
    uint64_t epoch;
    const int32_t *totalRowsPtr; // device word: rows kept by this dispatch (size of the last tile)
    bool consumerBeside;         // a consumer of the flags is expected to run beside this launch (the caller asked for a
                                 // metadata-ready event): keep the workgroups small enough to fit next to its waiting ones
    const char **kernelNameOut;  // optional: receives the name of the kernel template that was launched
    hipStream_t stream;
};

struct InvertLaunch {
    const int32_t *assist;
    const int32_t *counts;       // device counts array
    int64_t numCounts;
    bool countsArePrefix;        // memory route: rows = counts[numCounts-1]; MVP: rows = sum(clamped counts)
    int64_t maxRows;
    int64_t maxCountPerEntry;    // MVP: entries outside [0, this] read as 0
    int32_t rank;
    int64_t bs;
    int64_t topK;
    uint64_t epoch;
    uint64_t *inverse;           // [bs*topK] (epoch << 32) | row
    hipStream_t stream;
};

enum ReduceKind : int {
    kReduceFp32 = 0,             // memory route: fp32 accumulate in k order, one rounding
    kReducePerAdd = 1,           // MVP route: accumulator rounded to the element type after every add, row order
};

struct ReduceLaunch {
    const void *expertOut;
    int64_t rowBytes;
    const uint64_t *inverseTagged;   // either this (with epoch) ...
    uint64_t epoch;
    const int32_t *rowIndexMap;      // ... or a plain row map (-1 = none) ...
    const InvertLaunch *assistTable; // ... or the assist table itself (LaunchSmallReduce only)
    const uint64_t *orderKeys;       // optional, per-add kind: rows are summed in ascending orderKeys[row]
    const float *expertScales;       // optional [bs, topK]
    const uint8_t *tokenMask;        // optional [bs]
    const void *sharedExpertX;       // optional [bs, h]
    int reduceKind;
    int commQuant;                   // 0, 3, 4
    int inQuant;                     // 0, 2, 5
    const float *inScales;
    bool bf16;
    int64_t bs;
    int64_t h;
    int64_t topK;
    int64_t maxRows;                 // rows expertOut holds: map entries at or beyond it count as "no row"; 0 = unchecked
    int64_t sharedSlots;             // slots per token beyond topK (shared experts): summed after the routed ones
                                     // with weight 1; the row map / inverse then has topK + sharedSlots entries
                                     // per token while expertScales keeps topK
    void *y;
    const uint64_t *tileFlags;       // optional: a tile is ready once the upper half of its word equals flagEpoch
    int64_t tileRows;
    uint64_t flagEpoch;
    uint32_t *claimWord;             // launches that may wait: two device words the workgroups claim their tokens from,
                                     // zero between launches (the last workgroup to leave puts them back)
    bool producerOrdered;            // the producer of the flags was enqueued earlier on this very stream: every wait
                                     // succeeds at its first poll, so the launch need not leave room for a producer
    int64_t waitTimeoutTicks;        // in wall_clock64 ticks
    int32_t *deviceStatus;
    int numComputeUnits;
    const char **kernelNameOut;      // optional: receives the name of the kernel template that was launched
    hipStream_t stream;
};

// Combine of a small batch (at most kSmallRoutes routes, 16-bit rows, no readiness flags) in a single launch: every
// token's workgroup finds its rows in the assist table itself, so no launch has to invert the table first.
bool SmallReduceFits(const ReduceLaunch &l);
hipError_t LaunchSmallReduce(const ReduceLaunch &l);

// Memory-route dispatch of a small batch (plain copies, one rank, no mask, no readiness flags) in a single launch:
// every workgroup counts the whole id table itself instead of waiting for a counting kernel.
constexpr int kSmallRoutes = 2048;
struct SmallDispatchLaunch {
    const void *x;
    const int32_t *ids;
    int64_t bs;
    int64_t h;
    int64_t topK;
    int64_t numExperts;
    int64_t capacity;
    int32_t srcRank;
    int32_t expertIdBias;
    void *out;
    int32_t *assist;
    int32_t *rowOf;                  // optional
    int32_t *sendCountsOut;
    int64_t *expertTokenNumsOut;
    int tokenNumsType;
    uint64_t *tileFlags;             // optional: a readiness word per tile of rows, as LaunchScatter publishes them
    uint32_t *tileCounters;          // TileCounterWords(bs * topK, tileRows) zeroed words
    int64_t tileRows;
    uint64_t epoch;
    hipStream_t stream;
    const char **kernelNameOut = nullptr;   // optional: receives the name of the kernel template that was launched
};
bool SmallDispatchFits(const SmallDispatchLaunch &l);
hipError_t LaunchSmallDispatch(const SmallDispatchLaunch &l);

hipError_t LaunchRouteCount(const RouteCountLaunch &l);
hipError_t LaunchRoutePlace(const RoutePlaceLaunch &l);
hipError_t LaunchScatter(const ScatterLaunch &l);
// Whether LaunchScatter copies rows with one workgroup per (route, slice), each reading its own copy of the token row
// (plain payload, wide rows, 1024 tokens and more).  That kernel is the one that needs the token rows close by: it is
// what RouteCountLaunch::warmRows is for.
bool ScatterCopiesPerRoute(const void *x, const void *out, int64_t bs, int64_t h, int64_t topK, int quantMode);
hipError_t LaunchInvert(const InvertLaunch &l);
hipError_t LaunchReduce(const ReduceLaunch &l);

// Bytes of CountScratch arrays for a problem (used by the host to carve one allocation).
struct CountScratchLayout {
    int chunkShift;
    int64_t chunks;
    int64_t localRankOff, chunkHistOff, chunkExpHistOff, keyOffsetOff, keyKeptOff, expertTotalOff, rowOfOff;
    int64_t totalBytes;
};
CountScratchLayout PlanCountScratch(int64_t routes, int64_t numKeys, int64_t numExperts, bool expertHist);

} // namespace TileXREp

#endif // TILEXR_AMD_EP_LAUNCH_H
