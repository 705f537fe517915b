// libtilexr-ep for one MI355X: MoE expert-parallel dispatch and combine.
//
// Part 1 declares the eight entry points of the reference's EP library (src/include/tilexr_ep.h:23-71) with the
// same names, argument order, argument meaning and return codes, so code written against that header links
// against this library unchanged.  `aclrtStream` is an opaque pointer there; here it carries a `hipStream_t`.
// All tensor arguments are caller-owned device memory (HBM), every call is asynchronous on `stream`, and
// validation happens before a magic is drawn or anything is enqueued (reference:
// src/ep/host/ep_kernel_launch.cpp:304-317).
//
// Part 2 declares additions that have no counterpart in the reference; each says so.
//
// Common contract (reference: src/ep/host/ep_host.h:17-78, src/ep/common/ep_window.h:47-52):
//   x                     [bs, h] fp16 / bf16, row-major
//   expertIds             [bs, topK] int32; ids outside [0, moeExpertNum) are skipped, not errors
//   expandXOut            [rows, h] rows gathered for this rank's experts (same type as x, or int8 / fp8)
//   assistInfoForCombine  [rows, 4] int32 = {srcRank, tokenId, topKId, expertId}
//   expertTokenNumsOut    [localExpertNum] int64; type 1 = counts, type 0 = inclusive prefix sum
//   counts                MVP route: epRecvCounts[srcRank] plain counts;
//                         memory route: sendCounts[localExpert * rankSize + srcRank] inclusive prefix sum
//   yOut                  [bs, h] combined rows in token order
// Row order on a destination rank: MVP route = source rank, token, topK; memory route = local expert, source rank,
// route order (expert-contiguous).
#ifndef TILEXR_EP_H
#define TILEXR_EP_H

#ifdef __cplusplus

#include <cstdint>

#include "tilexr_api.h"
#include "tilexr_types.h"

#ifndef TILEXR_EP_HAVE_ACL_STREAM
typedef void *aclrtStream;   // holds a hipStream_t
#endif

namespace TileXREp {

// reference: src/include/tilexr_ep.h:14-18
enum TileXREpActiveMaskType : int64_t {
    TILEXR_EP_ACTIVE_MASK_NONE = 0,
    TILEXR_EP_ACTIVE_MASK_TOKEN = 1,    // bool [bs]
    TILEXR_EP_ACTIVE_MASK_EXPERT = 2,   // bool [bs, topK] (memory-route dispatch only)
};

// quantMode values accepted by the entry points below
enum TileXREpQuantMode : int64_t {
    TILEXR_EP_QUANT_NONE = 0,
    TILEXR_EP_QUANT_STATIC_INT8 = 1,        // MVP dispatch: q = clamp(round(x * scales[0]))
    TILEXR_EP_QUANT_TOKEN_INT8 = 2,         // per-row absmax int8 with one fp32 scale per row
    TILEXR_EP_QUANT_COMM_MXFP8_E5M2 = 3,    // memory combine: rows cross the exchange as MXFP8 e5m2
    TILEXR_EP_QUANT_MXFP8 = 4,              // memory dispatch: MXFP8 output; memory combine: MXFP8 e4m3 exchange
    TILEXR_EP_QUANT_FP8_BLOCK128 = 5,       // Part 2 only: fp8 e4m3 with one fp32 scale per 128 columns
};

} // namespace TileXREp

extern "C" {
#pragma GCC visibility push(default)   // the entry points below are what the shared library exports

// ---------------------------------------------------------------------------------------------------------
// Part 1: the reference's entry points
// ---------------------------------------------------------------------------------------------------------

// reference: src/include/tilexr_ep.h:25-28, src/ep/host/tilexr_ep_dispatch.cpp:85-94
int TileXRMoeEpDispatch(void *x, int32_t *expertIds, TileXRCommPtr comm,
    int64_t bs, int64_t h, int64_t topK, int64_t moeExpertNum,
    void *expandXOut, int64_t *expertTokenNumsOut, int32_t *epRecvCountsOut,
    int32_t *assistInfoForCombineOut, TileXR::TileXRDataType dtype, aclrtStream stream);

// reference: src/include/tilexr_ep.h:30-33, src/ep/host/tilexr_ep_memory_dispatch.cpp:73-82
int TileXRMoeEpDispatchMemory(void *x, int32_t *expertIds, TileXRCommPtr comm,
    int64_t bs, int64_t h, int64_t topK, int64_t moeExpertNum,
    void *expandXOut, int64_t *expertTokenNumsOut, int32_t *sendCountsOut,
    int32_t *assistInfoForCombineOut, TileXR::TileXRDataType dtype, aclrtStream stream);

// reference: src/include/tilexr_ep.h:35-37, src/ep/host/tilexr_ep_dispatch.cpp:96-102
int TileXRMoeEpCombine(void *expertOut, int32_t *assistInfoForCombine, int32_t *epRecvCounts,
    TileXRCommPtr comm, int64_t bs, int64_t h, int64_t topK, int64_t moeExpertNum,
    void *yOut, TileXR::TileXRDataType dtype, aclrtStream stream);

// reference: src/include/tilexr_ep.h:39-41, src/ep/host/tilexr_ep_memory_combine.cpp:61-68
int TileXRMoeEpCombineMemory(void *expertOut, int32_t *assistInfoForCombine, int32_t *epRecvCounts,
    TileXRCommPtr comm, int64_t bs, int64_t h, int64_t topK, int64_t moeExpertNum,
    void *yOut, TileXR::TileXRDataType dtype, aclrtStream stream);

// reference: src/include/tilexr_ep.h:43-45, src/ep/host/tilexr_ep_dispatch.cpp:104-123
int TileXRMoeEpCombineV2(void *expertOut, int32_t *assistInfoForCombine, int32_t *epRecvCounts,
    TileXRCommPtr comm, int64_t bs, int64_t h, int64_t topK, int64_t moeExpertNum,
    void *yOut, void *workspace, TileXR::TileXRDataType dtype, aclrtStream stream);

// reference: src/include/tilexr_ep.h:47-52, src/ep/host/tilexr_ep_memory_combine.cpp:25-59
int TileXRMoeEpCombineMemoryV2(void *expertOut, int32_t *assistInfoForCombine, int32_t *sendCounts,
    float *expertScales, bool *xActiveMask, int64_t activeMaskType, void *sharedExpertX,
    TileXRCommPtr comm, int64_t bs, int64_t h, int64_t topK, int64_t moeExpertNum,
    int64_t epWorldSize, int64_t epRankId, int64_t tpWorldSize, int64_t tpRankId,
    int64_t expertShardType, int64_t sharedExpertNum, int64_t sharedExpertRankNum,
    int64_t quantMode, int64_t globalBs, void *yOut, TileXR::TileXRDataType dtype, aclrtStream stream);

// reference: src/include/tilexr_ep.h:54-60, src/ep/host/tilexr_ep_dispatch.cpp:42-83
int TileXRMoeEpDispatchV2(void *x, int32_t *expertIds, void *scales, bool *xActiveMask, void *expertScales,
    TileXRCommPtr comm, int64_t bs, int64_t h, int64_t topK, int64_t moeExpertNum, int64_t epWorldSize,
    int64_t epRankId, int64_t tpWorldSize, int64_t tpRankId, int64_t expertShardType, int64_t sharedExpertNum,
    int64_t sharedExpertRankNum, int64_t quantMode, int64_t globalBs, int64_t expertTokenNumsType, void *expandXOut,
    void *dynamicScalesOut, int32_t *assistInfoForCombineOut, int64_t *expertTokenNumsOut, int32_t *epRecvCountsOut,
    int32_t *tpRecvCountsOut, void *expandScalesOut, void *workspace, TileXR::TileXRDataType dtype,
    aclrtStream stream);

// reference: src/include/tilexr_ep.h:62-69, src/ep/host/tilexr_ep_memory_dispatch.cpp:27-71
int TileXRMoeEpDispatchMemoryV2(void *x, int32_t *expertIds, void *scales, bool *xActiveMask,
    int64_t activeMaskType, void *expertScales, TileXRCommPtr comm, int64_t bs, int64_t h, int64_t topK,
    int64_t moeExpertNum,
    int64_t epWorldSize, int64_t epRankId, int64_t tpWorldSize, int64_t tpRankId, int64_t expertShardType,
    int64_t sharedExpertNum, int64_t sharedExpertRankNum, int64_t quantMode, int64_t globalBs,
    int64_t expertTokenNumsType, void *expandXOut, void *dynamicScalesOut, int32_t *assistInfoForCombineOut,
    int64_t *expertTokenNumsOut, int32_t *sendCountsOut, int32_t *tpRecvCountsOut, void *expandScalesOut,
    TileXR::TileXRDataType dtype, TileXR::TileXRDataType expandXOutDtype, aclrtStream stream);

// ---------------------------------------------------------------------------------------------------------
// Part 2: additions without a counterpart in the reference
// ---------------------------------------------------------------------------------------------------------

// Options of the extended memory-route calls.  Zero-initialise, then set what is needed.
struct TileXREpDispatchExOptions {
    int64_t quantMode;            // 0, 2 (input decoded by `dtype`), 4, 5
    int64_t expertCapacity;       // > 0: a source rank sends at most this many rows per expert, lowest flat
                                  //      route indices first; dropped routes get no row
    int64_t expertTokenNumsType;  // 0 prefix sum, 1 counts
    int64_t activeMaskType;
    bool *xActiveMask;
    int32_t *rowIndexMapOut;      // optional [bs, topK]: row of each route in expandXOut, -1 when it has none
    uint64_t *tileFlagsOut;       // optional readiness words, one per `tileRows` rows of expandXOut: a word
                                  //      becomes (epoch << 32) | rows in the tile, in one store, once every row of
                                  //      the tile (payload and scales) is complete in memory for every compute
                                  //      unit; until then it holds whatever an earlier epoch left (never cleared)
    int64_t tileRows;             // 1 .. 2^31 - 1 when tileFlagsOut is set; values above bs * topK name one tile
    int64_t *epochOut;            // optional host pointer: receives the epoch the flags are tagged with.  Epochs
                                  //      are 32 bits wide, never 0 and drawn from one counter for the whole process,
                                  //      so flag arrays may be shared by communicators; a zero-filled array is
                                  //      "not ready" for every epoch
    void *metaReadyEvent;         // optional hipEvent_t recorded on `stream` once counts, assist tuples,
                                  //      rowIndexMapOut and the reset flag words are enqueued (before rows move)
};

// Memory-route dispatch (same outputs and order as TileXRMoeEpDispatchMemoryV2) for one rank per device, with
// per-token int8 / block fp8 payloads, per-expert capacity and tile readiness flags.  No reference counterpart:
// the reference's memory route accepts quantMode 0 and 4 only and has no capacity or caller-visible flags.
int TileXRMoeEpDispatchMemoryEx(void *x, int32_t *expertIds, TileXRCommPtr comm, int64_t bs, int64_t h,
    int64_t topK, int64_t moeExpertNum, const TileXREpDispatchExOptions *options, void *expandXOut,
    void *dynamicScalesOut, int32_t *assistInfoForCombineOut, int64_t *expertTokenNumsOut, int32_t *sendCountsOut,
    TileXR::TileXRDataType dtype, TileXR::TileXRDataType expandXOutDtype, aclrtStream stream);

struct TileXREpCombineExOptions {
    int64_t commQuantMode;        // 0, 3, 4: as quantMode of TileXRMoeEpCombineMemoryV2
    int64_t expertOutQuantMode;   // 0: expertOut is `dtype`; 2 / 5: expertOut holds int8 / fp8 e4m3 rows that are
                                  //    dequantised with expertOutScales, rounded to `dtype`, then reduced
    void *expertOutScales;        // fp32 [rows] (mode 2) or [rows, ceil(h/128)] (mode 5)
    float *expertScales;          // optional gate weights [bs, topK]
    int64_t activeMaskType;       // NONE or TOKEN
    bool *xActiveMask;
    void *sharedExpertX;          // optional [bs, h]
    const int32_t *rowIndexMap;   // optional [bs, topK] from dispatch: skips rebuilding the inverse map
    const uint64_t *tileFlags;    // optional: before a row is read, wait until the upper half of its tile's word
                                  //      equals flagEpoch; the rows are then read from memory, not from a cache.
                                  //      A producer other than the dispatch above (an expert stage) publishes
                                  //      its tiles with the device functions of tilexr_ep_publish.hip.h (installed
                                  //      beside this header; it states the ordering rule and holds the one
                                  //      implementation of the release that is waited for).  The producer's
                                  //      work must be enqueued BEFORE this call: streams of a process may share a
                                  //      hardware queue, where a waiting kernel keeps later kernels behind it
                                  //      Waiting workgroups stay resident (two per compute unit): a producer
                                  //      that runs beside them needs room for at least one workgroup of its own
                                  //      on the compute units, or the waits expire
    int64_t tileRows;             // 1 .. 2^31 - 1 when tileFlags is set
    int64_t flagEpoch;            // epoch the producer tags its flag words with
    int64_t waitTimeoutUs;        // bound of every flag wait; 0 = library default (2 s)
    int32_t *deviceStatusOut;     // device int32, required with tileFlags (-3 without it): set to 1 when a flag
                                  //      wait expired; the waits that follow in that launch give up at once.  A
                                  //      token with an expired wait gets a row of zeros in yOut, never a partial sum.
                                  //      The caller clears the word before the call.  A combine on the stream of
                                  //      the very dispatch that published these flags (same array, same epoch)
                                  //      never waits, its producer being done before it starts: a word that is
                                  //      not there then counts as expired at once
};

// Memory-route combine (same result as TileXRMoeEpCombineMemoryV2) with quantised expert output, a ready-made
// inverse map and tile readiness flags, so tiles can be reduced as soon as the expert stage publishes them.
// No reference counterpart: there the flag protocol is private to the kernels.
int TileXRMoeEpCombineMemoryEx(void *expertOut, int32_t *assistInfoForCombine, int32_t *sendCounts,
    TileXRCommPtr comm, int64_t bs, int64_t h, int64_t topK, int64_t moeExpertNum,
    const TileXREpCombineExOptions *options, void *yOut, TileXR::TileXRDataType dtype, aclrtStream stream);

// TileXRMoeEpDispatchMemory for callers that cannot allocate device memory at call time.  No counterpart in the
// reference.  It is for code under HIP graph capture, serving loops that have handed all device memory to a pool of
// their own, and harnesses that forbid hipMalloc: this call makes no hipMalloc / hipFree and calls no allocating
// library routine.  Arguments, outputs, order of rows and return codes are those of TileXRMoeEpDispatchMemory; the
// caller still passes every input and output.  What differs is where the kernels' scratch (per-route ranks, per-chunk
// histograms, per-expert offsets) lives: in one static array of 2 MiB that every GPU the library runs on holds until
// the process ends, instead of a buffer the communicator allocates and grows.
//   * limits: rankSize 1; bs * topK routes and moeExpertNum experts whose count scratch fits the array (131 072 routes
//     over 2048 experts do; about 8.3 bytes per route + 264 bytes per expert and 1024-route chunk).  Larger calls
//     return TILEXR_ERROR_NOT_SUPPORT (-6) with a line on stderr that names the sizes, before a magic is drawn.
//   * all calls on one GPU share that GPU's array, whatever their communicator or stream: calls that overlap in time
//     on one GPU race on it.  Calls that follow one another on a stream, or are otherwise ordered, are fine; the array
//     keeps the previous call's contents and the call clears what it needs cleared itself.
//   * the array's device address is resolved when a communicator is created on the device (TileXRCommInitRankLocal);
//     -1 (TILEXR_ERROR_NOT_INITIALIZED) if that failed.
int TileXRMoeEpDispatchMemoryNoAlloc(void *x, int32_t *expertIds, TileXRCommPtr comm,
    int64_t bs, int64_t h, int64_t topK, int64_t moeExpertNum,
    void *expandXOut, int64_t *expertTokenNumsOut, int32_t *sendCountsOut,
    int32_t *assistInfoForCombineOut, TileXR::TileXRDataType dtype, aclrtStream stream);

// Measurement aid without a reference counterpart: while a pair of hipEvent_t is set for a kernel, every call on
// `comm` that launches that kernel records `startEvent` immediately before and `stopEvent` immediately after it, on
// the stream of the call.  Pass null events to clear.  Kernel ids: 0 count, 1 place, 2 scatter, 3 invert, 4 reduce.
// Ids 2 and 4 also cover the scatter and reduce kernels of the plan-driven stages (tilexr_moonep.h).
int TileXREpSetKernelTimingEvents(TileXRCommPtr comm, int kernel, void *startEvent, void *stopEvent);

// Debug aids without a reference counterpart as an API (the reference's kernels leave breadcrumbs of the same kind:
// RunPosRecord, src/ep/kernels/tilexr_ep_dispatch_memory_kernel.h:1319-1328).  Stamps cover every kernel a call on
// `comm` launches; the poison fill applies to the dispatches of a one-rank communicator.  Null options switch both off.
struct TileXREpDebugOptions {
    uint64_t *phaseStamps;        // optional device ring of phaseStampCapacity records of four uint64 each:
                                  //   {magic of the call, kernel id (as TileXREpSetKernelTimingEvents), edge: 0 written
                                  //   by a one-thread kernel enqueued ahead of that kernel / 1 behind it, device clock
                                  //   (100 MHz ticks)}.  Records are written in call order, record i at index
                                  //   i % phaseStampCapacity; after a wait that expired, or a run that never came back,
                                  //   the ring says which phase was reached and how long each took on the device
    int64_t phaseStampCapacity;   // > 0 exactly when phaseStamps is set, at most 2^24
    int64_t poisonUnwrittenRows;  // non-zero: a dispatch first fills every row it may write (bs * topK of them, or
                                  //   moeExpertNum * expertCapacity when that is less), their assist tuples and their
                                  //   scales with 0x7f bytes (bf16 3.4e38, int8 127, the e4m3 NaN code, int32
                                  //   2139062143), so that a row which was counted but never written cannot pass for
                                  //   data.  Costs a full pass over the output buffers
};
int TileXREpSetDebugOptions(TileXRCommPtr comm, const TileXREpDebugOptions *options);

// Measurement aid without a reference counterpart: name of the kernel template the last call on `comm` launched
// for a kernel id (the data kernels have several templates, chosen by row width, alignment and payload type), so
// that a harness can match its event timings with a profiler's per-kernel rows.  Null before the first launch.
const char *TileXREpLastKernelName(TileXRCommPtr comm, int kernel);

// Library build identification ("tilexr-ep gfx950 <abi version>").
const char *TileXREpVersion(void);

#pragma GCC visibility pop
}

#endif // __cplusplus

#endif // TILEXR_EP_H
