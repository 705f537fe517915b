/*
 * Plan-driven MoE dispatch / combine ("MoonEP" stages) for ranks that share one MI355X.
 *
 * The reference's libtilexr-moonep exposes five stages behind versioned argument structures
 * (src/include/tilexr_moonep.h:1-309).  This header declares the two stages that move token rows -- Dispatch and
 * Combine, V1 argument structures -- with the reference's names, structure layouts, flag values and return codes, so a
 * caller of those two stages links against this library unchanged.  Planning, PrefetchWeight and ReduceGrad are not
 * part of this library: they are not declared, and the capability calls report them in neither set.
 *
 * What the two stages do (reference: src/moonep/dispatch/design.md, src/moonep/combine/design.md):
 *
 *   A plan gives every route (token t, slot j) of a rank one signed 32-bit word dst[t * K + j].
 *       raw  = dst >= 0 ? dst : -dst - 1        rank = raw / NvS        row = raw % NvS
 *   Dispatch copies token t's hidden row to row `row` of rank `rank`'s receive tensor hiddenNvsh [NvS, H] and the
 *   route's weight to routeWeightsNvs[row].  A negative word marks a DUPLICATE: an earlier route of the same token
 *   already goes to that rank, so the row is not sent again; the destination fills it from that earlier ("primary")
 *   row.  The duplicate plan {dupGroups, dupLoffs, dupCounts} lists, per destination rank, each primary row with its
 *   duplicates; Dispatch builds it when TILEXR_MOONEP_FLAG_BUILD_DEDUP is set and consumes it as given otherwise.
 *   Rows of hiddenNvsh / routeWeightsNvs that no route names are set to zero.
 *
 *   Combine is the inverse.  dstLocal [NvS] names, for every receive row of the calling rank, the origin
 *   (rank * NvS + t * K + j) it returns to, or -1.  Each duplicate group is first summed into its primary row in fp32
 *   and rounded to bf16; duplicate rows are not returned.  The origin then sums its K slots in slot order in fp32
 *   (missing slots count as zero) and rounds once to bf16 into hiddenSh [S, H]; weights come back unchanged into
 *   routeWeightsSk [S, K] (zero where nothing was returned).
 *
 * All tensors are caller-owned device memory; every call is asynchronous on `stream` (a hipStream_t carried as the
 * reference's opaque aclrtStream); validation happens before a magic is drawn or anything is enqueued.  With more than
 * one rank in the communicator's world every rank must make the call (any order, any host thread, its own stream): a
 * rank's outputs are complete once all ranks have called and its stream has been synchronised.  The ranks of a world
 * must agree on S, K, H, NvS, the flags and on whether weights travel.  A call that disagrees with the calls already
 * filed for the same exchange returns INVALID_ARGUMENT and cancels them: each cancelled rank finds the remote-failure
 * status naming the disagreeing rank in its plan->status[0] (stored in the order of its stream), its outputs are left
 * as they were, and every rank has to call again.  A second call of one rank while its first still waits for its
 * peers returns INTERNAL.
 *
 * Differences from the reference, all deliberate:
 *   - a world of ONE rank is accepted by both stages (the reference's combine needs at least two,
 *     src/moonep/common/moonep_combine_schedule.h:166-171); worlds above 16 ranks return NOT_SUPPORTED;
 *   - the registered-workspace (URMA) variant of Dispatch (registeredWorkspace != NULL, or DispatchV2) returns
 *     NOT_SUPPORTED: there is no second device to register memory with;
 *   - no row passes through a peer window, so the window-capacity checks of the reference's layout code
 *     (src/moonep/dispatch/host/dispatch_layout.cpp:63-108) do not apply and hidden rows are never chunked.
 */
#ifndef TILEXR_MOONEP_H
#define TILEXR_MOONEP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#pragma GCC visibility push(default)   // the entry points below are what the shared library exports
#endif

#ifndef TILEXR_EP_HAVE_ACL_STREAM
typedef void *aclrtStream;   /* holds a hipStream_t */
#endif

typedef void *TileXRCommPtr;

/* reference: src/include/tilexr_moonep.h:16-27 */
#define TILEXR_MOONEP_ABI_VERSION_V1 UINT32_C(1)
#define TILEXR_MOONEP_ABI_VERSION_V2 UINT32_C(2)
#define TILEXR_MOONEP_MAX_TENSOR_RANK UINT32_C(4)
#define TILEXR_MOONEP_FLAG_NONE UINT64_C(0)
#define TILEXR_MOONEP_FLAG_BUILD_DEDUP (UINT64_C(1) << 0)           /* Dispatch: build the duplicate plan */
#define TILEXR_MOONEP_FLAG_SKIP_INTER_RANK_SYNC (UINT64_C(1) << 1)  /* Dispatch: accepted, no effect here */
#define TILEXR_MOONEP_FLAG_ZERO_COPY (UINT64_C(1) << 2)             /* both stages: NOT_SUPPORTED, as in the reference */
#define TILEXR_MOONEP_FLAG_COMBINE_PUBLISH_ONLY (UINT64_C(1) << 3)  /* Combine: INVALID_ARGUMENT, as in the reference */
#define TILEXR_MOONEP_FLAG_COMBINE_CONSUME_ONLY (UINT64_C(1) << 4)  /* Combine: INVALID_ARGUMENT, as in the reference */
#define TILEXR_MOONEP_FLAG_RESET_STATUS (UINT64_C(1) << 5)

/* reference: src/include/tilexr_moonep.h:29-34 */
typedef enum TileXRMoonEpStatus {
    TILEXR_MOONEP_SUCCESS = 0,
    TILEXR_MOONEP_ERROR_INVALID_ARGUMENT = -3,
    TILEXR_MOONEP_ERROR_INTERNAL = -4,
    TILEXR_MOONEP_ERROR_NOT_SUPPORTED = -6
} TileXRMoonEpStatus;

/* reference: src/include/tilexr_moonep.h:36-41 (values of TileXR::TileXRDataType) */
typedef enum TileXRMoonEpDType {
    TILEXR_MOONEP_DTYPE_INT32 = 2,
    TILEXR_MOONEP_DTYPE_FLOAT16 = 3,
    TILEXR_MOONEP_DTYPE_FLOAT32 = 4,
    TILEXR_MOONEP_DTYPE_BFLOAT16 = 11
} TileXRMoonEpDType;

/* reference: src/include/tilexr_moonep.h:43-49 */
typedef enum TileXRMoonEpStage {
    TILEXR_MOONEP_STAGE_PLANNING = 1u << 0,
    TILEXR_MOONEP_STAGE_DISPATCH = 1u << 1,
    TILEXR_MOONEP_STAGE_PREFETCH_WEIGHT = 1u << 2,
    TILEXR_MOONEP_STAGE_COMBINE = 1u << 3,
    TILEXR_MOONEP_STAGE_REDUCE_GRAD = 1u << 4
} TileXRMoonEpStage;

/* Values the stages leave in plan->status[0] (device memory) once the stream has run.
 * reference: src/moonep/common/moonep_peer_window.h:36-43; the combine kernel stores its first failure, which is 0
 * on success (src/moonep/combine/kernels/tilexr_moonep_combine_kernel.cpp:727-733).
 *
 * Which value a rank gets when plans are invalid is a closed-form function of F, the set of ranks whose OWN plan is
 * invalid in this exchange (R = ranks of the world):
 *   dispatch  rank r in F:      TILEXR_MOONEP_DISPATCH_STATUS_INVALID_ROUTE
 *             rank r not in F:  TILEXR_MOONEP_DISPATCH_STATUS_REMOTE_FAILURE_BASE + p, p the first member of F in the
 *                               order r+1, r+2, ..., R-1, 0, ..., r-1; SUCCESS when F is empty
 *   combine   rank r in F:      TILEXR_MOONEP_COMBINE_STATUS_INVALID_ROUTE
 *             rank r not in F:  TILEXR_MOONEP_COMBINE_STATUS_REMOTE_FAILURE_BASE + min(F); SUCCESS when F is empty
 * What the output tensors of such an exchange hold is unspecified.  The orders are those in which the reference's kernels wait
 * for their peers (dispatch: WaitAllPeers, tilexr_moonep_dispatch_kernel.cpp:506-521, peer = (rank + offset) % R;
 * combine: CrossRankBarrier, tilexr_moonep_combine_kernel.cpp:391-411, rank order).  There a rank that failed because
 * of a peer raises the same failed flag as the peer itself, so a third rank that meets that flag first names the
 * messenger instead of the origin, depending on timing; here only members of F are ever named, which is the outcome
 * of the reference's walk when no messenger's flag is seen before the origin's. */
#define TILEXR_MOONEP_DISPATCH_STATUS_SUCCESS 2000
#define TILEXR_MOONEP_DISPATCH_STATUS_INVALID_ROUTE 2001
#define TILEXR_MOONEP_DISPATCH_STATUS_REMOTE_FAILURE_BASE 2100   /* + rank of the peer whose plan was invalid */
#define TILEXR_MOONEP_COMBINE_STATUS_SUCCESS 0
#define TILEXR_MOONEP_COMBINE_STATUS_INVALID_ROUTE 3001
#define TILEXR_MOONEP_COMBINE_STATUS_REMOTE_FAILURE_BASE 3100

/* Tensor descriptor.  reference: src/include/tilexr_moonep.h:58-66 (64 bytes) */
typedef struct TileXRMoonEpTensorV1 {
    uint32_t structSize;      /* >= sizeof(TileXRMoonEpTensorV1) */
    uint32_t abiVersion;      /* TILEXR_MOONEP_ABI_VERSION_V1 */
    void *data;               /* device memory */
    uint64_t elementCount;    /* product of shape[0 .. rank) */
    uint32_t dtype;           /* TileXRMoonEpDType */
    uint32_t rank;            /* 1 .. 4 */
    int64_t shape[TILEXR_MOONEP_MAX_TENSOR_RANK];   /* entries at and beyond `rank` are 0 */
} TileXRMoonEpTensorV1;

/* Plan descriptor; every pointer is device memory.  reference: src/include/tilexr_moonep.h:68-85 (120 bytes) */
typedef struct TileXRMoonEpPlanV1 {
    uint32_t structSize;
    uint32_t abiVersion;
    int64_t n;                /* routes of this rank = S * K */
    int64_t r;                /* ranks; must equal the communicator's rankSize */
    int64_t e;                /* experts, a multiple of r */
    int64_t b;                /* prefetch slots per rank, 1 .. e / r */
    int64_t nvS;              /* rows of every rank's receive tensor, >= n; r * nvS <= 2^31 */
    int64_t k;                /* routes per token, 1 .. 32 */
    void *dst;                /* int32 [n] signed route words */
    void *expertsToCopy;      /* not read by Dispatch / Combine; must be non-null */
    void *zeroFillRanges;     /* not read by Dispatch / Combine; must be non-null */
    void *remoteStats;        /* not read by Dispatch / Combine; must be non-null */
    void *dupGroups;          /* int32 [nvS, 3] {primary row, first index into dupLoffs, count} */
    void *dupLoffs;           /* int32 [nvS] duplicate rows, one contiguous slice per group */
    void *dupCounts;          /* int32 [2] {groups, duplicates} */
    void *status;             /* int32 [>= 1]; entry 0 receives the stage's device status */
} TileXRMoonEpPlanV1;

/* reference: src/include/tilexr_moonep.h:101-110 (40 bytes).  Tracing is not offered: `trace` must be null. */
typedef struct TileXRMoonEpDispatchTraceV1 {
    uint32_t structSize;
    uint32_t abiVersion;
    void *buffer;
    uint64_t bufferBytes;
    uint32_t iteration;
    uint32_t iterationCount;
    uint32_t eventCapacity;
    uint32_t reserved;
} TileXRMoonEpDispatchTraceV1;

/* reference: src/include/tilexr_moonep.h:112-125 (88 bytes).  A caller compiled against the older, shorter structure
 * passes structSize = offsetof(registeredWorkspace) and is accepted (src/moonep/host/tilexr_moonep.cpp:300-320). */
typedef struct TileXRMoonEpDispatchArgsV1 {
    uint32_t structSize;
    uint32_t abiVersion;
    TileXRCommPtr comm;
    const TileXRMoonEpPlanV1 *plan;
    const TileXRMoonEpTensorV1 *hiddenSh;          /* bf16 [S, H] */
    const TileXRMoonEpTensorV1 *routeWeightsSk;    /* fp32 [S, K], or null together with routeWeightsNvs */
    TileXRMoonEpTensorV1 *hiddenNvsh;              /* bf16 [NvS, H] out */
    TileXRMoonEpTensorV1 *routeWeightsNvs;         /* fp32 [NvS] out */
    uint64_t flags;                                /* BUILD_DEDUP | SKIP_INTER_RANK_SYNC */
    void *registeredWorkspace;                     /* must be null here */
    uint64_t registeredWorkspaceBytes;             /* must be 0 here */
    const TileXRMoonEpDispatchTraceV1 *trace;      /* must be null */
} TileXRMoonEpDispatchArgsV1;

/* reference: src/include/tilexr_moonep.h:145-156 (72 bytes) */
typedef struct TileXRMoonEpCombineArgsV1 {
    uint32_t structSize;
    uint32_t abiVersion;
    TileXRCommPtr comm;
    const TileXRMoonEpPlanV1 *plan;
    const int32_t *dstLocal;                       /* int32 [NvS] origin of every receive row, -1 = none */
    const TileXRMoonEpTensorV1 *hiddenNvsh;        /* bf16 [NvS, H] */
    const TileXRMoonEpTensorV1 *routeWeightsNvs;   /* fp32 [NvS], or null together with routeWeightsSk */
    TileXRMoonEpTensorV1 *hiddenSh;                /* bf16 [S, H] out */
    TileXRMoonEpTensorV1 *routeWeightsSk;          /* fp32 [S, K] out */
    uint64_t flags;                                /* must be TILEXR_MOONEP_FLAG_NONE */
} TileXRMoonEpCombineArgsV1;

/* reference: src/include/tilexr_moonep.h:258, src/moonep/host/tilexr_moonep.cpp:232-235 -- returns 2 */
uint32_t TileXRMoonEpGetAbiVersion(void);

/* reference: src/include/tilexr_moonep.h:260-262, src/moonep/host/tilexr_moonep.cpp:237-257.  Here both calls report
 * nativeStages = DISPATCH | COMBINE and stubStages = 0. */
int TileXRMoonEpGetCapabilitiesV1(uint64_t *nativeStages, uint64_t *stubStages);
int TileXRMoonEpGetCapabilitiesV2(uint64_t *nativeStages, uint64_t *stubStages);

/* reference: src/include/tilexr_moonep.h:273, src/moonep/host/tilexr_moonep.cpp:300-320,
 * src/moonep/dispatch/host/dispatch_host.cpp:9-60 (argument rules), dispatch_layout.cpp:12-76 (tensor rules),
 * src/moonep/dispatch/kernels/tilexr_moonep_dispatch_kernel.cpp:108-147 (what is computed). */
int TileXRMoonEpDispatchV1(const TileXRMoonEpDispatchArgsV1 *args, aclrtStream stream);

/* reference: src/include/tilexr_moonep.h:284, src/moonep/combine/host/combine_host.cpp:7-58 (argument rules),
 * combine_layout.cpp:13-37,101-120 (tensor rules), src/moonep/combine/kernels/tilexr_moonep_combine_kernel.cpp:117-177
 * (what is computed). */
int TileXRMoonEpCombineV1(const TileXRMoonEpCombineArgsV1 *args, aclrtStream stream);

/* No counterpart in the reference: a tuning knob of this library.  Dispatch copies token rows with one of two kernels:
 * the faster one when the rows are still in the device's memory-side cache (256 MiB on MI355X), one that keeps most of
 * its speed when they have to come from HBM.  It picks by the bytes of token rows of the whole world (ranks * S * H * 2)
 * against the value set here (default 256 MiB; 0 = always the HBM-tolerant kernel).  Process-wide, thread-safe;
 * returns the previous value.  Results do not depend on it. */
int64_t TileXRMoonEpSetCachedRowBytes(int64_t bytes);

#ifdef __cplusplus
#pragma GCC visibility pop
}
#endif

#endif /* TILEXR_MOONEP_H */
