// Plain-C view of libtilexr-ep's host-side arithmetic and argument rules (see hooks.cpp).
// Pointers are described by presence bits, so the rules can be exercised without device memory -- the same way
// the reference's own host tests fabricate a CommArgs (tests/ep/unit/test_tilexr_ep_host_validation.cpp:145-177).
#ifndef TILEXR_AMD_HOOKS_H
#define TILEXR_AMD_HOOKS_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#pragma GCC visibility push(default)   // the entry points below are what the shared library exports
#endif

enum {
    TILEXR_HOOK_X = 1 << 0,              /* x / expertOut */
    TILEXR_HOOK_EXPERT_IDS = 1 << 1,
    TILEXR_HOOK_SCALES = 1 << 2,         /* scales / sharedExpertX */
    TILEXR_HOOK_ACTIVE_MASK = 1 << 3,
    TILEXR_HOOK_EXPERT_SCALES = 1 << 4,
    TILEXR_HOOK_COMM = 1 << 5,
    TILEXR_HOOK_EXPAND_X = 1 << 6,       /* expandXOut / yOut */
    TILEXR_HOOK_DYNAMIC_SCALES = 1 << 7,
    TILEXR_HOOK_ASSIST = 1 << 8,
    TILEXR_HOOK_TOKEN_NUMS = 1 << 9,
    TILEXR_HOOK_COUNTS = 1 << 10,
    TILEXR_HOOK_TP_COUNTS = 1 << 11,
    TILEXR_HOOK_EXPAND_SCALES = 1 << 12,
    TILEXR_HOOK_WORKSPACE = 1 << 13,
    TILEXR_HOOK_STREAM = 1 << 14
};

enum {
    TILEXR_HOOK_RULE_BASIC = 0,
    TILEXR_HOOK_RULE_V2 = 1,
    TILEXR_HOOK_RULE_MVP = 2,
    TILEXR_HOOK_RULE_MEMORY = 3,
    TILEXR_HOOK_RULE_MEMORY_UNCAPPED = 4
};

typedef struct {
    int32_t rank;
    int32_t rankSize;
    int32_t localRankSize;
    uint32_t extraFlag;
    int32_t nullPeer;        /* index of a peer whose memory is missing, -1 for none */
    int32_t hasUdma;         /* UDMA info + registry pointers present */
    uint32_t blockDim;
} TileXREpHookComm;

typedef struct {
    uint32_t has;
    int64_t activeMaskType, bs, h, topK, moeExpertNum, epWorldSize, epRankId, tpWorldSize, tpRankId, expertShardType,
        sharedExpertNum, sharedExpertRankNum, quantMode, globalBs, expertTokenNumsType;
    int32_t dtype;
    int32_t expandXOutDtype;
} TileXREpHookDispatch;

typedef struct {
    uint32_t has;
    int64_t activeMaskType, bs, h, topK, moeExpertNum, epWorldSize, epRankId, tpWorldSize, tpRankId, expertShardType,
        sharedExpertNum, sharedExpertRankNum, quantMode, globalBs;
    int32_t dtype;
} TileXREpHookCombine;

int TileXREpHookValidateDispatch(int which, const TileXREpHookDispatch *dispatch, const TileXREpHookComm *comm);
int TileXREpHookValidateCombine(int which, const TileXREpHookCombine *combine, const TileXREpHookComm *comm);
int TileXREpHookWindowConfig(int64_t rankSize, int64_t expertRankSize, int64_t bs, int64_t h, int64_t topK,
    int64_t moeExpertNum, int64_t sharedExpertNum, int64_t sharedExpertRankNum, int dtype, int64_t payloadExtraBytes,
    int64_t *out9);
int TileXREpHookMemoryDispatchConfig(int64_t rankSize, int64_t rank, int64_t bs, int64_t h, int64_t topK,
    int64_t moeExpertNum, int64_t sharedExpertNum, int64_t sharedExpertRankNum, int64_t globalBs, int dtype,
    int expandXOutDtype, int64_t quantMode, uint32_t blockDim, int64_t *out19);
int TileXREpHookMemoryCombineConfig(int64_t rankSize, int64_t rank, int64_t bs, int64_t h, int64_t topK,
    int64_t moeExpertNum, int64_t sharedExpertNum, int64_t sharedExpertRankNum, int64_t globalBs, int dtype,
    int64_t quantMode, uint32_t blockDim, int64_t *out10);
uint32_t TileXREpHookMemoryCountCoreNum(int64_t totalExpertNum, int64_t rscvStatusNum, uint32_t blockDim);
int TileXREpHookDstRank(int32_t expertId, int64_t localExpertNum);
int TileXREpHookLocalExpert(int32_t expertId, int64_t localExpertNum);
int64_t TileXREpHookDataTypeSize(int dtype);
int64_t TileXREpHookAlignUp(int64_t value, int64_t alignment);
int64_t TileXREpHookUdmaOperationBytes(int64_t totalBytes, int64_t rankSize, int64_t slotBytes);
int64_t TileXREpHookUdmaWorkspaceBytes(int64_t totalBytes, int64_t rankSize, int64_t slotBytes);

/* Runs the readiness-tile bookkeeping of the scatter kernels (ep_tile_publish.h) on `threads` CPU threads that land
 * the parts of `totalRows` rows in a seeded random order, `rounds` dispatches in a row on the same counters and
 * flags.  Checks on the way: a readiness word is stored only when every part of every row of its tile has landed,
 * and exactly once per dispatch.  Checks at the end of each dispatch: every word is (epoch << 32) | rows in the
 * tile, every counter is back to zero.  Returns 0, or a negative code naming the first violated check.
 * `fault` plants a caller-side mistake so that a test can see the checks fire: 1 = a part is reported before it has
 * landed, 2 = one part is reported twice. */
int TileXREpHookTilePublishStress(int totalRows, int maxRows, int tileRows, int parts, int threads, int rounds,
    uint32_t seed, int fault);

#ifdef __cplusplus
#pragma GCC visibility pop
}
#endif

#endif /* TILEXR_AMD_HOOKS_H */
