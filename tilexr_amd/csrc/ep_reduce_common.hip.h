// Shared by the translation units of the reduce: launch arguments, the row map, tile readiness flags on the consumer
// side and the loop that hands a workgroup its tokens.  (The kernels are spread over several files so that they compile
// side by side; the code of one kernel is in one place.)
#ifndef TILEXR_AMD_EP_REDUCE_COMMON_HIP_H
#define TILEXR_AMD_EP_REDUCE_COMMON_HIP_H

#include <hip/hip_runtime.h>

#include <type_traits>

#include "ep_kernel_common.hip.h"
#include "ep_launch.h"
#include "ep_numerics.hip.h"
#include "ep_tile_publish.h"
#include "ep_token_claim.h"
#include "tilexr_ep.h"

namespace TileXREp {

struct ReduceArgs {
    const void *expertOut;
    int64_t rowBytes;
    const uint64_t *inverseTagged;
    uint64_t epoch;
    const int32_t *rowIndexMap;
    const uint64_t *orderKeys;
    const float *expertScales;
    const uint8_t *tokenMask;
    const void *sharedExpertX;
    const float *inScales;
    int bs;
    int h;
    int topK;
    int maxRows;                     // rows expertOut holds
    int slots;                       // rows summed per token: topK routed ones, then the shared-expert slots
    void *y;
    int colSlices;                   // slices a row is cut into (vec kernel, wide rows), else 1
    const uint64_t *tileFlags;
    int tileRows;
    int tileShift;                   // log2(tileRows) where that is a whole number, else -1
    uint64_t flagEpoch;
    int64_t waitTimeoutTicks;
    int32_t *deviceStatus;
    int flagsSettled;                // the producer of the flags finished before this launch began (same stream)
    uint32_t *claim;                 // launches that may wait: two words, zero at launch and again when the launch is
                                     // over (the next group nobody has claimed yet; workgroups that have left)
};

// Launchers of the register-resident kernels, one translation unit per (element type, with / without readiness flags).
// g, v: lanes per token (or per slice of a token's row) and 16-byte vectors per lane; a combination that a unit does
// not hold is a programming error and launches nothing.
void LaunchReduceVecBf16(int g, int v, const ReduceLaunch &l, const ReduceArgs &a, int gridLimit);
void LaunchReduceVecBf16Flags(int g, int v, const ReduceLaunch &l, const ReduceArgs &a, int gridLimit);
void LaunchReduceVecFp16(int g, int v, const ReduceLaunch &l, const ReduceArgs &a, int gridLimit);
void LaunchReduceVecFp16Flags(int g, int v, const ReduceLaunch &l, const ReduceArgs &a, int gridLimit);
void LaunchReduceQuantBf16(int g, int v, const ReduceLaunch &l, const ReduceArgs &a, int gridLimit);
void LaunchReduceQuantBf16Flags(int g, int v, const ReduceLaunch &l, const ReduceArgs &a, int gridLimit);
void LaunchReduceQuantFp16(int g, int v, const ReduceLaunch &l, const ReduceArgs &a, int gridLimit);
void LaunchReduceQuantFp16Flags(int g, int v, const ReduceLaunch &l, const ReduceArgs &a, int gridLimit);
void LaunchReduceQuantBf16Settled(int g, int v, const ReduceLaunch &l, const ReduceArgs &a, int gridLimit);
void LaunchReduceQuantFp16Settled(int g, int v, const ReduceLaunch &l, const ReduceArgs &a, int gridLimit);

namespace {

// Row of a (token, slot), -1 for none.  A row at or beyond `maxRows` (only a corrupted map has one) counts as none: the
// kernels never read outside the rows the caller's buffer holds.
__device__ __forceinline__ int LookupRow(const ReduceArgs &a, int64_t slot)
{
    int row;
    if (a.rowIndexMap != nullptr) {
        row = a.rowIndexMap[slot];
    } else {
        const uint64_t e = a.inverseTagged[slot];
        row = (e >> 32) == a.epoch ? static_cast<int>(e & 0xffffffffu) : -1;
    }
    return static_cast<unsigned>(row) < static_cast<unsigned>(a.maxRows) ? row : -1;
}

__device__ __forceinline__ int TileOf(const ReduceArgs &a, int row)
{
    return a.tileShift >= 0 ? (row >> a.tileShift) : (row / a.tileRows);
}

// Bounded wait until the tile holding `row` has been published for this epoch (its word carries the epoch).  The poll itself is a relaxed
// device-scope load (no cache maintenance per iteration -- an acquire in the loop would invalidate this XCD's L2 on
// every spin and starve the producer).  What the caller reads afterwards must not come from a stale L2 line: the
// register-resident kernels read published rows with agent-scope loads, which are served from memory; in the
// element-granular kernel every wave issues an acquire of its own once all the token's waits have succeeded.
__device__ inline bool WaitTile(const ReduceArgs &a, int row)
{
    const int tile = TileOf(a, row);
    const uint64_t start = wall_clock64();
    // every poll is a round trip to memory (agent scope): the gap between polls doubles up to about 3 us
    int backoff = 0;
    while (true) {
        const uint64_t w = __hip_atomic_load(&a.tileFlags[tile], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        if (TileWordReady(w, a.flagEpoch)) {
            return true;
        }
        // a producer that finished before this launch began has nothing more to publish
        if (a.flagsSettled != 0 || static_cast<int64_t>(wall_clock64() - start) > a.waitTimeoutTicks) {
            return false;
        }
        // once one wait of the launch has expired the producer is taken to be gone: later waits give up at once,
        // so a launch whose flags never arrive ends after about one timeout, not one per tile
        if (a.deviceStatus != nullptr &&
            __hip_atomic_load(a.deviceStatus, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) != 0) {
            return false;
        }
        switch (backoff) {                  // s_sleep takes an immediate: 64 clocks per unit
            case 0: __builtin_amdgcn_s_sleep(8); break;
            case 1: __builtin_amdgcn_s_sleep(16); break;
            case 2: __builtin_amdgcn_s_sleep(32); break;
            case 3: __builtin_amdgcn_s_sleep(64); break;
            default: __builtin_amdgcn_s_sleep(127); break;
        }
        backoff += backoff < 4 ? 1 : 0;
    }
}

// Insertion sort of row indices, absent rows (-1) last.  The order is the row index itself, or -- when rows come
// from several expert ranks -- the (expert rank, row) key recorded for each slot.  K is small.
__device__ inline void SortRows(int *rows, int k, const uint64_t *orderKeys)
{
    if (orderKeys != nullptr) {
        for (int i = 1; i < k; ++i) {
            const int v = rows[i];
            const uint64_t kv = v < 0 ? ~0ull : orderKeys[v];
            int j = i - 1;
            while (j >= 0 && (rows[j] < 0 ? ~0ull : orderKeys[rows[j]]) > kv) {
                rows[j + 1] = rows[j];
                --j;
            }
            rows[j + 1] = v;
        }
        return;
    }
    for (int i = 1; i < k; ++i) {
        const int v = rows[i];
        const unsigned kv = static_cast<unsigned>(v);      // -1 becomes the largest key
        int j = i - 1;
        while (j >= 0 && static_cast<unsigned>(rows[j]) > kv) {
            rows[j + 1] = rows[j];
            --j;
        }
        rows[j + 1] = v;
    }
}

// Row loads of the register-resident kernels.  FL = false: non-temporal loads.  FL = true (rows published through
// readiness flags, possibly a moment ago by a workgroup on another XCD): agent-scope loads, served from memory, so
// that no acquire fence (an invalidate of this XCD's whole L2) is needed per token.
template <bool FL>
__device__ __forceinline__ u32x4 RowLoad(const char *rowBase, __amdgpu_buffer_rsrc_t rsrc, int byteOffset)
{
    if (FL) {
        return __builtin_amdgcn_raw_buffer_load_b128(rsrc, byteOffset, 0, kAuxAgentScope);
    }
    return __builtin_nontemporal_load(reinterpret_cast<const u32x4 *>(rowBase + byteOffset));
}

template <bool FL>
__device__ __forceinline__ float ScaleLoad(const float *p)
{
    if (FL) {
        return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
    return *p;
}

// One look at the tile holding `row`: published for this epoch or not.
__device__ __forceinline__ bool TilePublished(const ReduceArgs &a, int row)
{
    const uint64_t w = __hip_atomic_load(&a.tileFlags[TileOf(a, row)], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    return TileWordReady(w, a.flagEpoch);
}

// Fills s_row / s_w for one token and deals with tile flags.  BLOCK: every slot waits (bounded) for its tile.  Otherwise
// `mode` says what a slot does about its tile (ep_token_claim.h: SlotLooksAtTile, JudgeSlot):
//   kRouteCheck    look once; a tile that is not there yet leaves kRowPending in the slot and the call returns true
//                  ("come back later")
//   kRouteTrusted  nothing: the caller has just seen every tile of this token published
//   kRouteGiveUp   look once; a tile that is not there turns the slot into an expired one
// An expired wait sets the launch's status word and leaves kRowExpired in the slot: the token then gets a row of zeros
// (AnyExpired), never the sum of the rows that happened to be ready.
__device__ __forceinline__ bool AnyExpired(const int *rows, int slots)
{
    bool expired = false;
    for (int k = 0; k < slots; ++k) {
        expired |= rows[k] == kRowExpired;
    }
    return expired;
}

// A launch whose producer finished before it began (flagsSettled) waits for nothing, but a tile word that does not
// carry the launch's epoch still means that the rows of that tile were never written: the token gets a row of zeros and
// the launch's status word is set, at once.  Lane k of a wave holds the row of slot k (-1: none).  The word is asked for
// before the rows and looked at after the last of them has been used: the memory counter runs in order, so by then it
// has long arrived, and nothing waits for it on the way (an ordinary load: the words are final, this XCD's L2 may keep
// them).
// (Only the half of the word that holds the epoch is loaded: one register less for the whole K loop, and the kernels
// that use this are tuned to the register.)
__device__ __forceinline__ uint32_t SettledWordLoad(const ReduceArgs &a, int slotRow)
{
    static_assert(__BYTE_ORDER__ == __ORDER_LITTLE_ENDIAN__, "the epoch is the word's upper half");
    return slotRow >= 0 ? reinterpret_cast<const uint32_t *>(a.tileFlags + TileOf(a, slotRow))[1] : 0u;
}

__device__ __forceinline__ bool SettledWordMissing(const ReduceArgs &a, int slotRow, uint32_t epochOfWord, int waveLane)
{
    const bool missing = __ballot(slotRow >= 0 && epochOfWord != static_cast<uint32_t>(a.flagEpoch)) != 0;
    if (missing && waveLane == 0 && a.deviceStatus != nullptr) {
        atomicExch(a.deviceStatus, 1);
    }
    return missing;
}

template <bool BLOCK>
__device__ __forceinline__ bool LoadRoutes(const ReduceArgs &a, int token, bool tokOk, int lane, int lanes, int *rows,
    float *weights, int mode)
{
    bool pending = false;
    for (int k = lane; k < a.slots; k += lanes) {
        const int64_t slot = static_cast<int64_t>(tokOk ? token : 0) * a.slots + k;
        // shared-expert slots follow the routed ones and carry no gate weight
        // (reference: src/ep/kernels/tilexr_ep_combine_memory_kernel.h:650-657)
        // The weight is asked for before the row is looked at: one trip to memory for both, not one after the other.
        const float weight = (tokOk && a.expertScales != nullptr && k < a.topK) ?
            a.expertScales[static_cast<int64_t>(token) * a.topK + k] : 1.0f;
        int row = tokOk ? LookupRow(a, slot) : -1;
        if (row >= 0 && a.tileFlags != nullptr && SlotLooksAtTile(BLOCK, mode)) {
            const bool there = BLOCK ? WaitTile(a, row) : TilePublished(a, row);
            const int verdict = JudgeSlot(BLOCK, mode, there);
            if (verdict == kSlotComeBack) {
                row = kRowPending;
                pending = true;
            } else if (verdict == kSlotExpire) {
                if (a.deviceStatus != nullptr) {
                    atomicExch(a.deviceStatus, 1);
                }
                row = kRowExpired;
            }
        }
        rows[k] = row;
        weights[k] = weight;
    }
    return pending;
}

// Runs unit(group) for this workgroup's groups: blockIdx.x, blockIdx.x + gridDim.x, ...  `load(group, mode)`
// fills the workgroup's route tables for a group and returns (per lane) whether a tile it needs is not published yet;
// `tokenAt(group, t)` names the t-th of a group's `tokensPerGroup` tokens (-1 = none).
//
// Without readiness flags, or with flags that were all published before the launch began, that is a plain loop.  A
// launch that may have to wait (WAITS, flags not settled) never sits on one group while others are ready: a token needs
// the tiles of all its rows, which a producer that works tile by tile finishes at unrelated times, so tokens become
// ready in no particular order.  A workgroup holds a few groups at a time.  Fresh ones are looked at once and reduced
// if their tiles are there.  For what is left it goes in rounds: all lanes together look once at every tile the held
// groups need (one round trip for the lot), the groups that have become complete are reduced, and a round without any
// is followed by a sleep that grows to about 14 us.  When nothing it holds has become ready for the wait bound, or
// another workgroup has reported an expired wait, the rest is given up: those tokens get rows of zeros and the launch's
// status word is set.
template <bool WAITS, typename TokenAt, typename Load, typename Unit>
__device__ __forceinline__ void ForEachGroup(const ReduceArgs &a, int groups, int tokensPerGroup, TokenAt tokenAt,
    Load load, Unit unit)
{
    const bool plainLoop = !WAITS || a.flagsSettled != 0;
    if (plainLoop) {
        // no flags, or flags that were all published before this launch began: the route tables trust every tile, and
        // the kernel looks at the words itself, beside the rows (SettledWordLoad)
        for (int group = blockIdx.x; group < groups; group += gridDim.x) {
            __syncthreads();        // the previous iteration's readers are done with the route tables
            load(group, kRouteTrusted);
            __syncthreads();
            unit(group);
        }
        return;
    }
    if constexpr (WAITS) {
        // the control flow is ClaimAndReduce of ep_token_claim.h (the host-side model of the protocol runs the same
        // code); what follows are its operations for a workgroup: atomics, barriers, LDS
        __shared__ uint32_t s_notReady;
        __shared__ int s_group[kClaimHeld];
        __shared__ int s_base;
        struct WorkgroupEnv {
            const ReduceArgs &a;
            TokenAt &tokenAt;
            Load &load;
            Unit &unit;
            uint32_t *notReady;
            int *group;
            int *base;
            int perGroup;                   // (token, slot) pairs of a group
            int tokensPerGroup;
            int dealt;                      // next group by block index (launches without a claim counter)
            uint64_t idleSince;

            __device__ __forceinline__ int Claim(int want)
            {
                if (a.claim == nullptr) {
                    return 0;
                }
                __syncthreads();            // readers of *base from the previous refill are done
                if (threadIdx.x == 0) {
                    *base = static_cast<int>(__hip_atomic_fetch_add(a.claim, static_cast<uint32_t>(want), __ATOMIC_RELAXED,
                        __HIP_MEMORY_SCOPE_AGENT));
                }
                __syncthreads();
                return *base;
            }
            __device__ __forceinline__ int NextGroup(int *next)
            {
                if (a.claim != nullptr) {
                    return (*next)++;
                }
                const int mine = dealt;
                dealt += static_cast<int>(gridDim.x);
                return mine;
            }
            __device__ __forceinline__ void Hold(int slot, int g)
            {
                if (threadIdx.x == 0) {
                    group[slot] = g;
                }
            }
            __device__ __forceinline__ void HoldDone()
            {
                __syncthreads();
            }
            __device__ __forceinline__ bool Try(int slot, int mode)
            {
                const int g = group[slot];
                __syncthreads();
                const bool waiting = load(g, mode);
                if (__syncthreads_or((mode == kRouteCheck && waiting) ? 1 : 0) != 0) {
                    return false;           // uniform: every lane gets the same answer
                }
                unit(g);
                return true;
            }
            __device__ __forceinline__ uint32_t Scan(uint32_t pending)
            {
                // all lanes together look once at every tile the held groups need: one round trip for the lot
                if (threadIdx.x == 0) {
                    *notReady = 0u;
                }
                __syncthreads();
                for (int idx = threadIdx.x; idx < kClaimHeld * perGroup; idx += blockDim.x) {
                    const int i = idx / perGroup;
                    if (((pending >> i) & 1u) == 0u) {
                        continue;
                    }
                    const int token = tokenAt(group[i], (idx % perGroup) / a.slots);
                    if (token < 0) {
                        continue;
                    }
                    const int row = LookupRow(a, static_cast<int64_t>(token) * a.slots + idx % a.slots);
                    if (row >= 0 && !TilePublished(a, row)) {
                        atomicOr(notReady, 1u << i);
                    }
                }
                __syncthreads();
                return *notReady;
            }
            __device__ __forceinline__ bool GiveUpNow()
            {
                bool stop = false;
                if (threadIdx.x == 0) {
                    stop = static_cast<int64_t>(wall_clock64() - idleSince) > a.waitTimeoutTicks ||
                        (a.deviceStatus != nullptr &&
                         __hip_atomic_load(a.deviceStatus, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) != 0);
                }
                return __syncthreads_or(stop ? 1 : 0) != 0;
            }
            __device__ __forceinline__ void Touch()
            {
                idleSince = wall_clock64();
            }
            __device__ __forceinline__ void Sleep(int level)
            {
                for (int r = 0; r < (1 << level); ++r) {
                    __builtin_amdgcn_s_sleep(127);      // 127 x 64 clocks, about 3.5 us
                }
            }
            __device__ __forceinline__ void Leave()
            {
                if (a.claim != nullptr && threadIdx.x == 0) {
                    DeviceTileOps ops;
                    LeaveClaimWords(ops, a.claim, gridDim.x);
                }
            }
        };
        WorkgroupEnv env {a, tokenAt, load, unit, &s_notReady, s_group, &s_base, tokensPerGroup * a.slots, tokensPerGroup,
            static_cast<int>(blockIdx.x), 0};
        ClaimAndReduce(env, groups);
    }
}

} // namespace
} // namespace TileXREp

#endif // TILEXR_AMD_EP_REDUCE_COMMON_HIP_H
