// reduce: y[token] = sum over the token's rows, gathered through the inverse map (gfx950, wave64).
//
// HBM-bound: topK row reads per output row, < 0.5 FLOP per byte, no MFMA.  G lanes cooperate on one token and keep
// V x 8 fp32 accumulators in registers; for each route in k order a lane issues all V of its 128-bit non-temporal
// loads of that row before touching the accumulators, so 64-128 bytes per lane are in flight while the previous
// row is being summed.  Measured on MI355X this moves 4096 x 7168 bf16 x top-8 (529 MB) at about 6 TB/s.
//
//   KIND fp32     sum = 0; for k = 0..K-1: sum = sum + (w_k * row_k) in fp32 (separate multiply and add), then the
//                 shared-expert row, then one round-to-nearest-even (saturating for fp16) to the output type;
//                 an inactive token (mask) gives zeros
//                 (reference: src/ep/kernels/tilexr_ep_combine_memory_kernel.h:505-553, 555-571, 573-601, 632-662)
//   KIND per-add  rows in ascending row index; y = T(float(y) + float(row)) after every add
//                 (reference: src/ep/kernels/tilexr_ep_combine_kernel.cpp:15-26, 54-101)
//   COMMQ 3/4     every row first takes the MXFP8 e5m2 / e4m3 round trip and is accumulated as
//                 ((fp8 * 2^(s-127)) * w) (reference: src/ep/kernels/tilexr_ep_mxfp8_quant.h:286-352)
//   INQ 2/5       rows hold int8 / fp8 payloads that are dequantised with their scales and rounded to the element
//                 type first (no reference counterpart)
#include <hip/hip_runtime.h>

#include <type_traits>

#include "ep_kernel_common.hip.h"
#include "ep_launch.h"
#include "ep_numerics.hip.h"
#include "ep_tile_publish.h"
#include "tilexr_ep.h"

namespace TileXREp {
namespace {

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
    uint64_t flagEpoch;
    int64_t waitTimeoutTicks;
    int32_t *deviceStatus;
    int flagsSettled;                // the producer of the flags finished before this launch began (same stream)
};

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

// Bounded wait until the tile holding `row` has been published for this epoch (its word carries the epoch).  The poll itself is a relaxed
// device-scope load (no cache maintenance per iteration -- an acquire in the loop would invalidate this XCD's L2 on
// every spin and starve the producer).  What the caller reads afterwards must not come from a stale L2 line: the
// register-resident kernels read published rows with agent-scope loads, which are served from memory; the
// element-granular kernel issues one acquire fence after all its waits have succeeded.
__device__ bool WaitTile(const ReduceArgs &a, int row)
{
    const int tile = row / a.tileRows;
    const uint64_t start = wall_clock64();
    // every poll is a round trip to memory (agent scope): the gap between polls doubles up to about 3 us
    int backoff = 0;
    while (true) {
        const uint64_t w = __hip_atomic_load(&a.tileFlags[tile], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        if (TileWordReady(w, a.flagEpoch)) {
            return true;
        }
        if (static_cast<int64_t>(wall_clock64() - start) > a.waitTimeoutTicks) {
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
__device__ void SortRows(int *rows, int k, const uint64_t *orderKeys)
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
    const uint64_t w = __hip_atomic_load(&a.tileFlags[row / a.tileRows], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    return TileWordReady(w, a.flagEpoch);
}

// Fills s_row / s_w for one token and deals with tile flags.  BLOCK: every slot waits (bounded) for its tile.  Otherwise
// `mode` says what a slot does about its tile:
//   kRouteCheck    look once; a tile that is not there yet leaves kRowPending in the slot and the call returns true
//                  ("come back later")
//   kRouteTrusted  nothing: the caller has just seen every tile of this token published
//   kRouteGiveUp   look once; a tile that is not there turns the slot into an expired one
//   kRouteSettled  the producer finished before this launch began, so nothing is waited for and no read can come too
//                  early: the slot gets its row at once and the call returns whether the tile's word says otherwise,
//                  a value the caller needs only after the rows have been read (the word travels beside the rows
//                  instead of ahead of them: one dependent round trip less)
// An expired wait sets the launch's status word and leaves kRowExpired in the slot: the token then gets a row of zeros
// (AnyExpired), never the sum of the rows that happened to be ready.
constexpr int kRowExpired = -2;
constexpr int kRowPending = -3;
enum RouteMode : int { kRouteCheck = 0, kRouteTrusted = 1, kRouteGiveUp = 2, kRouteSettled = 3 };

__device__ __forceinline__ bool AnyExpired(const int *rows, int slots)
{
    bool expired = false;
    for (int k = 0; k < slots; ++k) {
        expired |= rows[k] == kRowExpired;
    }
    return expired;
}

template <bool FENCE, bool BLOCK>
__device__ __forceinline__ bool LoadRoutes(const ReduceArgs &a, int token, bool tokOk, int lane, int lanes, int *rows,
    float *weights, int mode)
{
    bool pending = false;
    for (int k = lane; k < a.slots; k += lanes) {
        const int64_t slot = static_cast<int64_t>(tokOk ? token : 0) * a.slots + k;
        int row = tokOk ? LookupRow(a, slot) : -1;
        const bool settled = !BLOCK && mode == kRouteSettled;
        if (!settled && row >= 0 && a.tileFlags != nullptr && (BLOCK || mode != kRouteTrusted)) {
            const bool there = BLOCK ? WaitTile(a, row) : TilePublished(a, row);
            if (!there && !BLOCK && mode == kRouteCheck) {
                row = kRowPending;
                pending = true;
            } else if (!there) {
                if (a.deviceStatus != nullptr) {
                    atomicExch(a.deviceStatus, 1);
                }
                row = kRowExpired;
            }
        }
        rows[k] = row;
        // shared-expert slots follow the routed ones and carry no gate weight
        // (reference: src/ep/kernels/tilexr_ep_combine_memory_kernel.h:650-657)
        weights[k] = (tokOk && a.expertScales != nullptr && k < a.topK) ?
            a.expertScales[static_cast<int64_t>(token) * a.topK + k] : 1.0f;
        if (settled && row >= 0 && a.tileFlags != nullptr) {
            // the last load of all: the memory counter runs in order, so nothing that is needed before the rows may
            // come after it
            // (an ordinary load: the words are final, this XCD's L2 may keep them)
            pending |= !TileWordReady(a.tileFlags[row / a.tileRows], a.flagEpoch);
        }
    }
    if (FENCE && a.tileFlags != nullptr && lane < a.slots) {
        // pairs with the producer's release: rows read after this fence (by this wave, or by the other waves of the
        // workgroup after the barrier that follows) are at least as new as the flag values seen above
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "agent");
    }
    return pending;
}

// Runs unit(group, beforeStores) for this workgroup's groups: blockIdx.x, blockIdx.x + gridDim.x, ...  beforeStores is
// a callable the unit invokes once, after its last load has been used and before its first store.  `load(group, mode)`
// fills the workgroup's route tables for a group and returns (per lane) whether a tile it needs is not published yet;
// `tokenAt(group, t)` names the t-th of a group's `tokensPerGroup` tokens (-1 = none).
//
// Without readiness flags that is a plain loop.  With them (WAITS) a workgroup never sits on one group while others it
// owes are ready: a token needs the tiles of all its rows, which a producer that works tile by tile finishes at
// unrelated times, so tokens become ready in no particular order.  The workgroup takes its groups 32 at a time.  A
// first pass reduces every group whose tiles are there already (all of them when the producer ran earlier on the same
// stream).  For what is left it then goes in rounds: all lanes together look once at every tile the pending groups need
// (one round trip for the lot), the groups that have become complete are reduced, and a round without any is followed
// by a sleep that grows to about 14 us.  When nothing it owes has become ready for the wait bound, or another workgroup
// has reported an expired wait, the rest is given up: those tokens get rows of zeros and the launch's status word is set.
template <bool WAITS, typename TokenAt, typename Load, typename Unit>
__device__ __forceinline__ void ForEachGroup(const ReduceArgs &a, int groups, int tokensPerGroup, TokenAt tokenAt,
    Load load, Unit unit)
{
    if constexpr (!WAITS) {
        for (int group = blockIdx.x; group < groups; group += gridDim.x) {
            __syncthreads();        // the previous iteration's readers are done with the route tables
            load(group, kRouteTrusted);
            __syncthreads();
            unit(group, [] {});
        }
    } else {
        if (a.flagsSettled != 0) {
            // No barrier of the kind that waits for memory after the rows have been stored: a workgroup that has to see
            // its stores complete before it may leave stays a store round trip longer (2048-byte fp8 rows: 53 instead of
            // 43 us).  The verdict on the tile words goes through LDS, two slots taken in turn so that the reset of one
            // is a whole iteration away from its last readers.
            __shared__ int s_missing[2];
            int turn = 0;
            for (int group = blockIdx.x; group < groups; group += gridDim.x, turn ^= 1) {
                if (threadIdx.x == 0) {
                    s_missing[turn] = 0;
                }
                __syncthreads();
                const bool missing = load(group, kRouteSettled);
                LdsBarrier();                       // the tile words are still on their way: nothing waits for them here
                // the verdict is handed over between the last use of the rows and the first store: whoever asks for the
                // tile word there finds it long since arrived (it was requested ahead of the rows), and the barrier
                // below does not wait for the stores
                unit(group, [&] {
                    if (missing) {
                        s_missing[turn] = 1;
                    }
                });
                LdsBarrier();
                if (s_missing[turn] != 0) {
                    // a word that is not there now never will be: the token gets a row of zeros and the status is set
                    __syncthreads();
                    load(group, kRouteGiveUp);
                    __syncthreads();
                    unit(group, [] {});
                }
            }
            return;
        }
        __shared__ uint32_t s_notReady;
        const int first = static_cast<int>(blockIdx.x);
        const int stride = static_cast<int>(gridDim.x);
        const int mine = groups > first ? (groups - 1 - first) / stride + 1 : 0;
        const int perGroup = tokensPerGroup * a.slots;
        for (int base = 0; base < mine; base += 32) {
            const int inWindow = mine - base < 32 ? mine - base : 32;
            uint32_t pending = inWindow == 32 ? 0xffffffffu : ((1u << inWindow) - 1u);
            for (uint32_t m = pending; m != 0u; m &= m - 1u) {
                const int i = __builtin_ctz(m);
                const int group = first + (base + i) * stride;
                __syncthreads();
                const bool waiting = load(group, kRouteCheck);
                if (__syncthreads_or(waiting ? 1 : 0) != 0) {
                    continue;                       // uniform: every lane gets the same answer
                }
                unit(group, [] {});
                pending &= ~(1u << i);
            }
            uint64_t idleSince = wall_clock64();
            int backoff = 0;
            while (pending != 0u) {
                if (threadIdx.x == 0) {
                    s_notReady = 0u;
                }
                __syncthreads();
                for (int idx = threadIdx.x; idx < inWindow * perGroup; idx += blockDim.x) {
                    const int i = idx / perGroup;
                    if (((pending >> i) & 1u) == 0u) {
                        continue;
                    }
                    const int token = tokenAt(first + (base + i) * stride, (idx % perGroup) / a.slots);
                    if (token < 0) {
                        continue;
                    }
                    const int row = LookupRow(a, static_cast<int64_t>(token) * a.slots + idx % a.slots);
                    if (row >= 0 && !TilePublished(a, row)) {
                        atomicOr(&s_notReady, 1u << i);
                    }
                }
                __syncthreads();
                const uint32_t ready = pending & ~s_notReady;
                if (ready == 0u) {
                    bool stop = false;
                    if (threadIdx.x == 0) {
                        stop = static_cast<int64_t>(wall_clock64() - idleSince) > a.waitTimeoutTicks ||
                            (a.deviceStatus != nullptr &&
                             __hip_atomic_load(a.deviceStatus, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) != 0);
                    }
                    if (__syncthreads_or(stop ? 1 : 0) != 0) {
                        for (uint32_t m = pending; m != 0u; m &= m - 1u) {
                            const int group = first + (base + __builtin_ctz(m)) * stride;
                            __syncthreads();
                            load(group, kRouteGiveUp);
                            __syncthreads();
                            unit(group, [] {});
                        }
                        pending = 0u;
                        break;
                    }
                    for (int r = 0; r < (1 << backoff); ++r) {
                        __builtin_amdgcn_s_sleep(127);      // 127 x 64 clocks, about 3.5 us
                    }
                    backoff += backoff < 2 ? 1 : 0;
                    continue;
                }
                for (uint32_t m = ready; m != 0u; m &= m - 1u) {
                    const int i = __builtin_ctz(m);
                    const int group = first + (base + i) * stride;
                    __syncthreads();
                    load(group, kRouteTrusted);
                    __syncthreads();
                    unit(group, [] {});
                    pending &= ~(1u << i);
                }
                idleSince = wall_clock64();
                backoff = 0;
            }
        }
    }
}

template <int G, int V, int KIND, bool BF16, int COMMQ, bool FL>
__global__ __launch_bounds__(kThreads) void ep_reduce_vec_kernel(ReduceArgs a)
{
    constexpr int kTokens = kThreads / G;
    constexpr bool kMx = COMMQ != 0;
    constexpr bool kCommE5m2 = COMMQ == TILEXR_EP_QUANT_COMM_MXFP8_E5M2;
    __shared__ int s_row[kTokens][kMaxTopK];
    __shared__ float s_w[kTokens][kMaxTopK];

    const int tg = threadIdx.x / G;
    const int lane = threadIdx.x % G;
    // Rows in flight per lane.  A whole workgroup per token is the geometry of launches that may wait on flags: at most two
    // such workgroups run per compute unit, so a wave may use half a SIMD's registers and keeps four rows in flight
    // whatever the row width; the other geometries run many more waves and trade rows in flight for occupancy.
    constexpr int KB = G == kThreads ? 4 : (V <= 2 ? 4 : (V <= 4 ? 2 : 1));
    const int vecs = a.h / 8;
    // a unit is one token, or -- for wide rows -- one slice of G * V vectors of a token
    const int units = a.bs * a.colSlices;
    // the launch may use fewer waves per workgroup than kThreads / kWave (single-wave workgroups for sliced rows)
    const int unitsPerGroup = static_cast<int>(blockDim.x) / G;
    const int groups = (units + unitsPerGroup - 1) / unitsPerGroup;

    auto tokenAt = [&](int group, int t) {
        const int unit = group * unitsPerGroup + t;
        return unit < units ? unit / a.colSlices : -1;
    };
    auto load = [&](int group, int mode) {
        const int unit = group * unitsPerGroup + tg;
        return LoadRoutes<false, false>(a, unit / a.colSlices, unit < units, lane, G, s_row[tg], s_w[tg], mode);
    };
    auto reduceUnit = [&](int group, auto beforeStores) {
        const int unit = group * unitsPerGroup + tg;
        const bool tokOk = unit < units;
        const int token = unit / a.colSlices;
        const int colBase = (unit % a.colSlices) * (G * V);
        if (KIND == kReducePerAdd) {
            if (lane == 0) {
                SortRows(s_row[tg], a.slots, a.orderKeys);
            }
            __syncthreads();
        }
        const bool active = tokOk && (a.tokenMask == nullptr || a.tokenMask[token] != 0) && !(FL && AnyExpired(s_row[tg], a.slots));

        float acc[V][8];
#pragma unroll
        for (int j = 0; j < V; ++j) {
#pragma unroll
            for (int e = 0; e < 8; ++e) {
                acc[j][e] = 0.0f;
            }
        }
        // control flow below is uniform across the lanes that share a token (the MXFP8 round trip shuffles)
        for (int k0 = 0; k0 < a.slots; k0 += KB) {
            u32x4 v16[KB][V];
            int rowOfK[KB];
#pragma unroll
            for (int u = 0; u < KB; ++u) {
                const int k = k0 + u;
                // the lanes of a wave share one token, so the row is wave-uniform
                const int row = __builtin_amdgcn_readfirstlane((k < a.slots && active) ? s_row[tg][k] : -1);
                rowOfK[u] = row;
                const char *base = static_cast<const char *>(a.expertOut) + static_cast<int64_t>(row < 0 ? 0 : row) * a.rowBytes;
                const __amdgpu_buffer_rsrc_t rsrc = RowResource(base, vecs * 16);
#pragma unroll
                for (int j = 0; j < V; ++j) {
                    const int idx = colBase + j * G + lane;
                    v16[u][j] = (row >= 0 && idx < vecs) ? RowLoad<FL>(base, rsrc, idx * 16) : u32x4{0u, 0u, 0u, 0u};
                }
            }
#pragma unroll
            for (int u = 0; u < KB; ++u) {
                if (rowOfK[u] < 0) {
                    continue;
                }
                const float w = s_w[tg][k0 + u];
#pragma unroll
                for (int j = 0; j < V; ++j) {
                    float f[8];
#pragma unroll
                    for (int q = 0; q < 4; ++q) {
                        f[2 * q] = Decode16<BF16>(v16[u][j][q] & 0xffffu);
                        f[2 * q + 1] = Decode16<BF16>(v16[u][j][q] >> 16);
                    }
                    if (kMx) {
                        float amax = 0.0f;
#pragma unroll
                        for (int e = 0; e < 8; ++e) {
                            amax = fmaxf(amax, fabsf(f[e]));
                        }
                        amax = fmaxf(amax, __shfl_xor(amax, 1));
                        amax = fmaxf(amax, __shfl_xor(amax, 2));
                        const int se = MxSharedExponent<kCommE5m2>(amax);
                        const float up = Exp2Int(se);
#pragma unroll
                        for (int e = 0; e < 8; ++e) {
                            const float back = Fp8Decode<kCommE5m2>(Fp8Encode<kCommE5m2>(ldexpf(f[e], -se)));
                            f[e] = __fmul_rn(back, up);
                        }
                    }
                    if (KIND == kReducePerAdd) {
#pragma unroll
                        for (int e = 0; e < 8; ++e) {
                            acc[j][e] = RoundTo16<BF16>(__fadd_rn(acc[j][e], f[e]));
                        }
                    } else {
#pragma unroll
                        for (int e = 0; e < 8; ++e) {
                            acc[j][e] = __fadd_rn(acc[j][e], __fmul_rn(f[e], w));
                        }
                    }
                }
            }
        }
        if (a.sharedExpertX != nullptr && active) {
            const u32x4 *sx = reinterpret_cast<const u32x4 *>(static_cast<const char *>(a.sharedExpertX) +
                static_cast<int64_t>(token) * a.h * 2);
#pragma unroll
            for (int j = 0; j < V; ++j) {
                const int idx = colBase + j * G + lane;
                if (idx < vecs) {
                    const u32x4 v = sx[idx];
#pragma unroll
                    for (int q = 0; q < 4; ++q) {
                        acc[j][2 * q] = __fadd_rn(acc[j][2 * q], Decode16<BF16>(v[q] & 0xffffu));
                        acc[j][2 * q + 1] = __fadd_rn(acc[j][2 * q + 1], Decode16<BF16>(v[q] >> 16));
                    }
                }
            }
        }
        beforeStores();
        if (tokOk) {
            u32x4 *dst = reinterpret_cast<u32x4 *>(static_cast<char *>(a.y) + static_cast<int64_t>(token) * a.h * 2);
#pragma unroll
            for (int j = 0; j < V; ++j) {
                const int idx = colBase + j * G + lane;
                if (idx < vecs) {
                    u32x4 o;
#pragma unroll
                    for (int q = 0; q < 4; ++q) {
                        o[q] = active ? EncodePair16Sat<BF16>(acc[j][2 * q], acc[j][2 * q + 1]) : 0u;
                    }
                    __builtin_nontemporal_store(o, dst + idx);
                }
            }
        }
    };
    ForEachGroup<FL>(a, groups, unitsPerGroup, tokenAt, load, reduceUnit);
}

// Quantised expert output: int8 rows with one fp32 scale per row, or fp8 e4m3 rows with one fp32 scale per 128
// columns.  Each value is dequantised, rounded to the output element type, then accumulated exactly like an ordinary
// row (fp32, k order, separate multiply and add).  Rows are a quarter the bytes of bf16 rows, so a lane owns 16
// consecutive columns per vector (one 16-byte load) and KB rows are kept in flight at once.
template <int G, int V, int INQ, bool BF16, bool FL>
__global__ __launch_bounds__(kThreads, (V == 1 && !FL && BF16) ? 7 : 1) void ep_reduce_quant_kernel(ReduceArgs a)
{
    constexpr int kTokens = kThreads / G;
    constexpr int KB = V >= 4 ? 2 : 4;
    __shared__ int s_row[kTokens][kMaxTopK];
    __shared__ float s_w[kTokens][kMaxTopK];

    const int tg = threadIdx.x / G;
    const int lane = threadIdx.x % G;
    const int vecs = a.h / 16;
    const int groups = (a.bs + kTokens - 1) / kTokens;
    const int b128 = (a.h + 127) / 128;

    auto tokenAt = [&](int group, int t) {
        const int token = group * kTokens + t;
        return token < a.bs ? token : -1;
    };
    auto load = [&](int group, int mode) {
        const int token = group * kTokens + tg;
        return LoadRoutes<false, false>(a, token, token < a.bs, lane, G, s_row[tg], s_w[tg], mode);
    };
    auto reduceUnit = [&](int group, auto beforeStores) {
        const int token = group * kTokens + tg;
        const bool tokOk = token < a.bs;
        const bool active = tokOk && (a.tokenMask == nullptr || a.tokenMask[token] != 0) && !(FL && AnyExpired(s_row[tg], a.slots));

        float acc[V][16];
        // The K loop.  fp8 rows are decoded by the hardware convert alone, which differs from the reference decode in
        // one respect only (the sign of the NaN it returns for code 0x7f); a NaN code always surfaces as a NaN in the
        // sum, so a wave that finds a NaN among its sums runs the loop once more with the exact decode.  That keeps a
        // test of every word (four instructions and a branch per four values) out of the loop that everything else
        // shares.
        // throughMemory: rows and scales are read past this XCD's L2, as they must be while their producer may still
        // be writing neighbours of theirs.  Once the producer has finished (flagsSettled) the L2 is as good as memory,
        // and the scales, which the lanes of a token share, are worth keeping there (4096 x int8 rows: 58 -> 49 us).
        auto accumulate = [&](auto exactDecode, auto throughMemory) {
            constexpr bool kExactDecode = decltype(exactDecode)::value;
            constexpr bool kThroughMemory = decltype(throughMemory)::value;
#pragma unroll
            for (int j = 0; j < V; ++j) {
#pragma unroll
                for (int e = 0; e < 16; ++e) {
                    acc[j][e] = 0.0f;
                }
            }
            for (int k0 = 0; k0 < a.slots; k0 += KB) {
                u32x4 q[KB][V];
                float sc[KB][V];
                int rowOfK[KB];
#pragma unroll
                for (int u = 0; u < KB; ++u) {
                    const int k = k0 + u;
                    const int row = __builtin_amdgcn_readfirstlane((k < a.slots && active) ? s_row[tg][k] : -1);
                    rowOfK[u] = row;
                    // Bounds are the buffer resources' business: an absent row gets resources of zero bytes, so its loads, like
                    // those of the lanes past the end of a row, return zeros without a branch (and without the register
                    // clears a branch would need).
                    const int64_t rowAt = row < 0 ? 0 : row;
                    const char *base = static_cast<const char *>(a.expertOut) + rowAt * a.rowBytes;
                    const __amdgpu_buffer_rsrc_t rsrc = RowResource(base, row < 0 ? 0 : vecs * 16);
                    const bool perRow = INQ == TILEXR_EP_QUANT_TOKEN_INT8;
                    const float *scaleBase = a.inScales + (perRow ? rowAt : rowAt * b128);
                    const __amdgpu_buffer_rsrc_t scaleRsrc = RowResource(scaleBase, row < 0 ? 0 : (perRow ? 4 : b128 * 4));
#pragma unroll
                    for (int j = 0; j < V; ++j) {
                        const int idx = j * G + lane;
                        q[u][j] = __builtin_amdgcn_raw_buffer_load_b128(rsrc, idx * 16, 0,
                            kThroughMemory ? kAuxAgentScope : kAuxNonTemporal);
                        sc[u][j] = __uint_as_float(__builtin_amdgcn_raw_buffer_load_b32(scaleRsrc, perRow ? 0 : (idx >> 3) * 4, 0,
                            kThroughMemory ? kAuxAgentScope : 0));
                    }
                }
#pragma unroll
                for (int u = 0; u < KB; ++u) {
                    if (rowOfK[u] < 0) {
                        continue;                       // uniform across the lanes of a token
                    }
                    const float w = s_w[tg][k0 + u];
#pragma unroll
                    for (int j = 0; j < V; ++j) {
#pragma unroll
                        for (int d = 0; d < 4; ++d) {
                            const uint32_t word = q[u][j][d];
                            float f[4];
                            if (INQ == TILEXR_EP_QUANT_TOKEN_INT8) {
#pragma unroll
                                for (int e = 0; e < 4; ++e) {
                                    f[e] = static_cast<float>(static_cast<int>(static_cast<int8_t>((word >> (8 * e)) & 0xffu)));
                                }
                            } else if (kExactDecode) {
                                Fp8E4m3DecodeWord(word, f);
                            } else {
                                Fp8E4m3DecodeWordFast(word, f);
                            }
#pragma unroll
                            for (int e = 0; e < 4; e += 2) {
                                const float d0 = __fmul_rn(f[e], sc[u][j]);
                                const float d1 = __fmul_rn(f[e + 1], sc[u][j]);
                                float r0;
                                float r1;
                                if (BF16) {
                                    r0 = FloatRoundedToBf16(d0);
                                    r1 = FloatRoundedToBf16(d1);
                                } else {
                                    r0 = __half2float(__ushort_as_half(static_cast<unsigned short>(FloatToHalfRneSat(d0))));
                                    r1 = __half2float(__ushort_as_half(static_cast<unsigned short>(FloatToHalfRneSat(d1))));
                                }
                                acc[j][4 * d + e] = __fadd_rn(acc[j][4 * d + e], __fmul_rn(r0, w));
                                acc[j][4 * d + e + 1] = __fadd_rn(acc[j][4 * d + e + 1], __fmul_rn(r1, w));
                            }
                        }
                    }
                }
            }
        };
        const bool throughMemory = FL && a.flagsSettled == 0;
        if (throughMemory) {
            accumulate(std::false_type {}, std::true_type {});
        } else {
            accumulate(std::false_type {}, std::false_type {});
        }
        if (INQ == TILEXR_EP_QUANT_FP8_BLOCK128) {
            bool sawNan = false;
#pragma unroll
            for (int j = 0; j < V; ++j) {
#pragma unroll
                for (int e = 0; e < 16; ++e) {
                    sawNan |= acc[j][e] != acc[j][e];
                }
            }
            if (__any(sawNan ? 1 : 0)) {
                if (throughMemory) {
                    accumulate(std::true_type {}, std::true_type {});
                } else {
                    accumulate(std::true_type {}, std::false_type {});
                }
            }
        }
        if (a.sharedExpertX != nullptr && active) {
            const u32x4 *sx = reinterpret_cast<const u32x4 *>(static_cast<const char *>(a.sharedExpertX) +
                static_cast<int64_t>(token) * a.h * 2);
#pragma unroll
            for (int j = 0; j < V; ++j) {
                const int idx = j * G + lane;
                if (idx < vecs) {
#pragma unroll
                    for (int half = 0; half < 2; ++half) {
                        const u32x4 v = sx[idx * 2 + half];
#pragma unroll
                        for (int q2 = 0; q2 < 4; ++q2) {
                            float &lo = acc[j][half * 8 + 2 * q2];
                            float &hi = acc[j][half * 8 + 2 * q2 + 1];
                            lo = __fadd_rn(lo, Decode16<BF16>(v[q2] & 0xffffu));
                            hi = __fadd_rn(hi, Decode16<BF16>(v[q2] >> 16));
                        }
                    }
                }
            }
        }
        beforeStores();
        if (tokOk) {
            u32x4 *dst = reinterpret_cast<u32x4 *>(static_cast<char *>(a.y) + static_cast<int64_t>(token) * a.h * 2);
#pragma unroll
            for (int j = 0; j < V; ++j) {
                const int idx = j * G + lane;
                if (idx < vecs) {
#pragma unroll
                    for (int half = 0; half < 2; ++half) {
                        u32x4 o;
#pragma unroll
                        for (int q2 = 0; q2 < 4; ++q2) {
                            o[q2] = active ? EncodePair16Sat<BF16>(acc[j][half * 8 + 2 * q2], acc[j][half * 8 + 2 * q2 + 1]) : 0u;
                        }
                        __builtin_nontemporal_store(o, dst + idx * 2 + half);
                    }
                }
            }
        }
    };
    ForEachGroup<FL>(a, groups, kTokens, tokenAt, load, reduceUnit);
}

// Element-granular reduce for any h / alignment.  One workgroup per token; a thread owns whole 32-column blocks so
// that the MXFP8 round trip needs no cross-lane traffic.
template <bool BF16>
__global__ __launch_bounds__(kThreads) void ep_reduce_generic_kernel(ReduceArgs a, int kind, int inq, int commq)
{
    __shared__ int s_row[kMaxTopK];
    __shared__ float s_w[kMaxTopK];
    const int tid = threadIdx.x;
    const int b128 = (a.h + 127) / 128;
    for (int token = blockIdx.x; token < a.bs; token += gridDim.x) {
        __syncthreads();
        LoadRoutes<true, true>(a, token, true, tid, kThreads, s_row, s_w, kRouteCheck);
        __syncthreads();
        if (kind == kReducePerAdd) {
            if (tid == 0) {
                SortRows(s_row, a.slots, a.orderKeys);
            }
            __syncthreads();
        }
        const bool active = (a.tokenMask == nullptr || a.tokenMask[token] != 0) &&
            !(a.tileFlags != nullptr && AnyExpired(s_row, a.slots));
        uint16_t *dst = static_cast<uint16_t *>(a.y) + static_cast<int64_t>(token) * a.h;
        const int blocks = (a.h + 31) / 32;
        for (int b = tid; b < blocks; b += kThreads) {
            const int begin = b * 32;
            const int end = min(begin + 32, a.h);
            float acc[32];
            for (int i = 0; i < 32; ++i) {
                acc[i] = 0.0f;
            }
            if (active) {
                for (int k = 0; k < a.slots; ++k) {
                    const int row = s_row[k];
                    if (row < 0) {
                        continue;
                    }
                    const float w = s_w[k];
                    const char *base = static_cast<const char *>(a.expertOut) + static_cast<int64_t>(row) * a.rowBytes;
                    float f[32];
                    float amax = 0.0f;
                    for (int i = begin; i < end; ++i) {
                        float v;
                        if (inq == 0) {
                            v = Decode16<BF16>(reinterpret_cast<const uint16_t *>(base)[i]);
                        } else {
                            const uint32_t byte = reinterpret_cast<const uint8_t *>(base)[i];
                            const float d = inq == TILEXR_EP_QUANT_TOKEN_INT8 ?
                                __fmul_rn(static_cast<float>(static_cast<int>(static_cast<int8_t>(byte))), a.inScales[row]) :
                                __fmul_rn(Fp8Decode<false>(byte), a.inScales[static_cast<int64_t>(row) * b128 + i / 128]);
                            v = BF16 ? __uint_as_float(FloatToBf16Rne(d) << 16) :
                                       __half2float(__ushort_as_half(static_cast<unsigned short>(FloatToHalfRneSat(d))));
                        }
                        f[i - begin] = v;
                        amax = fmaxf(amax, fabsf(v));
                    }
                    if (commq != 0) {
                        const bool e5 = commq == TILEXR_EP_QUANT_COMM_MXFP8_E5M2;
                        const int se = e5 ? MxSharedExponent<true>(amax) : MxSharedExponent<false>(amax);
                        const float up = Exp2Int(se);
                        for (int i = 0; i < end - begin; ++i) {
                            const float s = ldexpf(f[i], -se);
                            const float back = e5 ? Fp8Decode<true>(Fp8Encode<true>(s)) : Fp8Decode<false>(Fp8Encode<false>(s));
                            f[i] = __fmul_rn(back, up);
                        }
                    }
                    for (int i = 0; i < end - begin; ++i) {
                        if (kind == kReducePerAdd) {
                            acc[i] = RoundTo16<BF16>(__fadd_rn(acc[i], f[i]));
                        } else {
                            acc[i] = __fadd_rn(acc[i], __fmul_rn(f[i], w));
                        }
                    }
                }
                if (a.sharedExpertX != nullptr) {
                    const uint16_t *sx = static_cast<const uint16_t *>(a.sharedExpertX) + static_cast<int64_t>(token) * a.h;
                    for (int i = begin; i < end; ++i) {
                        acc[i - begin] = __fadd_rn(acc[i - begin], Decode16<BF16>(sx[i]));
                    }
                }
            }
            for (int i = begin; i < end; ++i) {
                dst[i] = active ? static_cast<uint16_t>(Encode16Sat<BF16>(acc[i - begin])) : static_cast<uint16_t>(0);
            }
        }
    }
}

template <int G, int V, int KIND, bool BF16, int COMMQ>
void LaunchVec(const ReduceArgs &a, int gridLimit, hipStream_t stream)
{
    if constexpr (G == kThreads) {
        // whole-workgroup tokens are only used for rows published through readiness flags
        int grid = a.bs;
        if (gridLimit > 0 && grid > gridLimit) {
            grid = gridLimit;
        }
        hipLaunchKernelGGL((ep_reduce_vec_kernel<G, V, KIND, BF16, COMMQ, true>), dim3(grid), dim3(kThreads), 0, stream, a);
        return;
    }
    // sliced rows: one wave per workgroup, so that no wave waits at a barrier for another slice's rows
    const int threads = a.colSlices > 1 ? G : kThreads;
    const int perGroup = threads / G;
    const int64_t units = static_cast<int64_t>(a.bs) * a.colSlices;
    int grid = static_cast<int>((units + perGroup - 1) / perGroup);
    if (gridLimit > 0 && grid > gridLimit * (kThreads / threads)) {
        grid = gridLimit * (kThreads / threads);
    }
    if (a.tileFlags != nullptr) {
        hipLaunchKernelGGL((ep_reduce_vec_kernel<G, V, KIND, BF16, COMMQ, true>), dim3(grid), dim3(threads), 0, stream, a);
    } else {
        hipLaunchKernelGGL((ep_reduce_vec_kernel<G, V, KIND, BF16, COMMQ, false>), dim3(grid), dim3(threads), 0, stream, a);
    }
}

template <int G, int V, bool BF16>
void LaunchByMode(const ReduceLaunch &l, const ReduceArgs &a, int gridLimit)
{
    if (l.reduceKind == kReducePerAdd) {
        LaunchVec<G, V, kReducePerAdd, BF16, 0>(a, gridLimit, l.stream);
    } else if (l.commQuant == TILEXR_EP_QUANT_COMM_MXFP8_E5M2) {
        LaunchVec<G, V, kReduceFp32, BF16, TILEXR_EP_QUANT_COMM_MXFP8_E5M2>(a, gridLimit, l.stream);
    } else if (l.commQuant == TILEXR_EP_QUANT_MXFP8) {
        LaunchVec<G, V, kReduceFp32, BF16, TILEXR_EP_QUANT_MXFP8>(a, gridLimit, l.stream);
    } else {
        LaunchVec<G, V, kReduceFp32, BF16, 0>(a, gridLimit, l.stream);
    }
}

template <int G, int V>
void LaunchByType(const ReduceLaunch &l, const ReduceArgs &a, int gridLimit)
{
    if (l.bf16) {
        LaunchByMode<G, V, true>(l, a, gridLimit);
    } else {
        LaunchByMode<G, V, false>(l, a, gridLimit);
    }
}

template <int G, int V, int INQ>
void LaunchQuantKernel(const ReduceLaunch &l, const ReduceArgs &a, dim3 g, dim3 b)
{
    if (l.bf16) {
        if (a.tileFlags != nullptr) {
            hipLaunchKernelGGL((ep_reduce_quant_kernel<G, V, INQ, true, true>), g, b, 0, l.stream, a);
        } else {
            hipLaunchKernelGGL((ep_reduce_quant_kernel<G, V, INQ, true, false>), g, b, 0, l.stream, a);
        }
    } else {
        if (a.tileFlags != nullptr) {
            hipLaunchKernelGGL((ep_reduce_quant_kernel<G, V, INQ, false, true>), g, b, 0, l.stream, a);
        } else {
            hipLaunchKernelGGL((ep_reduce_quant_kernel<G, V, INQ, false, false>), g, b, 0, l.stream, a);
        }
    }
}

template <int G, int V>
void LaunchQuant(const ReduceLaunch &l, const ReduceArgs &a, int gridLimit)
{
    constexpr int kTokens = kThreads / G;
    int grid = (a.bs + kTokens - 1) / kTokens;
    if (gridLimit > 0 && grid > gridLimit) {
        grid = gridLimit;
    }
    const dim3 g(grid);
    const dim3 b(kThreads);
    if (l.inQuant == TILEXR_EP_QUANT_TOKEN_INT8) {
        LaunchQuantKernel<G, V, TILEXR_EP_QUANT_TOKEN_INT8>(l, a, g, b);
    } else {
        LaunchQuantKernel<G, V, TILEXR_EP_QUANT_FP8_BLOCK128>(l, a, g, b);
    }
}

} // namespace

hipError_t LaunchReduce(const ReduceLaunch &l)
{
    ReduceArgs a {};
    a.expertOut = l.expertOut;
    a.rowBytes = l.rowBytes;
    a.inverseTagged = l.inverseTagged;
    a.epoch = l.epoch;
    a.rowIndexMap = l.rowIndexMap;
    a.orderKeys = l.orderKeys;
    a.expertScales = l.expertScales;
    a.tokenMask = l.tokenMask;
    a.sharedExpertX = l.sharedExpertX;
    a.inScales = l.inScales;
    a.bs = static_cast<int>(l.bs);
    a.h = static_cast<int>(l.h);
    a.topK = static_cast<int>(l.topK);
    a.slots = static_cast<int>(l.topK + l.sharedSlots);
    a.maxRows = l.maxRows > 0 ? static_cast<int>(l.maxRows) : 0x7fffffff;
    a.y = l.y;
    a.tileFlags = l.tileFlags;
    a.tileRows = static_cast<int>(l.tileRows);
    a.flagEpoch = l.flagEpoch;
    a.waitTimeoutTicks = l.waitTimeoutTicks;
    a.deviceStatus = l.deviceStatus;
    a.flagsSettled = (l.tileFlags != nullptr && l.producerOrdered) ? 1 : 0;
    a.colSlices = 1;
    // A kernel that waits on flags must never crowd out the producer it waits for: its waiting waves keep their
    // registers, and with three or more of these workgroups per compute unit a producer workgroup no longer fits
    // beside them (measured: flag waits expire at six).  Two workgroups per compute unit walk the tokens.
    // A launch whose flags were published earlier on its own stream never waits and gets the ordinary geometry.
    const bool mayWait = l.tileFlags != nullptr && !l.producerOrdered;
    const int gridLimit = mayWait ? 2 * (l.numComputeUnits > 0 ? l.numComputeUnits : 256) : 0;
    const int64_t vecs = l.h / 8;
    const bool plain = l.inQuant == 0 && l.h % 8 == 0 && Aligned16(l.y) && vecs <= 8 * kThreads &&
        Aligned16(l.expertOut) && l.rowBytes % 16 == 0 &&
        (l.sharedExpertX == nullptr || Aligned16(l.sharedExpertX)) && (l.commQuant == 0 || l.h % 32 == 0);
    const int64_t qvecs = l.h / 16;
    const bool quant = l.inQuant != 0 && l.commQuant == 0 && l.reduceKind == kReduceFp32 && l.h % 16 == 0 &&
        qvecs <= 4 * kThreads && Aligned16(l.y) && Aligned16(l.expertOut) && l.rowBytes % 16 == 0 &&
        (l.sharedExpertX == nullptr || Aligned16(l.sharedExpertX));
    if (l.kernelNameOut != nullptr) {
        *l.kernelNameOut = quant ? "ep_reduce_quant_kernel" : (plain ? "ep_reduce_vec_kernel" : "ep_reduce_generic_kernel");
    }
    if (quant) {
        if (qvecs <= kWave) {
            LaunchQuant<kWave, 1>(l, a, gridLimit);
        } else if (qvecs <= 2 * kWave) {
            LaunchQuant<2 * kWave, 1>(l, a, gridLimit);
        } else if (qvecs <= kThreads) {
            LaunchQuant<kThreads, 1>(l, a, gridLimit);
        } else if (qvecs <= 2 * kThreads) {
            LaunchQuant<kThreads, 2>(l, a, gridLimit);
        } else {
            LaunchQuant<kThreads, 4>(l, a, gridLimit);
        }
    } else if (plain) {
        // a wave per token for narrow rows; wide rows are cut into slices of 128 vectors, one wave each (many small
        // independent waves with four rows in flight each reach the highest gather bandwidth here)
        a.colSlices = 1;
        if (vecs <= 2 * kWave) {
            LaunchByType<kWave, 2>(l, a, gridLimit);
        } else if (vecs <= 4 * kWave) {
            LaunchByType<kWave, 4>(l, a, gridLimit);
        } else if (mayWait) {
            // readiness flags that may still be pending: one workgroup per token, so that one wave polls the token's
            // tiles instead of one per slice, and few enough workgroups that the producer fits beside them
            if (vecs <= 2 * kThreads) {
                LaunchByType<kThreads, 2>(l, a, gridLimit);
            } else if (vecs <= 4 * kThreads) {
                LaunchByType<kThreads, 4>(l, a, gridLimit);
            } else {
                LaunchByType<kThreads, 8>(l, a, gridLimit);
            }
        } else {
            a.colSlices = static_cast<int>((vecs + 2 * kWave - 1) / (2 * kWave));
            LaunchByType<kWave, 2>(l, a, gridLimit);
        }
    } else {
        int grid = static_cast<int>(l.bs);
        if (gridLimit > 0 && grid > gridLimit) {
            grid = gridLimit;
        }
        if (l.bf16) {
            hipLaunchKernelGGL((ep_reduce_generic_kernel<true>), dim3(grid), dim3(kThreads), 0, l.stream, a,
                l.reduceKind, l.inQuant, l.commQuant);
        } else {
            hipLaunchKernelGGL((ep_reduce_generic_kernel<false>), dim3(grid), dim3(kThreads), 0, l.stream, a,
                l.reduceKind, l.inQuant, l.commQuant);
        }
    }
    return hipGetLastError();
}

} // namespace TileXREp
