// rows: destination row and assist tuple of every route in ONE launch (gfx950, wave64; memory route, one rank, keys =
// experts, no mask, no capacity limit, up to kRowsTableRoutes routes).  Replaces the count launch's ticket and
// last-workgroup scan and the separate place launch.
//
// What such a kernel costs on this part, measured: a hand-over between launches or workgroups is a round trip through
// memory, 2 to 4 us while other traffic is about; LDS atomics run at about four lanes a clock (a histogram of 32 768
// ids is 4 to 5 us however the counters are laid out); and a wave that runs alone on its SIMD issues a dependent
// instruction only every 4 ns or so, so 1500 instructions per wave are 6 us whatever they do.  Hence: no hand-over, no
// histogram, few instructions per wave, many waves.
//
// The work is cut by KEY, not by route.  A workgroup of 16 waves takes key k and reads the WHOLE id table, wave w the
// w-th sixteenth of it in flat route order (16-byte loads, eight in flight per lane; L2 hits after an XCD's first
// workgroup).  Without a capacity limit
//   row of a route with id k = (valid ids below k in the whole table) + (earlier routes with id k)
// so pass 1 is two compares and two adds per id, all per lane, and one reduction per wave at its end; the waves'
// counts meet in LDS; pass 2 ranks the lanes that hold id k, slot by slot, and writes their rows and tuples.  Nobody
// waits for another workgroup; every rowOf entry and every tuple is written by exactly one workgroup (routes whose id
// names no expert get their -1 from one more workgroup behind those of the keys).  Workgroup k also knows
// sendCounts[k] (ids up to k) and expertTokenNums[k] without any scan.  Counting is cheap and ranking is not (a wave
// ranks its slots one after the other), so when the keys are few a key gets several workgroups: each counts the whole
// table and ranks one part of every wave's sixteenth.
//
// Same definitions as the count + place pair (reference: src/ep/kernels/tilexr_ep_dispatch_memory_kernel.h:791-818
// rank within expert, :820-1089 count exchange and inclusive cumulative sum, :1142-1168 count outputs, :1240-1258
// assist tuple).
#include <hip/hip_runtime.h>

#include "ep_chunk_rank.hip.h"
#include "ep_kernel_common.hip.h"
#include "ep_launch.h"
#include "ep_numerics.hip.h"

namespace TileXREp {
namespace {

constexpr int kRowsThreads = 1024;
constexpr int kRowsWaves = kRowsThreads / kWave;
constexpr int kRowsSlotRoutes = 4 * kWave;             // routes a wave takes with one 16-byte load per lane
constexpr int kRowsWarmLoads = 4;
constexpr int kRowsBatch = 8;                          // 16-byte loads a lane has in flight
constexpr int kRowsPartSlots = 16;                     // slots a wave ranks at most: four bits per slot in one 64-bit word
constexpr int kRowsMaxParts = 16;
static_assert(kRowsTableRoutes <= kRowsMaxParts * kRowsPartSlots * kRowsWaves * kRowsSlotRoutes, "parts x slots cover the largest table");

struct RouteRowsArgs {
    const int32_t *ids;
    int n;
    int topK;
    int numKeys;
    int slots;                   // slots per wave: wave w owns routes [w, w + 1) * slots * 256 (its sixteenth of the table)
    int parts;                   // workgroups per key
    int partSlots;               // slots of its sixteenth that a wave of workgroup (key, part) ranks: [part, part + 1) * partSlots
    int32_t srcRank;
    int32_t expertIdBias;
    int32_t *rowOf;              // [n] out
    int32_t *assist;             // [rows, 4] out
    int assistAligned;           // the tuples can go out as one 16-byte store each
    int32_t *totalRowsOut;       // device word: rows the dispatch keeps
    int32_t *sendCountsOut;
    int64_t *expertTokenNumsOut;
    int tokenNumsType;
    const u32x4 *warmRows;
    int64_t warmVecs;
};

typedef int i32x4 __attribute__((ext_vector_type(4)));


__device__ __forceinline__ int WaveSum(int v)
{
#pragma unroll
    for (int off = kWave / 2; off >= 1; off >>= 1) {
        v += __shfl_xor(v, off);
    }
    return v;
}

// Slots s0 .. s0 + kRowsBatch - 1 of the wave's sixteenth (those below `slots`), all requested before any is looked
// at: slot s, lane l holds routes waveFirst + s * 256 + l * 4 ... + 3.  Elements beyond the table read as 0 (the buffer
// bound sees to that), which names an expert: the kernel corrects its counts by their number, which it knows, instead
// of patching the registers (they come last in route order, so they disturb no rank).
__device__ __forceinline__ void LoadSlots(const __amdgpu_buffer_rsrc_t &table, int waveFirst, int s0, int slots, int lane,
    i32x4 (&id)[kRowsBatch])
{
#pragma unroll
    for (int u = 0; u < kRowsBatch; ++u) {
        if (s0 + u < slots) {
            id[u] = __builtin_bit_cast(i32x4, __builtin_amdgcn_raw_buffer_load_b128(table, (waveFirst + (s0 + u) * kRowsSlotRoutes + lane * 4) * 4, 0, 0));
        }
    }
}

// The kernel stays within 64 registers per lane whatever the table's size (ids are streamed, eight loads a lane at a
// time, and only one bit per id is kept), so that two workgroups of 1024 lanes fit a compute unit: the workgroups that
// read token rows start beside the routing ones instead of behind them (58.7 MB read in 15.6 us when they had to wait,
// the routing workgroups alone taking 9).
//
// SPLIT: a key has several workgroups (a.parts > 1).  The common case of one per key is compiled without the tests
// that tell a workgroup's own slots from the rest.
template <bool SPLIT>
__global__ __launch_bounds__(kRowsThreads, 8) void ep_route_rows_kernel(RouteRowsArgs a)
{
    __shared__ int s_less[kRowsWaves];
    __shared__ int s_same[kRowsWaves];

    const int tid = threadIdx.x;
    const int wave = tid / kWave;
    const int lane = tid & (kWave - 1);
    const int keyBlocks = SPLIT ? a.numKeys * a.parts : a.numKeys;
    const int block = blockIdx.x;
    if (block > keyBlocks) {
        // not a routing workgroup.  A routing workgroup takes half a compute unit's wave slots, so only one of these
        // fits beside it: each carries four loads per lane to keep as much in flight as the smaller ones did
        WarmTokenRows<kRowsThreads, kRowsWarmLoads>(a.warmRows, a.warmVecs, block - keyBlocks - 1);
        return;
    }
    const int waveFirst = wave * a.slots * kRowsSlotRoutes;
    const __amdgpu_buffer_rsrc_t table = RowResource(a.ids, a.n * 4);

    if (block == keyBlocks) {
        // ids outside [0, E) are skipped, not errors: their routes have no row, and this workgroup says so
        const unsigned keys = static_cast<unsigned>(a.numKeys);
#pragma unroll 1
        for (int s0 = 0; s0 < a.slots; s0 += kRowsBatch) {
            i32x4 id[kRowsBatch];
            LoadSlots(table, waveFirst, s0, a.slots, lane, id);
#pragma unroll
            for (int u = 0; u < kRowsBatch; ++u) {
                if (s0 + u < a.slots) {
                    const bool none = static_cast<unsigned>(id[u][0]) >= keys || static_cast<unsigned>(id[u][1]) >= keys ||
                        static_cast<unsigned>(id[u][2]) >= keys || static_cast<unsigned>(id[u][3]) >= keys;
                    if (__ballot(none) != 0ull) {
                        const int route = waveFirst + (s0 + u) * kRowsSlotRoutes + lane * 4;
#pragma unroll 1
                        for (int e = 0; e < 4; ++e) {
                            if (route + e < a.n && static_cast<unsigned>(id[u][e]) >= keys) {
                                a.rowOf[route + e] = -1;
                            }
                        }
                    }
                }
            }
        }
        return;
    }
    const int key = SPLIT ? block / a.parts : block;
    const int part = SPLIT ? block - key * a.parts : 0;
    const int mineFirst = SPLIT ? part * a.partSlots : 0;           // the slots this workgroup's waves rank: [mineFirst, mineEnd)
    const int mineEnd = SPLIT ? (mineFirst + a.partSlots < a.slots ? mineFirst + a.partSlots : a.slots) : a.slots;

    // pass 1, over the wave's whole sixteenth: per lane, ids below the key (unsigned compare: negative ids are above
    // every key) and ids equal to it, those ahead of the workgroup's own slots counted apart; which elements of its own
    // slots are equal is kept, four bits per slot, so that pass 2 needs no id any more
    int less = 0;
    int same = 0;
    int sameAhead = 0;
    uint64_t bits = 0;
#pragma unroll 1
    for (int s0 = 0; s0 < a.slots; s0 += kRowsBatch) {
        i32x4 id[kRowsBatch];
        LoadSlots(table, waveFirst, s0, a.slots, lane, id);
#pragma unroll
        for (int u = 0; u < kRowsBatch; ++u) {
            const int s = s0 + u;
            if (s < a.slots) {
                uint32_t mine = 0u;
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    less += static_cast<unsigned>(id[u][e]) < static_cast<unsigned>(key) ? 1 : 0;
                    mine |= id[u][e] == key ? 1u << e : 0u;
                }
                const int hits = __popc(mine);
                same += hits;
                if (SPLIT) {
                    sameAhead += s < mineFirst ? hits : 0;
                }
                if (!SPLIT || (s >= mineFirst && s < mineEnd)) {
                    bits |= static_cast<uint64_t>(mine) << ((s - mineFirst) * 4);
                }
            }
        }
    }
    less = WaveSum(less);
    same = WaveSum(same);
    if (lane == 0) {
        s_less[wave] = less;
        s_same[wave] = same;
    }
    __syncthreads();
    // elements beyond the table read as id 0: below every other key, equal to key 0
    const int beyond = kRowsWaves * a.slots * kRowsSlotRoutes - a.n;
    // lane w of every wave takes wave w's two counts; sums over the lanes (few registers: this kernel has 64)
    const int lessOf = lane < kRowsWaves ? s_less[lane] : 0;
    const int sameOf = lane < kRowsWaves ? s_same[lane] : 0;
    const int lessTotal = WaveSum(lessOf) - (key > 0 ? beyond : 0);
    const int total = WaveSum(sameOf) - (key == 0 ? beyond : 0);

    // pass 2: slot by slot, the lanes that hold the key are ranked (flat route order within a slot: lane, then element)
    if (__ballot(bits != 0ull) != 0ull) {
        // routes with this key earlier in route order: in earlier waves' sixteenths, and ahead of these slots in this one
        const int before = WaveSum((lane < wave ? sameOf : 0) + sameAhead);
        const unsigned long long lt = LaneMaskLt();
        int running = lessTotal + before;
        // (token, k) of the lane's first route, then 256 routes on per slot: one division per wave, none per route
        const int first = waveFirst + mineFirst * kRowsSlotRoutes + lane * 4;
        int token = first / a.topK;
        int k = first - token * a.topK;
        const int stepToken = kRowsSlotRoutes / a.topK;
        const int stepK = kRowsSlotRoutes - stepToken * a.topK;
#pragma unroll 1
        for (int s = 0; s < mineEnd - mineFirst; ++s) {
            const uint32_t mine = static_cast<uint32_t>(bits >> (s * 4)) & 15u;
            if (__ballot(mine != 0u) != 0ull) {
                const unsigned long long hit0 = __ballot((mine & 1u) != 0u);
                const unsigned long long hit1 = __ballot((mine & 2u) != 0u);
                const unsigned long long hit2 = __ballot((mine & 4u) != 0u);
                const unsigned long long hit3 = __ballot((mine & 8u) != 0u);
                int row = running + __popcll(hit0 & lt) + __popcll(hit1 & lt) + __popcll(hit2 & lt) + __popcll(hit3 & lt);
                running += __popcll(hit0) + __popcll(hit1) + __popcll(hit2) + __popcll(hit3);
                // a lane seldom holds more than one route of the key in a slot: a loop over its set bits, not its elements
                const int route = first + s * kRowsSlotRoutes;
                for (uint32_t left = mine; left != 0u; left &= left - 1u) {
                    const int e = __builtin_ctz(left);
                    if (route + e >= a.n) {
                        break;              // beyond the table (key 0 only): nothing real follows in this lane
                    }
                    int kOf = k + e;
                    int tokenOf = token;
                    while (kOf >= a.topK) {
                        kOf -= a.topK;
                        ++tokenOf;
                    }
                    const i32x4 tuple = {a.srcRank, tokenOf, kOf, key + a.expertIdBias};
                    int32_t *out = a.assist + static_cast<int64_t>(row) * 4;
                    if (a.assistAligned != 0) {
                        *reinterpret_cast<i32x4 *>(out) = tuple;
                    } else {
                        out[0] = tuple[0];
                        out[1] = tuple[1];
                        out[2] = tuple[2];
                        out[3] = tuple[3];
                    }
                    a.rowOf[route + e] = row;
                    ++row;
                }
            }
            token += stepToken;
            k += stepK;
            if (k >= a.topK) {
                k -= a.topK;
                ++token;
            }
        }
    }
    if (tid == 0 && part == 0) {
        // ids up to this key = the inclusive cumulative sum the counts output holds
        const int incl = lessTotal + total;
        if (a.sendCountsOut != nullptr) {
            a.sendCountsOut[key] = incl;
        }
        if (a.expertTokenNumsOut != nullptr) {
            a.expertTokenNumsOut[key] = a.tokenNumsType == 0 ? incl : total;
        }
        if (key == a.numKeys - 1) {
            *a.totalRowsOut = incl;
        }
    }
}

} // namespace

bool RouteRowsFits(const int32_t *ids, int64_t routes, int64_t numKeys, int maskMode, int64_t capacity)
{
    return routes > 0 && routes <= kRowsTableRoutes && numKeys > 0 && numKeys <= kMaxKeys && maskMode == kMaskNone &&
        capacity <= 0 && Aligned16(ids);
}

// Where the one-launch routing is the faster choice.  Every key's workgroups read and count the whole table, so the
// launch grows with routes x experts where the count launch does not.  Measured on dispatch + combine layers over
// 8192 .. 262 144 routes x 8 .. 2048 experts against count (+ place), both kernels forced in turn on the same buffers:
//   up to 16 384 routes              2-6 us faster throughout (level at 2048 experts without a place launch to save)
//   with workgroups that read token rows ahead in the same launch (14 KiB rows, bf16)
//     32 768 routes                  2-4 us faster up to 256 experts against count + place (rowsAhead: readiness flags
//                                    or the metadata event want the rows resolved before the scatter), level against a
//                                    count launch alone; 4-14 us slower from 1024 experts on
//     49 152 routes and more         level at best, 5-28 us slower from 512 experts on
//   without them (quantised payloads, 4 KiB rows)
//     32 768 routes                  1-4 us faster up to 512 experts
//     65 536 routes                  1-4 us faster up to 64 experts, level up to 256, slower beyond
//     131 072 routes and more        slower from 64 experts on (3-14 us at 128-256 experts, 200 us at 262 144 x 1024)
bool RouteRowsPays(int64_t routes, int64_t numKeys, bool rowsAhead, bool readsRowsAhead)
{
    if (routes <= 16384) {
        return rowsAhead || numKeys <= 1024;
    }
    if (readsRowsAhead) {
        return rowsAhead && routes <= 32768 && numKeys <= 256;
    }
    return routes <= 32768 ? numKeys <= 512 : (routes <= 65536 && numKeys <= 64);
}

hipError_t LaunchRouteRows(const RouteRowsLaunch &l)
{
    const int64_t n = l.bs * l.topK;
    if (!RouteRowsFits(l.ids, n, l.numKeys, kMaskNone, 0)) {
        return hipErrorInvalidValue;
    }
    RouteRowsArgs a {};
    a.ids = l.ids;
    a.n = static_cast<int>(n);
    a.topK = static_cast<int>(l.topK);
    a.numKeys = static_cast<int>(l.numKeys);
    a.slots = static_cast<int>((n + kRowsWaves * kRowsSlotRoutes - 1) / (kRowsWaves * kRowsSlotRoutes));
    // Workgroups per key: more while the keys alone leave most compute units without a routing workgroup (each one
    // reads and counts the whole table, but ranks only its share of the key's routes, which is the longer part), and
    // as many as it takes to keep a wave's share within kRowsPartSlots slots.
    int parts = 1;
    while (parts < kRowsMaxParts && l.numKeys * parts < 256 && parts * 2 <= a.slots) {
        parts *= 2;
    }
    while ((a.slots + parts - 1) / parts > kRowsPartSlots) {
        parts *= 2;
    }
    a.partSlots = (a.slots + parts - 1) / parts;
    a.parts = (a.slots + a.partSlots - 1) / a.partSlots;
    a.srcRank = l.srcRank;
    a.expertIdBias = l.expertIdBias;
    a.rowOf = l.rowOf;
    a.assist = l.assist;
    a.assistAligned = Aligned16(l.assist) ? 1 : 0;
    a.totalRowsOut = l.totalRowsOut;
    a.sendCountsOut = l.sendCountsOut;
    a.expertTokenNumsOut = l.expertTokenNumsOut;
    a.tokenNumsType = l.tokenNumsType;
    // the keys' workgroups, one for the routes without an expert, then those that read token rows
    unsigned blocks = static_cast<unsigned>(l.numKeys) * static_cast<unsigned>(a.parts) + 1u;
    if (l.warmRows != nullptr && l.warmBytes >= 16 && Aligned16(l.warmRows)) {
        a.warmRows = static_cast<const u32x4 *>(l.warmRows);
        a.warmVecs = l.warmBytes / 16;
        blocks += WarmWorkgroups(a.warmVecs, kRowsThreads, kRowsWarmLoads);
    }
    if (a.parts > 1) {
        hipLaunchKernelGGL(ep_route_rows_kernel<true>, dim3(blocks), dim3(kRowsThreads), 0, l.stream, a);
    } else {
        hipLaunchKernelGGL(ep_route_rows_kernel<false>, dim3(blocks), dim3(kRowsThreads), 0, l.stream, a);
    }
    return hipGetLastError();
}

} // namespace TileXREp
