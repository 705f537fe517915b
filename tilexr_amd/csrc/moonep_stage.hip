// Plan-driven (MoonEP) dispatch / combine kernels for ranks that share one MI355X (gfx950, wave64).
//
// HBM-bound row movement, no MFMA.  A plan names the destination row of every route directly, so there is nothing to
// count: dispatch is one read of each token row and one write per route; combine is one read per route and one write
// per token.  Row copies use two 16-byte loads and two 16-byte stores per lane, and the workgroups of one token are
// given block indices that land on one XCD (block b runs on XCD b % 8) so the token row is read from HBM once.
//
//   what is computed  reference: src/moonep/dispatch/kernels/tilexr_moonep_dispatch_kernel.cpp:108-147, 268-461
//                                src/moonep/combine/kernels/tilexr_moonep_combine_kernel.cpp:117-177, 285-366, 449-541,
//                                568-606, 648-733
#include <hip/hip_runtime.h>

#include "ep_kernel_common.cuh"
#include "ep_numerics.cuh"
#include "moonep_stage.h"

namespace TileXRMoon {
namespace {

using TileXREp::u32x4;
using TileXREp::kThreads;
using TileXREp::kWave;

constexpr int kXcds = 8;
constexpr int kRowVecs = 2;     // 16-byte vectors per lane per row slice

const char *gScatterName = "";
const char *gReduceName = "";

__device__ __forceinline__ bool Tagged(uint64_t word, uint64_t epoch)
{
    return (word >> 32) == epoch;
}

__device__ __forceinline__ uint64_t Tag(uint64_t epoch, uint32_t value)
{
    return (epoch << 32) | value;
}

// Row tag values: a route names the row (its weight is written); a route also wrote the row's hidden values.
constexpr uint32_t kRowNamed = 2u;
constexpr uint32_t kRowWritten = 1u;

// reference: dispatch kernel :268-279
struct Route {
    int peer;
    int row;
    bool duplicate;
    bool ok;
};

__device__ __forceinline__ Route Decode(int32_t encoded, int64_t nvS, int world)
{
    const int64_t e = encoded;
    const int64_t raw = e >= 0 ? e : -e - 1;
    const int64_t peer = raw / nvS;
    Route r;
    r.ok = peer < world;
    r.peer = r.ok ? static_cast<int>(peer) : 0;
    r.row = static_cast<int>(raw % nvS);
    r.duplicate = encoded < 0;
    return r;
}

__device__ __forceinline__ void RecordFailure(const WorldTables &t, int rank, uint64_t epoch, int32_t code)
{
    __hip_atomic_store(&t.fail[rank], Tag(epoch, static_cast<uint32_t>(code)), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

// ---------------------------------------------------------------------------------------------------------------
// dispatch: scatter
// ---------------------------------------------------------------------------------------------------------------
struct ScatterArgs {
    const int32_t *dst;
    const void *hiddenSh;
    const float *weightsSk;
    int s, k, h;
    int64_t nvS;
    int world;
    int srcRank;
    int colSlices;
    ReceiveTable out;
    WorldTables t;
    uint64_t epoch;
};

// What the route's first workgroup records besides the row: the weight, the row tag and -- while the duplicate plan is
// being built -- which primary a duplicate belongs to and where it stands among that primary's duplicates.  Called by
// the first wave of the workgroup, all 64 lanes; s_dst holds the token's K route words.
//   primary of a duplicate = first earlier non-duplicate route of the token to the same rank (dispatch kernel :281-301)
//   the plan lists a primary's duplicates in ascending row order (dispatch kernel :393-419), so the rank of a
//   duplicate within its group is the number of the token's duplicates to that rank with a smaller row
template <bool FRESH>
__device__ __forceinline__ void RouteRecords(const ScatterArgs &a, int token, int k, const Route &r, const int32_t *s_dst)
{
    const int lane = threadIdx.x;
    const int64_t at = static_cast<int64_t>(r.peer) * a.t.stride + r.row;
    if (lane == 0) {
        if (a.weightsSk != nullptr) {
            a.out.weights[r.peer][r.row] = a.weightsSk[static_cast<int64_t>(token) * a.k + k];
        }
        a.t.rowTag[at] = Tag(a.epoch, (FRESH || !r.duplicate) ? (kRowNamed | kRowWritten) : kRowNamed);
    }
    if (!FRESH || !r.duplicate) {
        return;
    }
    Route other {0, 0, false, false};
    if (lane < a.k) {
        other = Decode(s_dst[lane], a.nvS, a.world);
    }
    const bool samePeer = lane < a.k && other.ok && other.peer == r.peer;
    const uint64_t primaries = __ballot(samePeer && !other.duplicate && lane < k);
    const uint64_t siblings = __ballot(samePeer && other.duplicate);
    const uint64_t before = __ballot(samePeer && other.duplicate && other.row < r.row);
    if (primaries == 0) {
        if (lane == 0) {
            RecordFailure(a.t, a.srcRank, a.epoch, kDispatchInvalidRoute);
        }
        return;
    }
    const int primaryLane = __ffsll(static_cast<unsigned long long>(primaries)) - 1;
    const int primaryRow = __shfl(other.row, primaryLane);
    if (lane == 0) {
        a.t.parentTag[at] = Tag(a.epoch, static_cast<uint32_t>(primaryRow) + 1u);
        a.t.sibling[at] = static_cast<uint32_t>(__popcll(before)) | (static_cast<uint32_t>(__popcll(siblings)) << 16);
    }
}

// One workgroup per (token, route, slice of 512 vectors).  FRESH: the duplicate plan is being built from these very
// route words, so a duplicate row is by construction a copy of this token's row and is written here; otherwise
// duplicate rows are left to the fill kernel, which copies them from the primary the saved plan names.
template <bool FRESH>
__global__ __launch_bounds__(kThreads) void moon_scatter_kernel(ScatterArgs a)
{
    __shared__ int32_t s_dst[kMaxTopK];
    const int xcd = blockIdx.x % kXcds;
    const int j = blockIdx.x / kXcds;
    const int perToken = a.k * a.colSlices;
    const int token = (j / perToken) * kXcds + xcd;
    const int k = (j % perToken) / a.colSlices;
    const int slice = (j % perToken) % a.colSlices;
    if (token >= a.s) {
        return;
    }
    const int lane = threadIdx.x;
    const int vecs = a.h / 8;
    const int colBase = slice * (kRowVecs * kThreads);
    const int32_t *words = a.dst + static_cast<int64_t>(token) * a.k;
    const bool records = slice == 0;
    if (FRESH && records && lane < a.k) {
        s_dst[lane] = words[lane];
    }
    const int32_t encoded = words[k];
    const u32x4 *src = reinterpret_cast<const u32x4 *>(static_cast<const char *>(a.hiddenSh) +
        static_cast<int64_t>(token) * a.h * 2);
    u32x4 v[kRowVecs];
#pragma unroll
    for (int i = 0; i < kRowVecs; ++i) {
        const int idx = colBase + i * kThreads + lane;
        v[i] = idx < vecs ? src[idx] : u32x4{0u, 0u, 0u, 0u};
    }
    const Route r = Decode(encoded, a.nvS, a.world);
    if (!r.ok) {
        if (records && lane == 0) {
            RecordFailure(a.t, a.srcRank, a.epoch, kDispatchInvalidRoute);
        }
        return;
    }
    if (FRESH || !r.duplicate) {
        u32x4 *dstRow = reinterpret_cast<u32x4 *>(static_cast<char *>(a.out.hidden[r.peer]) +
            static_cast<int64_t>(r.row) * a.h * 2);
#pragma unroll
        for (int i = 0; i < kRowVecs; ++i) {
            const int idx = colBase + i * kThreads + lane;
            if (idx < vecs) {
                __builtin_nontemporal_store(v[i], dstRow + idx);
            }
        }
    }
    if (records) {
        if (FRESH) {
            TileXREp::LdsBarrier();
        }
        if (lane < kWave) {
            RouteRecords<FRESH>(a, token, k, r, s_dst);
        }
    }
}

// Any hidden size and alignment: one workgroup per route, 2-byte elements.
template <bool FRESH>
__global__ __launch_bounds__(kThreads) void moon_scatter_generic_kernel(ScatterArgs a)
{
    __shared__ int32_t s_dst[kMaxTopK];
    const int token = blockIdx.x / a.k;
    const int k = blockIdx.x % a.k;
    const int lane = threadIdx.x;
    const int32_t *words = a.dst + static_cast<int64_t>(token) * a.k;
    if (FRESH && lane < a.k) {
        s_dst[lane] = words[lane];
    }
    const Route r = Decode(words[k], a.nvS, a.world);
    if (!r.ok) {
        if (lane == 0) {
            RecordFailure(a.t, a.srcRank, a.epoch, kDispatchInvalidRoute);
        }
        return;
    }
    if (FRESH || !r.duplicate) {
        const uint16_t *src = static_cast<const uint16_t *>(a.hiddenSh) + static_cast<int64_t>(token) * a.h;
        uint16_t *dstRow = static_cast<uint16_t *>(a.out.hidden[r.peer]) + static_cast<int64_t>(r.row) * a.h;
        for (int c = lane; c < a.h; c += kThreads) {
            dstRow[c] = src[c];
        }
    }
    if (FRESH) {
        TileXREp::LdsBarrier();
    }
    if (lane < kWave) {
        RouteRecords<FRESH>(a, token, k, r, s_dst);
    }
}

// ---------------------------------------------------------------------------------------------------------------
// dispatch: duplicate plan of one destination rank from the parent records (fresh plans)
// ---------------------------------------------------------------------------------------------------------------
struct BuildArgs {
    int64_t nvS;
    int rank;
    WorldTables t;
    uint64_t epoch;
    int32_t *dupGroups;
    int32_t *dupLoffs;
    int32_t *dupCounts;
};

// The reference scans the destination's rows in ascending order: a group is opened by the first duplicate row of its
// primary, groups take their dupLoffs slices in that order, and each slice lists its duplicates in ascending row order
// (dispatch kernel :330-424).  With the rank-within-group and group size recorded by the sources, both numberings are
// exclusive prefix sums over the rows: group index = number of earlier group-opening rows, slice start = sum of their
// group sizes.  One workgroup walks the rows 2048 at a time with a running carry.
constexpr int kBuildRows = 2048;
__global__ __launch_bounds__(kThreads) void moon_dedup_build_kernel(BuildArgs a)
{
    constexpr int kPer = kBuildRows / kThreads;
    __shared__ int s_part[2][kThreads / kWave];
    __shared__ int s_carry[2];
    const int tid = threadIdx.x;
    const int lane = tid & (kWave - 1);
    const int wave = tid / kWave;
    const uint64_t *parent = a.t.parentTag + static_cast<int64_t>(a.rank) * a.t.stride;
    const uint32_t *sibling = a.t.sibling + static_cast<int64_t>(a.rank) * a.t.stride;
    uint64_t *groupStart = a.t.groupStart + static_cast<int64_t>(a.rank) * a.t.stride;
    if (tid == 0) {
        s_carry[0] = 0;
        s_carry[1] = 0;
    }
    __syncthreads();
    for (int64_t base = 0; base < a.nvS; base += kBuildRows) {
        int opens[kPer];
        int sizes[kPer];
        int primaries[kPer];
        int localOpen = 0;
        int localSize = 0;
#pragma unroll
        for (int i = 0; i < kPer; ++i) {
            const int64_t row = base + tid * kPer + i;
            opens[i] = 0;
            sizes[i] = 0;
            primaries[i] = -1;
            if (row < a.nvS) {
                const uint64_t p = parent[row];
                if (Tagged(p, a.epoch)) {
                    const uint32_t sib = sibling[row];
                    primaries[i] = static_cast<int>(p & 0xffffffffu) - 1;
                    opens[i] = (sib & 0xffffu) == 0 ? 1 : 0;
                    sizes[i] = opens[i] ? static_cast<int>(sib >> 16) : 0;
                }
            }
            localOpen += opens[i];
            localSize += sizes[i];
        }
        int inclOpen = localOpen;
        int inclSize = localSize;
#pragma unroll
        for (int off = 1; off < kWave; off <<= 1) {
            const int upOpen = __shfl_up(inclOpen, off);
            const int upSize = __shfl_up(inclSize, off);
            inclOpen += lane >= off ? upOpen : 0;
            inclSize += lane >= off ? upSize : 0;
        }
        if (lane == kWave - 1) {
            s_part[0][wave] = inclOpen;
            s_part[1][wave] = inclSize;
        }
        __syncthreads();
        int group = s_carry[0] + inclOpen - localOpen;
        int start = s_carry[1] + inclSize - localSize;
        int totalOpen = 0;
        int totalSize = 0;
#pragma unroll
        for (int w = 0; w < kThreads / kWave; ++w) {
            group += w < wave ? s_part[0][w] : 0;
            start += w < wave ? s_part[1][w] : 0;
            totalOpen += s_part[0][w];
            totalSize += s_part[1][w];
        }
#pragma unroll
        for (int i = 0; i < kPer; ++i) {
            if (opens[i]) {
                int32_t *g = a.dupGroups + static_cast<int64_t>(group) * 3;
                g[0] = primaries[i];
                g[1] = start;
                g[2] = sizes[i];
                __hip_atomic_store(&groupStart[primaries[i]], Tag(a.epoch, static_cast<uint32_t>(start)), __ATOMIC_RELAXED,
                    __HIP_MEMORY_SCOPE_AGENT);
                group += 1;
                start += sizes[i];
            }
        }
        __syncthreads();
        if (tid == 0) {
            s_carry[0] += totalOpen;
            s_carry[1] += totalSize;
        }
        __syncthreads();
    }
    if (tid == 0) {
        a.dupCounts[0] = s_carry[0];
        a.dupCounts[1] = s_carry[1];
    }
    // every group start is written: make the stores complete before any lane of this workgroup reads them back
    TileXREp::WaitOwnStores();
    __syncthreads();
    for (int64_t row = tid; row < a.nvS; row += kThreads) {
        const uint64_t p = parent[row];
        if (!Tagged(p, a.epoch)) {
            continue;
        }
        const int primary = static_cast<int>(p & 0xffffffffu) - 1;
        const uint64_t gs = __hip_atomic_load(&groupStart[primary], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        if (Tagged(gs, a.epoch)) {
            // a plan in which two duplicates of a token name the same row can claim more slots than there are rows
            const int64_t at = static_cast<int64_t>(gs & 0xffffffffu) + (sibling[row] & 0xffffu);
            if (at < a.nvS) {
                a.dupLoffs[at] = static_cast<int32_t>(row);
            } else {
                RecordFailure(a.t, a.rank, a.epoch, kDispatchInvalidRoute);
            }
        }
    }
}

// ---------------------------------------------------------------------------------------------------------------
// saved duplicate plan -> per-row records (dispatch: parentTag; combine: dupMask and groupOf)
// ---------------------------------------------------------------------------------------------------------------
struct WalkArgs {
    int64_t nvS;
    int rank;
    bool combine;
    const int32_t *dupGroups;
    const int32_t *dupLoffs;
    const int32_t *dupCounts;
    WorldTables t;
    uint64_t epoch;
};

// One thread per group.  Checks follow the reference (dispatch kernel :428-457, combine kernel :307-345).
__global__ __launch_bounds__(kThreads) void moon_group_walk_kernel(WalkArgs a)
{
    const int32_t groupCount = a.dupCounts[0];
    const int32_t duplicateCount = a.dupCounts[1];
    const int32_t invalid = a.combine ? kCombineInvalidRoute : kDispatchInvalidRoute;
    if (groupCount < 0 || groupCount > a.nvS || duplicateCount < 0 || duplicateCount > a.nvS) {
        if (blockIdx.x == 0 && threadIdx.x == 0) {
            RecordFailure(a.t, a.rank, a.epoch, invalid);
        }
        return;
    }
    const int64_t g = static_cast<int64_t>(blockIdx.x) * kThreads + threadIdx.x;
    if (g >= groupCount) {
        return;
    }
    const int32_t primary = a.dupGroups[g * 3];
    const int32_t start = a.dupGroups[g * 3 + 1];
    const int32_t count = a.dupGroups[g * 3 + 2];
    if (primary < 0 || primary >= a.nvS || start < 0 || count <= 0 || static_cast<int64_t>(start) + count > duplicateCount) {
        RecordFailure(a.t, a.rank, a.epoch, invalid);
        return;
    }
    const int64_t base = static_cast<int64_t>(a.rank) * a.t.stride;
    // nothing is recorded for a group with a bad entry: the reduce kernel follows these records without checking them
    for (int32_t i = 0; i < count; ++i) {
        const int32_t dup = a.dupLoffs[start + i];
        if (dup < 0 || dup >= a.nvS || (a.combine && dup == primary)) {
            RecordFailure(a.t, a.rank, a.epoch, invalid);
            return;
        }
    }
    if (a.combine) {
        a.t.groupOf[base + primary] = Tag(a.epoch, static_cast<uint32_t>(g) + 1u);
    }
    for (int32_t i = 0; i < count; ++i) {
        const int32_t dup = a.dupLoffs[start + i];
        if (a.combine) {
            a.t.dupMask[base + dup] = Tag(a.epoch, 1u);
        } else {
            a.t.parentTag[base + dup] = Tag(a.epoch, static_cast<uint32_t>(primary) + 1u);
        }
    }
}

// ---------------------------------------------------------------------------------------------------------------
// dispatch: rows nobody wrote
// ---------------------------------------------------------------------------------------------------------------
struct FillArgs {
    int64_t nvS;
    int h;
    int world;
    int rank;
    bool expand;
    void *hiddenNvsh;
    float *weightsNvs;
    WorldTables t;
    uint64_t epoch;
    int32_t *status;
};

// Work item of the fill kernel: row | kind << 30.
constexpr int32_t kFillZero = 0;
constexpr int32_t kFillCopy = 1;

// One thread per row decides what is left to do for it: nothing (a route wrote it), zeros (no route wrote it: the
// reference clears the whole window first, dispatch kernel :206-230), or -- saved plans -- a copy of its primary row
// (dispatch kernel :426-461).  The weight of a row no route names is zero for the same reason.  Each workgroup packs its rows' work items into its own segment of the work list, so
// nothing has to be reset between calls.  Workgroup 0 also writes the device status.
__global__ __launch_bounds__(kRowsPerGroup) void moon_classify_kernel(FillArgs a)
{
    __shared__ int s_waveCount[kRowsPerGroup / kWave];
    const int tid = threadIdx.x;
    const int lane = tid & (kWave - 1);
    const int wave = tid / kWave;
    const int64_t base = static_cast<int64_t>(a.rank) * a.t.stride;
    const int64_t row = static_cast<int64_t>(blockIdx.x) * kRowsPerGroup + tid;
    int32_t item = -1;
    if (row < a.nvS) {
        const uint64_t tag = a.t.rowTag[base + row];
        const bool named = Tagged(tag, a.epoch) && (tag & kRowNamed) != 0;
        const bool written = Tagged(tag, a.epoch) && (tag & kRowWritten) != 0;
        const uint64_t p = a.t.parentTag[base + row];
        if (a.expand && Tagged(p, a.epoch)) {
            item = static_cast<int32_t>(row) | (kFillCopy << 30);
        } else if (!written) {
            item = static_cast<int32_t>(row) | (kFillZero << 30);
        }
        if (!named && a.weightsNvs != nullptr) {
            a.weightsNvs[row] = 0.0f;
        }
    }
    const uint64_t have = __ballot(item >= 0);
    if (lane == 0) {
        s_waveCount[wave] = __popcll(have);
    }
    __syncthreads();
    int before = 0;
    int total = 0;
#pragma unroll
    for (int w = 0; w < kRowsPerGroup / kWave; ++w) {
        before += w < wave ? s_waveCount[w] : 0;
        total += s_waveCount[w];
    }
    if (item >= 0) {
        const int at = before + __popcll(have & ((1ull << lane) - 1ull));
        a.t.workList[base + static_cast<int64_t>(blockIdx.x) * kRowsPerGroup + at] = item;
    }
    if (tid == 0) {
        a.t.workCount[static_cast<int64_t>(a.rank) * a.t.groupStride + blockIdx.x] = total;
    }
    if (blockIdx.x == 0 && tid == 0) {
        // own failure first, then the first failed peer walking upwards from this rank (dispatch kernel :559-574)
        int32_t status = kDispatchOk;
        const uint64_t own = __hip_atomic_load(&a.t.fail[a.rank], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        if (Tagged(own, a.epoch)) {
            status = static_cast<int32_t>(own & 0xffffffffu);
        } else {
            for (int o = 1; o < a.world; ++o) {
                const int peer = (a.rank + o) % a.world;
                const uint64_t f = __hip_atomic_load(&a.t.fail[peer], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                if (Tagged(f, a.epoch)) {
                    status = kDispatchRemoteFailureBase + peer;
                    break;
                }
            }
        }
        a.status[0] = status;
    }
}

// kFillSplit workgroups share the work items of one classify group; a workgroup writes whole rows.
template <bool VEC>
__global__ __launch_bounds__(kThreads) void moon_fill_kernel(FillArgs a)
{
    const int group = blockIdx.x / kFillSplit;
    const int part = blockIdx.x % kFillSplit;
    const int64_t base = static_cast<int64_t>(a.rank) * a.t.stride;
    const int count = a.t.workCount[static_cast<int64_t>(a.rank) * a.t.groupStride + group];
    const int32_t *items = a.t.workList + base + static_cast<int64_t>(group) * kRowsPerGroup;
    const int lane = threadIdx.x;
    for (int i = part; i < count; i += kFillSplit) {
        const int32_t item = items[i];
        const int row = item & 0x3fffffff;
        bool copy = (item >> 30) == kFillCopy;
        int primary = 0;
        if (copy) {
            primary = static_cast<int>(a.t.parentTag[base + row] & 0xffffffffu) - 1;
            // a primary no route wrote is all zeros in the reference too (the window was cleared)
            const uint64_t tag = a.t.rowTag[base + primary];
            copy = Tagged(tag, a.epoch) && (tag & kRowWritten) != 0;
        }
        if (VEC) {
            const int vecs = a.h / 8;
            u32x4 *dstRow = reinterpret_cast<u32x4 *>(static_cast<char *>(a.hiddenNvsh) + static_cast<int64_t>(row) * a.h * 2);
            const u32x4 *srcRow = reinterpret_cast<const u32x4 *>(static_cast<const char *>(a.hiddenNvsh) +
                static_cast<int64_t>(primary) * a.h * 2);
            for (int idx = lane; idx < vecs; idx += kThreads) {
                const u32x4 v = copy ? srcRow[idx] : u32x4{0u, 0u, 0u, 0u};
                __builtin_nontemporal_store(v, dstRow + idx);
            }
        } else {
            uint16_t *dstRow = static_cast<uint16_t *>(a.hiddenNvsh) + static_cast<int64_t>(row) * a.h;
            const uint16_t *srcRow = static_cast<const uint16_t *>(a.hiddenNvsh) + static_cast<int64_t>(primary) * a.h;
            for (int c = lane; c < a.h; c += kThreads) {
                dstRow[c] = copy ? srcRow[c] : static_cast<uint16_t>(0);
            }
        }
    }
}

// ---------------------------------------------------------------------------------------------------------------
// combine: reverse routes -> slot table of the origin ranks
// ---------------------------------------------------------------------------------------------------------------
struct ReverseArgs {
    const int32_t *dstLocal;
    int64_t nvS, n;
    int world;
    int rank;
    WorldTables t;
    uint64_t epoch;
};

// reference: combine kernel :285-298 (decode), :350-366 (validation), :568-606 (which rows travel)
__global__ __launch_bounds__(kThreads) void moon_reverse_kernel(ReverseArgs a)
{
    const int64_t row = static_cast<int64_t>(blockIdx.x) * kThreads + threadIdx.x;
    if (row >= a.nvS) {
        return;
    }
    const int32_t encoded = a.dstLocal[row];
    if (encoded == -1) {
        return;
    }
    const int64_t peer = encoded / a.nvS;
    const int64_t target = encoded % a.nvS;
    if (encoded < 0 || peer >= a.world || target >= a.n) {
        RecordFailure(a.t, a.rank, a.epoch, kCombineInvalidRoute);
        return;
    }
    const int64_t base = static_cast<int64_t>(a.rank) * a.t.stride;
    const uint32_t duplicate = Tagged(a.t.dupMask[base + row], a.epoch) ? 0x80000000u : 0u;
    a.t.slotSrc[peer * a.t.stride + target] = Tag(a.epoch, duplicate | static_cast<uint32_t>(a.rank * a.nvS + row));
}

// ---------------------------------------------------------------------------------------------------------------
// combine: reduce
// ---------------------------------------------------------------------------------------------------------------
struct ReduceArgs {
    int s, k, h;
    int64_t nvS;
    int world;
    int rank;
    int colSlices;
    SourceTable src;
    WorldTables t;
    uint64_t epoch;
    void *hiddenSh;
    float *weightsSk;
    int32_t *status;
};

__device__ __forceinline__ void AddRow(float (&acc)[kRowVecs][8], const u32x4 (&v)[kRowVecs])
{
#pragma unroll
    for (int j = 0; j < kRowVecs; ++j) {
#pragma unroll
        for (int q = 0; q < 4; ++q) {
            acc[j][2 * q] = __fadd_rn(acc[j][2 * q], __uint_as_float(v[j][q] << 16));
            acc[j][2 * q + 1] = __fadd_rn(acc[j][2 * q + 1], __uint_as_float(v[j][q] & 0xffff0000u));
        }
    }
}

template <bool VEC>
struct RowReader;

// 16-byte vectors, two per lane; a unit is one slice of G * kRowVecs vectors of one token.
template <>
struct RowReader<true> {
    __device__ static __forceinline__ void Load(const void *tensor, int64_t row, int h, int colBase, int lane, int lanes,
        u32x4 (&v)[kRowVecs])
    {
        const u32x4 *p = reinterpret_cast<const u32x4 *>(static_cast<const char *>(tensor) + row * h * 2);
        const int vecs = h / 8;
#pragma unroll
        for (int j = 0; j < kRowVecs; ++j) {
            const int idx = colBase + j * lanes + lane;
            v[j] = idx < vecs ? __builtin_nontemporal_load(p + idx) : u32x4{0u, 0u, 0u, 0u};
        }
    }
};

// Slot sum of one token slice.  Slots are taken in slot order from zero (combine kernel :664-699); a slot that holds a
// primary with duplicates contributes bf16(fp32(primary) + fp32(dup) + ...) in the plan's list order (combine kernel
// :489-530); duplicate rows and slots nothing was returned to contribute nothing (their receive row stays zero).
template <int G>
__global__ __launch_bounds__(G) void moon_reduce_kernel(ReduceArgs a)
{
    __shared__ uint64_t s_slot[kMaxTopK];
    const int xcdUnits = a.s * a.colSlices;
    const int unit = blockIdx.x;
    if (unit >= xcdUnits) {
        return;
    }
    const int token = unit / a.colSlices;
    const int colBase = (unit % a.colSlices) * (G * kRowVecs);
    const int lane = threadIdx.x;
    const int vecs = a.h / 8;
    const uint64_t *slots = a.t.slotSrc + static_cast<int64_t>(a.rank) * a.t.stride + static_cast<int64_t>(token) * a.k;
    if (lane < a.k) {
        const uint64_t w = slots[lane];
        s_slot[lane] = w;
        if (colBase == 0 && a.weightsSk != nullptr) {
            float weight = 0.0f;
            if (Tagged(w, a.epoch)) {
                const uint32_t where = static_cast<uint32_t>(w) & 0x7fffffffu;
                weight = a.src.weights[where / a.nvS][where % a.nvS];
            }
            a.weightsSk[static_cast<int64_t>(token) * a.k + lane] = weight;
        }
    }
    if (G > kWave) {
        __syncthreads();
    }
    float acc[kRowVecs][8];
#pragma unroll
    for (int j = 0; j < kRowVecs; ++j) {
#pragma unroll
        for (int e = 0; e < 8; ++e) {
            acc[j][e] = 0.0f;
        }
    }
    for (int k = 0; k < a.k; ++k) {
        const uint64_t w = s_slot[k];
        const uint32_t low = static_cast<uint32_t>(w);
        if (!Tagged(w, a.epoch) || (low & 0x80000000u) != 0u) {
            continue;
        }
        const int q = static_cast<int>(low / a.nvS);
        const int64_t row = low % a.nvS;
        u32x4 v[kRowVecs];
        RowReader<true>::Load(a.src.hidden[q], row, a.h, colBase, lane, G, v);
        const uint64_t gw = a.t.groupOf[static_cast<int64_t>(q) * a.t.stride + row];
        if (!Tagged(gw, a.epoch)) {
            AddRow(acc, v);
            continue;
        }
        const int64_t g = static_cast<int64_t>(gw & 0xffffffffu) - 1;
        const int32_t start = a.src.dupGroups[q][g * 3 + 1];
        const int32_t count = a.src.dupGroups[q][g * 3 + 2];
        float sub[kRowVecs][8];
#pragma unroll
        for (int j = 0; j < kRowVecs; ++j) {
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                sub[j][2 * e] = __uint_as_float(v[j][e] << 16);
                sub[j][2 * e + 1] = __uint_as_float(v[j][e] & 0xffff0000u);
            }
        }
        constexpr int kBatch = 4;
        for (int i0 = 0; i0 < count; i0 += kBatch) {
            u32x4 d[kBatch][kRowVecs];
#pragma unroll
            for (int u = 0; u < kBatch; ++u) {
                if (i0 + u < count) {
                    RowReader<true>::Load(a.src.hidden[q], a.src.dupLoffs[q][start + i0 + u], a.h, colBase, lane, G, d[u]);
                }
            }
#pragma unroll
            for (int u = 0; u < kBatch; ++u) {
                if (i0 + u < count) {
                    AddRow(sub, d[u]);
                }
            }
        }
#pragma unroll
        for (int j = 0; j < kRowVecs; ++j) {
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                const uint32_t packed = TileXREp::FloatPairToBf16Rne(sub[j][2 * e], sub[j][2 * e + 1]);
                acc[j][2 * e] = __fadd_rn(acc[j][2 * e], __uint_as_float(packed << 16));
                acc[j][2 * e + 1] = __fadd_rn(acc[j][2 * e + 1], __uint_as_float(packed & 0xffff0000u));
            }
        }
    }
    u32x4 *out = reinterpret_cast<u32x4 *>(static_cast<char *>(a.hiddenSh) + static_cast<int64_t>(token) * a.h * 2);
#pragma unroll
    for (int j = 0; j < kRowVecs; ++j) {
        const int idx = colBase + j * G + lane;
        if (idx < vecs) {
            u32x4 o;
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                o[e] = TileXREp::FloatPairToBf16Rne(acc[j][2 * e], acc[j][2 * e + 1]);
            }
            __builtin_nontemporal_store(o, out + idx);
        }
    }
}

// Any hidden size and alignment: one workgroup per token, one element per thread step.
__global__ __launch_bounds__(kThreads) void moon_reduce_generic_kernel(ReduceArgs a)
{
    __shared__ uint64_t s_slot[kMaxTopK];
    const int token = blockIdx.x;
    const int lane = threadIdx.x;
    const uint64_t *slots = a.t.slotSrc + static_cast<int64_t>(a.rank) * a.t.stride + static_cast<int64_t>(token) * a.k;
    if (lane < a.k) {
        const uint64_t w = slots[lane];
        s_slot[lane] = w;
        if (a.weightsSk != nullptr) {
            float weight = 0.0f;
            if (Tagged(w, a.epoch)) {
                const uint32_t where = static_cast<uint32_t>(w) & 0x7fffffffu;
                weight = a.src.weights[where / a.nvS][where % a.nvS];
            }
            a.weightsSk[static_cast<int64_t>(token) * a.k + lane] = weight;
        }
    }
    __syncthreads();
    for (int c = lane; c < a.h; c += kThreads) {
        float acc = 0.0f;
        for (int k = 0; k < a.k; ++k) {
            const uint64_t w = s_slot[k];
            const uint32_t low = static_cast<uint32_t>(w);
            if (!Tagged(w, a.epoch) || (low & 0x80000000u) != 0u) {
                continue;
            }
            const int q = static_cast<int>(low / a.nvS);
            const int64_t row = low % a.nvS;
            const uint16_t *tensor = static_cast<const uint16_t *>(a.src.hidden[q]);
            float value = __uint_as_float(static_cast<uint32_t>(tensor[row * a.h + c]) << 16);
            const uint64_t gw = a.t.groupOf[static_cast<int64_t>(q) * a.t.stride + row];
            if (Tagged(gw, a.epoch)) {
                const int64_t g = static_cast<int64_t>(gw & 0xffffffffu) - 1;
                const int32_t start = a.src.dupGroups[q][g * 3 + 1];
                const int32_t count = a.src.dupGroups[q][g * 3 + 2];
                for (int32_t i = 0; i < count; ++i) {
                    const int64_t dup = a.src.dupLoffs[q][start + i];
                    value = __fadd_rn(value, __uint_as_float(static_cast<uint32_t>(tensor[dup * a.h + c]) << 16));
                }
                value = __uint_as_float(TileXREp::FloatToBf16Rne(value) << 16);
            }
            acc = __fadd_rn(acc, value);
        }
        static_cast<uint16_t *>(a.hiddenSh)[static_cast<int64_t>(token) * a.h + c] =
            static_cast<uint16_t>(TileXREp::FloatToBf16Rne(acc));
    }
}

// Device status of combine: own failure, else the first failed peer in rank order (combine kernel :391-411), else 0.
__global__ void moon_combine_status_kernel(WorldTables t, int world, int rank, uint64_t epoch, int32_t *status)
{
    int32_t value = kCombineOk;
    const uint64_t own = __hip_atomic_load(&t.fail[rank], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    if (Tagged(own, epoch)) {
        value = static_cast<int32_t>(own & 0xffffffffu);
    } else {
        for (int peer = 0; peer < world; ++peer) {
            const uint64_t f = __hip_atomic_load(&t.fail[peer], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            if (Tagged(f, epoch)) {
                value = kCombineRemoteFailureBase + peer;
                break;
            }
        }
    }
    status[0] = value;
}

bool VectorRows(int64_t h, const void *a, const void *b)
{
    return h % 8 == 0 && TileXREp::Aligned16(a) && TileXREp::Aligned16(b);
}

} // namespace

const char *MoonScatterKernelName()
{
    return gScatterName;
}

const char *MoonReduceKernelName()
{
    return gReduceName;
}

hipError_t LaunchMoonScatter(const ScatterLaunch &l)
{
    ScatterArgs a {};
    a.dst = l.dst;
    a.hiddenSh = l.hiddenSh;
    a.weightsSk = l.weightsSk;
    a.s = static_cast<int>(l.s);
    a.k = static_cast<int>(l.k);
    a.h = static_cast<int>(l.h);
    a.nvS = l.nvS;
    a.world = l.world;
    a.srcRank = l.srcRank;
    a.out = l.out;
    a.t = l.tables;
    a.epoch = l.epoch;
    bool vec = l.h % 8 == 0 && TileXREp::Aligned16(l.hiddenSh);
    for (int r = 0; r < l.world; ++r) {
        vec = vec && TileXREp::Aligned16(l.out.hidden[r]);
    }
    const int64_t vecs = l.h / 8;
    a.colSlices = static_cast<int>((vecs + kRowVecs * kThreads - 1) / (kRowVecs * kThreads));
    const int64_t blocks = (l.s + kXcds - 1) / kXcds * kXcds * l.k * a.colSlices;
    if (vec && blocks <= 0x7fffffff) {
        gScatterName = "moon_scatter_kernel";
        if (l.fresh) {
            hipLaunchKernelGGL(moon_scatter_kernel<true>, dim3(static_cast<unsigned>(blocks)), dim3(kThreads), 0, l.stream, a);
        } else {
            hipLaunchKernelGGL(moon_scatter_kernel<false>, dim3(static_cast<unsigned>(blocks)), dim3(kThreads), 0, l.stream, a);
        }
    } else {
        gScatterName = "moon_scatter_generic_kernel";
        const unsigned grid = static_cast<unsigned>(l.s * l.k);
        if (l.fresh) {
            hipLaunchKernelGGL(moon_scatter_generic_kernel<true>, dim3(grid), dim3(kThreads), 0, l.stream, a);
        } else {
            hipLaunchKernelGGL(moon_scatter_generic_kernel<false>, dim3(grid), dim3(kThreads), 0, l.stream, a);
        }
    }
    return hipGetLastError();
}

hipError_t LaunchMoonDedupBuild(const DedupBuildLaunch &l)
{
    BuildArgs a {};
    a.nvS = l.nvS;
    a.rank = l.rank;
    a.t = l.tables;
    a.epoch = l.epoch;
    a.dupGroups = l.dupGroups;
    a.dupLoffs = l.dupLoffs;
    a.dupCounts = l.dupCounts;
    hipLaunchKernelGGL(moon_dedup_build_kernel, dim3(1), dim3(kThreads), 0, l.stream, a);
    return hipGetLastError();
}

hipError_t LaunchMoonGroupWalk(const GroupWalkLaunch &l)
{
    WalkArgs a {};
    a.nvS = l.nvS;
    a.rank = l.rank;
    a.combine = l.combine;
    a.dupGroups = l.dupGroups;
    a.dupLoffs = l.dupLoffs;
    a.dupCounts = l.dupCounts;
    a.t = l.tables;
    a.epoch = l.epoch;
    const unsigned grid = static_cast<unsigned>((l.nvS + kThreads - 1) / kThreads);
    hipLaunchKernelGGL(moon_group_walk_kernel, dim3(grid), dim3(kThreads), 0, l.stream, a);
    return hipGetLastError();
}

hipError_t LaunchMoonFill(const FillLaunch &l)
{
    FillArgs a {};
    a.nvS = l.nvS;
    a.h = static_cast<int>(l.h);
    a.world = l.world;
    a.rank = l.rank;
    a.expand = l.expand;
    a.hiddenNvsh = l.hiddenNvsh;
    a.weightsNvs = l.weightsNvs;
    a.t = l.tables;
    a.epoch = l.epoch;
    a.status = l.status;
    const unsigned groups = static_cast<unsigned>((l.nvS + kRowsPerGroup - 1) / kRowsPerGroup);
    hipLaunchKernelGGL(moon_classify_kernel, dim3(groups), dim3(kRowsPerGroup), 0, l.stream, a);
    hipError_t err = hipGetLastError();
    if (err != hipSuccess) {
        return err;
    }
    if (VectorRows(l.h, l.hiddenNvsh, l.hiddenNvsh)) {
        hipLaunchKernelGGL(moon_fill_kernel<true>, dim3(groups * kFillSplit), dim3(kThreads), 0, l.stream, a);
    } else {
        hipLaunchKernelGGL(moon_fill_kernel<false>, dim3(groups * kFillSplit), dim3(kThreads), 0, l.stream, a);
    }
    return hipGetLastError();
}

hipError_t LaunchMoonReverse(const ReverseLaunch &l)
{
    ReverseArgs a {};
    a.dstLocal = l.dstLocal;
    a.nvS = l.nvS;
    a.n = l.n;
    a.world = l.world;
    a.rank = l.rank;
    a.t = l.tables;
    a.epoch = l.epoch;
    const unsigned grid = static_cast<unsigned>((l.nvS + kThreads - 1) / kThreads);
    hipLaunchKernelGGL(moon_reverse_kernel, dim3(grid), dim3(kThreads), 0, l.stream, a);
    return hipGetLastError();
}

hipError_t LaunchMoonReduce(const MoonReduceLaunch &l)
{
    ReduceArgs a {};
    a.s = static_cast<int>(l.s);
    a.k = static_cast<int>(l.k);
    a.h = static_cast<int>(l.h);
    a.nvS = l.nvS;
    a.world = l.world;
    a.rank = l.rank;
    a.src = l.src;
    a.t = l.tables;
    a.epoch = l.epoch;
    a.hiddenSh = l.hiddenSh;
    a.weightsSk = l.weightsSk;
    a.status = l.status;
    bool vec = l.h % 8 == 0 && TileXREp::Aligned16(l.hiddenSh);
    for (int r = 0; r < l.world; ++r) {
        vec = vec && TileXREp::Aligned16(l.src.hidden[r]);
    }
    const int64_t vecs = l.h / 8;
    constexpr int G = kWave;
    a.colSlices = static_cast<int>((vecs + G * kRowVecs - 1) / (G * kRowVecs));
    const int64_t units = l.s * a.colSlices;
    if (vec && units <= 0x7fffffff) {
        gReduceName = "moon_reduce_kernel";
        hipLaunchKernelGGL(moon_reduce_kernel<G>, dim3(static_cast<unsigned>(units)), dim3(G), 0, l.stream, a);
    } else {
        gReduceName = "moon_reduce_generic_kernel";
        hipLaunchKernelGGL(moon_reduce_generic_kernel, dim3(static_cast<unsigned>(l.s)), dim3(kThreads), 0, l.stream, a);
    }
    hipError_t err = hipGetLastError();
    if (err != hipSuccess) {
        return err;
    }
    hipLaunchKernelGGL(moon_combine_status_kernel, dim3(1), dim3(1), 0, l.stream, l.tables, l.world, l.rank, l.epoch, l.status);
    return hipGetLastError();
}

} // namespace TileXRMoon
