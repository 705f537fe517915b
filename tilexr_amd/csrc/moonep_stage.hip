// Plan-driven (MoonEP) dispatch / combine kernels for ranks that share one MI355X (gfx950, wave64).
//
// HBM-bound row movement, no MFMA.  A plan names the destination row of every route directly, so there is nothing to
// count: dispatch is one read of each token row and one write per route; combine is one read per route and one write
// per token.  Row copies use two 16-byte loads and two 16-byte stores per lane, and the workgroups of one token are
// given block indices that land on one XCD (block b runs on XCD b % 8) so the token row is read from HBM once.
// Every kernel is launched once for the whole world: blockIdx.y is the rank whose share the workgroup works on.
//
//   what is computed  reference: src/moonep/dispatch/kernels/tilexr_moonep_dispatch_kernel.cpp:108-147, 268-461
//                                src/moonep/combine/kernels/tilexr_moonep_combine_kernel.cpp:117-177, 285-366, 449-541,
//                                568-606, 648-733
#include <atomic>

#include <hip/hip_runtime.h>

#include "ep_kernel_common.hip.h"
#include "ep_numerics.hip.h"
#include "moonep_stage.h"

namespace TileXRMoon {
namespace {

using TileXREp::u32x4;
using TileXREp::kThreads;
using TileXREp::kWave;

constexpr int kXcds = 8;
constexpr int kRowVecs = 2;     // 16-byte vectors per lane per row slice

std::atomic<int64_t> gCachedRowBytes {int64_t{256} << 20};     // TileXRMoonEpSetCachedRowBytes
constexpr int kFusedPlanChunks = 1024;  // chunks of 2048 rows per rank up to which the scatter launch builds a fresh plan
constexpr int64_t kFusedPlanRowBytes = int64_t{256} << 20;     // ... and bytes of rows the world's routes write
constexpr int kSelfPlanChunks = 8;      // ... and up to which its plan workgroups add up the earlier chunks themselves
constexpr int64_t kWarmRowBytes = int64_t{128} << 20;          // token rows of a world that are read ahead of the per-route scatter

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

// Row tag bits.
constexpr uint32_t kRowWritten = 1u;    // a route wrote the row's hidden values
constexpr uint32_t kRowNamed = 2u;      // a route names the row: its weight is written
constexpr uint32_t kRowDirect = 4u;     // saved plan: a duplicate whose primary is a row of the same token, written by
                                        // the source like a fresh duplicate

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

// Row of the first non-duplicate route of the token, before route k, that goes to `peer`; -1 when there is none.
// reference: dispatch kernel :281-301
__device__ __forceinline__ int OwnPrimaryRow(const DispatchWorld &a, const int32_t *words, int k, int peer)
{
    for (int j = 0; j < k; ++j) {
        const int32_t e = words[j];
        if (e < 0) {
            continue;
        }
        const Route o = Decode(e, a.nvS, a.world);
        if (o.ok && o.peer == peer) {
            return o.row;
        }
    }
    return -1;
}

// What the route's first workgroup records besides the row: the weight, the row tag and -- while the duplicate plan is
// being built -- which primary a duplicate belongs to and where it stands among that primary's duplicates.  Called by
// the first wave of the workgroup, all 64 lanes; s_dst holds the token's K route words.
//   primary of a duplicate = first earlier non-duplicate route of the token to the same rank (dispatch kernel :281-301)
//   the plan lists a primary's duplicates in ascending row order (dispatch kernel :393-419), so the rank of a
//   duplicate within its group is the number of the token's duplicates to that rank with a smaller row
template <bool FRESH>
__device__ __forceinline__ void RouteRecords(const DispatchWorld &a, int src, int token, int k, const Route &r, uint32_t tagBits,
    const int32_t *s_dst)
{
    const int lane = threadIdx.x;
    const int64_t at = static_cast<int64_t>(r.peer) * a.tables.stride + r.row;
    if (lane == 0) {
        if (a.weightsSk[src] != nullptr) {
            a.weightsNvs[r.peer][r.row] = a.weightsSk[src][static_cast<int64_t>(token) * a.k + k];
        }
        a.tables.rowTag[at] = Tag(a.epoch, tagBits);
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
            RecordFailure(a.tables, src, a.epoch, kDispatchInvalidRoute);
        }
        return;
    }
    const int primaryLane = __ffsll(static_cast<unsigned long long>(primaries)) - 1;
    const int primaryRow = __shfl(other.row, primaryLane);
    if (lane == 0) {
        a.tables.parentTag[at] = Tag(a.epoch, static_cast<uint32_t>(primaryRow) + 1u);
        a.tables.sibling[at] = static_cast<uint32_t>(__popcll(before)) | (static_cast<uint32_t>(__popcll(siblings)) << 16);
    }
}

// Whether the source writes the row of this route, and the tag the row gets.
//   fresh plan   every route: the plan is being built from these very route words, so a duplicate row is by construction
//                a copy of this token's row
//   saved plan   non-duplicates; and a duplicate whose primary, according to the plan (parent records written by the walk
//                kernel), is the row this token's own non-duplicate route to that rank writes -- the copy the finish
//                kernel would make is a copy of this token's row (`direct`, worked out by the agree kernel).  Any other
//                duplicate is left to the finish kernel.
template <bool FRESH>
__device__ __forceinline__ bool SourceWrites(const Route &r, uint8_t direct, uint32_t *tagBits)
{
    if (FRESH || !r.duplicate) {
        *tagBits = kRowNamed | kRowWritten;
        return true;
    }
    if (direct != 0) {
        *tagBits = kRowNamed | kRowWritten | kRowDirect;
        return true;
    }
    *tagBits = kRowNamed;
    return false;
}

// Reads 8 KiB of the token rows of source rank blockIdx.y (two 16-byte loads per lane) and drops them, ahead of the
// per-route scatter.  That kernel is the fastest copy only while the token rows are in the memory-side cache: when its
// one reading workgroup in K has to fetch a row from HBM between the writes of the others it runs at little more than
// half its speed.  After this read it finds the rows in that cache whatever their history.
constexpr int kWarmLoads = 2;
__device__ __forceinline__ void WarmRows(const DispatchWorld &a, int rank, int64_t block, int64_t vecs)
{
    const u32x4 *rows = static_cast<const u32x4 *>(a.hiddenSh[rank]);
    const int64_t base = block * (kThreads * kWarmLoads) + threadIdx.x;
    u32x4 v[kWarmLoads];
#pragma unroll
    for (int i = 0; i < kWarmLoads; ++i) {
        const int64_t at = base + static_cast<int64_t>(i) * kThreads;
        v[i] = rows[at < vecs ? at : vecs - 1];
    }
#pragma unroll
    for (int i = 0; i < kWarmLoads; ++i) {
        asm volatile("" ::"v"(v[i]));
    }
}

// Saved plans, one thread per route of source rank blockIdx.y: whether the source may write a duplicate's row itself
// (see SourceWrites).  Done ahead of the scatter so that its workgroups find the answer with the route word, in one
// round trip, instead of looking up the parent record after decoding it.  The workgroups from `routeBlocks` on read the
// token rows ahead (WarmRows) when warmVecs is not zero: this launch waits on a few small loads and leaves the memory
// system idle, so the read costs a saved-plan Dispatch no launch of its own.
__global__ __launch_bounds__(kThreads) void moon_agree_kernel(DispatchWorld a, unsigned routeBlocks, int64_t warmVecs)
{
    if (blockIdx.x >= routeBlocks) {
        WarmRows(a, blockIdx.y, static_cast<int64_t>(blockIdx.x - routeBlocks), warmVecs);
        return;
    }
    const int src = blockIdx.y;
    const int64_t route = static_cast<int64_t>(blockIdx.x) * kThreads + threadIdx.x;
    if (route >= a.s * a.k) {
        return;
    }
    const int K = static_cast<int>(a.k);
    const int k = static_cast<int>(route % K);
    const int32_t *words = a.dst[src] + route - k;
    uint8_t direct = 0;
    const Route r = Decode(words[k], a.nvS, a.world);
    if (r.ok && r.duplicate) {
        const uint64_t p = a.tables.parentTag[static_cast<int64_t>(r.peer) * a.tables.stride + r.row];
        direct = Tagged(p, a.epoch) && static_cast<int>(p & 0xffffffffu) - 1 == OwnPrimaryRow(a, words, k, r.peer) ? 1 : 0;
    }
    a.tables.direct[static_cast<int64_t>(src) * a.tables.stride + route] = direct;
}

// The same read as a launch of its own, for a Dispatch that builds its plan: nothing runs ahead of its scatter.
__global__ __launch_bounds__(kThreads) void moon_warm_rows_kernel(DispatchWorld a, int64_t vecs)
{
    WarmRows(a, blockIdx.y, static_cast<int64_t>(blockIdx.x), vecs);
}

// Fresh plans, one thread per route of source rank blockIdx.y: everything a route records (RouteRecords) and the
// failure of a route that names no rank, ahead of the scatter.  Nothing the plan is built from is then written by the
// scatter launch, so extra workgroups of that launch build it (moon_scatter_kernel, PLAN) instead of launches after it.
// The workgroups from `routeBlocks` on read the token rows ahead, as in moon_agree_kernel.
__global__ __launch_bounds__(kThreads) void moon_records_kernel(DispatchWorld a, unsigned routeBlocks, int64_t warmVecs)
{
    if (blockIdx.x >= routeBlocks) {
        WarmRows(a, blockIdx.y, static_cast<int64_t>(blockIdx.x - routeBlocks), warmVecs);
        return;
    }
    const int src = blockIdx.y;
    const int64_t route = static_cast<int64_t>(blockIdx.x) * kThreads + threadIdx.x;
    if (route >= a.s * a.k) {
        return;
    }
    const int K = static_cast<int>(a.k);
    const int k = static_cast<int>(route % K);
    const int32_t *words = a.dst[src] + route - k;
    const float weight = a.weightsSk[src] != nullptr ? a.weightsSk[src][route] : 0.0f;
    const Route r = Decode(words[k], a.nvS, a.world);
    if (!r.ok) {
        RecordFailure(a.tables, src, a.epoch, kDispatchInvalidRoute);
        return;
    }
    const int64_t at = static_cast<int64_t>(r.peer) * a.tables.stride + r.row;
    if (a.weightsSk[src] != nullptr) {
        a.weightsNvs[r.peer][r.row] = weight;
    }
    a.tables.rowTag[at] = Tag(a.epoch, kRowNamed | kRowWritten);
    if (!r.duplicate) {
        return;
    }
    // the token's other routes to the same rank: the first non-duplicate before this one is the primary, the duplicates
    // with a smaller row stand before this one in the primary's group (RouteRecords, one lane per route there)
    int primaryRow = -1;
    uint32_t siblings = 0;
    uint32_t before = 0;
    for (int j = 0; j < K; ++j) {
        const Route o = Decode(words[j], a.nvS, a.world);
        if (!o.ok || o.peer != r.peer) {
            continue;
        }
        if (!o.duplicate) {
            primaryRow = (primaryRow < 0 && j < k) ? o.row : primaryRow;
        } else {
            siblings += 1u;
            before += o.row < r.row ? 1u : 0u;
        }
    }
    if (primaryRow < 0) {
        RecordFailure(a.tables, src, a.epoch, kDispatchInvalidRoute);
        return;
    }
    a.tables.parentTag[at] = Tag(a.epoch, static_cast<uint32_t>(primaryRow) + 1u);
    a.tables.sibling[at] = before | (siblings << 16);
}

// defined with the kernels that build the duplicate plan, below
template <bool SELF>
__device__ __forceinline__ void DedupGroupsOfChunk(const DispatchWorld &a, int rank, int chunk, bool lastChunk,
    int (*s_part)[kThreads / kWave], int *s_base);

// One workgroup per (token, route, slice of 512 vectors) of source rank blockIdx.y.
//
// PLAN: a fresh plan whose records were written ahead (moon_records_kernel) is built here as well: the first `planBlocks` workgroups
// of the launch (a multiple of eight, so that the rest keep their XCDs) take one chunk of destination rank blockIdx.y
// each.  They depend on nothing this launch writes and are done long before the rows are.  The totals of the chunks
// before its own a workgroup adds up itself while the chunks are few (planSelf), a trip to memory per chunk, and those
// trips are slow beside the scatter's traffic (measured: 5 us each; 32 chunks took longer than the rows); otherwise a
// launch of moon_dedup_totals_kernel ahead of this one has left them.
template <bool FRESH, bool PLAN>
__global__ __launch_bounds__(kThreads) void moon_scatter_kernel(DispatchWorld a, int colSlices, unsigned planBlocks, int planChunks,
    int planSelf)
{
    static_assert(FRESH || !PLAN, "only a Dispatch that builds its plan has plan workgroups");
    __shared__ int32_t s_dst[kMaxTopK];
    if (PLAN && blockIdx.x < planBlocks) {
        __shared__ int s_part[2][kThreads / kWave];
        __shared__ int s_base[2];
        const int chunk = blockIdx.x;
        if (chunk < planChunks && planSelf != 0) {
            DedupGroupsOfChunk<true>(a, blockIdx.y, chunk, chunk == planChunks - 1, s_part, s_base);
        } else if (chunk < planChunks) {
            DedupGroupsOfChunk<false>(a, blockIdx.y, chunk, chunk == planChunks - 1, s_part, s_base);
        }
        return;
    }
    const unsigned block = blockIdx.x - (PLAN ? planBlocks : 0u);
    const int src = blockIdx.y;
    const int xcd = block % kXcds;
    const int j = block / kXcds;
    const int K = static_cast<int>(a.k);
    const int perToken = K * colSlices;
    const int token = (j / perToken) * kXcds + xcd;
    const int k = (j % perToken) / colSlices;
    const int slice = (j % perToken) % colSlices;
    if (token >= a.s) {
        return;
    }
    const int lane = threadIdx.x;
    const int h = static_cast<int>(a.h);
    const int vecs = h / 8;
    const int colBase = slice * (kRowVecs * kThreads);
    const int32_t *words = a.dst[src] + static_cast<int64_t>(token) * K;
    const bool records = slice == 0 && !PLAN;       // PLAN: written ahead by moon_records_kernel
    if (FRESH && records && lane < K) {
        s_dst[lane] = words[lane];
    }
    const int32_t encoded = words[k];
    const uint8_t direct = FRESH ? 0 : a.tables.direct[static_cast<int64_t>(src) * a.tables.stride + static_cast<int64_t>(token) * K + k];
    const u32x4 *srcRow = reinterpret_cast<const u32x4 *>(static_cast<const char *>(a.hiddenSh[src]) +
        static_cast<int64_t>(token) * h * 2);
    u32x4 v[kRowVecs];
#pragma unroll
    for (int i = 0; i < kRowVecs; ++i) {
        const int idx = colBase + i * kThreads + lane;
        v[i] = idx < vecs ? srcRow[idx] : u32x4{0u, 0u, 0u, 0u};
    }
    const Route r = Decode(encoded, a.nvS, a.world);
    if (!r.ok) {
        if (records && lane == 0) {
            RecordFailure(a.tables, src, a.epoch, kDispatchInvalidRoute);
        }
        return;
    }
    uint32_t tagBits = 0;
    if (SourceWrites<FRESH>(r, direct, &tagBits)) {
        u32x4 *dstRow = reinterpret_cast<u32x4 *>(static_cast<char *>(a.hiddenNvsh[r.peer]) + static_cast<int64_t>(r.row) * h * 2);
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
            RouteRecords<FRESH>(a, src, token, k, r, tagBits, s_dst);
        }
    }
}

// One workgroup per (token, slice of kTokenThreads vectors) of source rank blockIdx.y: the slice is loaded once, one
// 16-byte vector per lane, and stored once per route.  For worlds whose token rows do not all stay in the memory-side
// cache from one call to the next (eight ranks of 4096 x 7168 on one device): a kernel whose every workgroup loads
// before it stores keeps most of its speed when the rows come from HBM (127 us per rank against 150-160 us for the
// workgroup-per-route kernel, which is the faster one, 104-107 against 113-116 us, while the rows are in that cache).
constexpr int kTokenThreads = 512;
template <bool FRESH>
__global__ __launch_bounds__(kTokenThreads) void moon_scatter_token_kernel(DispatchWorld a, int colSlices)
{
    __shared__ int32_t s_dst[kMaxTopK];
    __shared__ Route s_route[kMaxTopK];
    __shared__ uint32_t s_tag[kMaxTopK];        // row tag bits of the route; 0 = the source does not write the row
    __shared__ char *s_row[kMaxTopK];           // destination row
    const int src = blockIdx.y;
    const int token = blockIdx.x / colSlices;
    const int slice = blockIdx.x % colSlices;
    const int lane = threadIdx.x;
    const int K = static_cast<int>(a.k);
    const int h = static_cast<int>(a.h);
    const int vecs = h / 8;
    const int idx = slice * kTokenThreads + lane;
    if (lane < K) {
        // one lane per route decodes it (two 64-bit divisions) for the whole workgroup
        const int64_t route = static_cast<int64_t>(token) * K + lane;
        const int32_t word = a.dst[src][route];
        const uint8_t direct = FRESH ? 0 : a.tables.direct[static_cast<int64_t>(src) * a.tables.stride + route];
        const Route r = Decode(word, a.nvS, a.world);
        uint32_t tagBits = 0;
        const bool writes = r.ok && SourceWrites<FRESH>(r, direct, &tagBits);
        s_dst[lane] = word;
        s_route[lane] = r;
        s_tag[lane] = r.ok ? tagBits : 0u;
        s_row[lane] = writes ? static_cast<char *>(a.hiddenNvsh[r.peer]) + static_cast<int64_t>(r.row) * h * 2 : nullptr;
    }
    const u32x4 *srcRow = reinterpret_cast<const u32x4 *>(static_cast<const char *>(a.hiddenSh[src]) +
        static_cast<int64_t>(token) * h * 2);
    const u32x4 v = idx < vecs ? srcRow[idx] : u32x4{0u, 0u, 0u, 0u};
    __syncthreads();
    for (int k = 0; k < K; ++k) {
        char *row = s_row[k];
        if (row != nullptr && idx < vecs) {
            __builtin_nontemporal_store(v, reinterpret_cast<u32x4 *>(row) + idx);
        }
    }
    if (slice == 0 && lane < kWave) {
        for (int k = 0; k < K; ++k) {
            const Route r = s_route[k];
            if (!r.ok) {
                if (lane == 0) {
                    RecordFailure(a.tables, src, a.epoch, kDispatchInvalidRoute);
                }
                continue;
            }
            RouteRecords<FRESH>(a, src, token, k, r, s_tag[k], s_dst);
        }
    }
}

// Any hidden size and alignment: one workgroup per route, 2-byte elements.
template <bool FRESH>
__global__ __launch_bounds__(kThreads) void moon_scatter_generic_kernel(DispatchWorld a)
{
    __shared__ int32_t s_dst[kMaxTopK];
    const int src = blockIdx.y;
    const int K = static_cast<int>(a.k);
    const int token = blockIdx.x / K;
    const int k = blockIdx.x % K;
    const int lane = threadIdx.x;
    const int32_t *words = a.dst[src] + static_cast<int64_t>(token) * K;
    if (FRESH && lane < K) {
        s_dst[lane] = words[lane];
    }
    const Route r = Decode(words[k], a.nvS, a.world);
    if (!r.ok) {
        if (lane == 0) {
            RecordFailure(a.tables, src, a.epoch, kDispatchInvalidRoute);
        }
        return;
    }
    uint32_t tagBits = 0;
    const uint8_t direct = FRESH ? 0 : a.tables.direct[static_cast<int64_t>(src) * a.tables.stride + static_cast<int64_t>(token) * K + k];
    if (SourceWrites<FRESH>(r, direct, &tagBits)) {
        const uint16_t *srcRow = static_cast<const uint16_t *>(a.hiddenSh[src]) + static_cast<int64_t>(token) * a.h;
        uint16_t *dstRow = static_cast<uint16_t *>(a.hiddenNvsh[r.peer]) + static_cast<int64_t>(r.row) * a.h;
        for (int c = lane; c < a.h; c += kThreads) {
            dstRow[c] = srcRow[c];
        }
    }
    if (FRESH) {
        TileXREp::LdsBarrier();
    }
    if (lane < kWave) {
        RouteRecords<FRESH>(a, src, token, k, r, tagBits, s_dst);
    }
}

// ---------------------------------------------------------------------------------------------------------------
// dispatch: duplicate plan of every destination rank from the parent records (fresh plans)
// ---------------------------------------------------------------------------------------------------------------

// The reference scans the destination's rows in ascending order: a group is opened by the first duplicate row of its
// primary, groups take their dupLoffs slices in that order, and each slice lists its duplicates in ascending row order
// (dispatch kernel :330-424).  With the rank-within-group and group size recorded by the sources, both numberings are
// exclusive prefix sums over the rows: group index = number of earlier group-opening rows, slice start = sum of their
// group sizes.  A workgroup scans one chunk of 2048 rows after adding up the chunks before its own -- from the rows
// themselves while the chunks are few, from the totals a first launch leaves otherwise.  The slices are filled by the
// finish kernel, which visits every row anyway.
constexpr int kBuildRows = kChunkRows;
constexpr int kBuildPer = kBuildRows / kThreads;
constexpr unsigned kSelfTotalChunks = 2;    // up to this many chunks a workgroup sums the earlier ones itself (one after
                                            // the other: measured 30 us for 17 chunks against 5 us for the extra launch)

struct ChunkRows {
    int opens[kBuildPer];
    int sizes[kBuildPer];
    int primaries[kBuildPer];
    int localOpen;
    int localSize;
};

__device__ __forceinline__ ChunkRows LoadChunkRows(const DispatchWorld &a, int rank, int64_t base)
{
    const uint64_t *parent = a.tables.parentTag + static_cast<int64_t>(rank) * a.tables.stride;
    const uint32_t *sibling = a.tables.sibling + static_cast<int64_t>(rank) * a.tables.stride;
    ChunkRows c;
    c.localOpen = 0;
    c.localSize = 0;
#pragma unroll
    for (int i = 0; i < kBuildPer; ++i) {
        const int64_t row = base + static_cast<int64_t>(threadIdx.x) * kBuildPer + i;
        c.opens[i] = 0;
        c.sizes[i] = 0;
        c.primaries[i] = -1;
        if (row < a.nvS) {
            const uint64_t p = parent[row];
            if (Tagged(p, a.epoch)) {
                const uint32_t sib = sibling[row];
                c.primaries[i] = static_cast<int>(p & 0xffffffffu) - 1;
                c.opens[i] = (sib & 0xffffu) == 0 ? 1 : 0;
                c.sizes[i] = c.opens[i] ? static_cast<int>(sib >> 16) : 0;
            }
        }
        c.localOpen += c.opens[i];
        c.localSize += c.sizes[i];
    }
    return c;
}

// Exclusive prefix of (open, size) over the threads of the workgroup, and the workgroup totals.
__device__ __forceinline__ void ScanPair(int localOpen, int localSize, int (*s_part)[kThreads / kWave], int *exclOpen,
    int *exclSize, int *totalOpen, int *totalSize)
{
    const int lane = threadIdx.x & (kWave - 1);
    const int wave = threadIdx.x / kWave;
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
    *exclOpen = inclOpen - localOpen;
    *exclSize = inclSize - localSize;
    *totalOpen = 0;
    *totalSize = 0;
#pragma unroll
    for (int w = 0; w < kThreads / kWave; ++w) {
        *exclOpen += w < wave ? s_part[0][w] : 0;
        *exclSize += w < wave ? s_part[1][w] : 0;
        *totalOpen += s_part[0][w];
        *totalSize += s_part[1][w];
    }
}

__global__ __launch_bounds__(kThreads) void moon_dedup_totals_kernel(DispatchWorld a)
{
    __shared__ int s_part[2][kThreads / kWave];
    const int rank = blockIdx.y;
    const ChunkRows c = LoadChunkRows(a, rank, static_cast<int64_t>(blockIdx.x) * kBuildRows);
    int exclOpen, exclSize, totalOpen, totalSize;
    ScanPair(c.localOpen, c.localSize, s_part, &exclOpen, &exclSize, &totalOpen, &totalSize);
    if (threadIdx.x == 0) {
        int32_t *totals = a.tables.chunkTotals + (static_cast<int64_t>(rank) * a.tables.groupStride + blockIdx.x) * 2;
        totals[0] = totalOpen;
        totals[1] = totalSize;
    }
}

// What the thread's rows of the chunks before `chunks` add to their totals.  Both words of a row are asked for whatever
// the first one says: one trip to memory per chunk, not two.  (One chunk at a time: the kernel that runs this beside a
// scatter must stay small in registers, see LaunchMoonDispatch.)
constexpr int kTotalsAhead = 1;
__device__ __forceinline__ void AddEarlierChunks(const DispatchWorld &a, int rank, int chunks, int *open, int *size)
{
    const uint64_t *parent = a.tables.parentTag + static_cast<int64_t>(rank) * a.tables.stride;
    const uint32_t *sibling = a.tables.sibling + static_cast<int64_t>(rank) * a.tables.stride;
    for (int c0 = 0; c0 < chunks; c0 += kTotalsAhead) {
        uint64_t p[kTotalsAhead][kBuildPer];
        uint32_t sib[kTotalsAhead][kBuildPer];
#pragma unroll
        for (int u = 0; u < kTotalsAhead; ++u) {
#pragma unroll
            for (int i = 0; i < kBuildPer; ++i) {
                const int64_t row = static_cast<int64_t>(c0 + u) * kBuildRows + static_cast<int64_t>(threadIdx.x) * kBuildPer + i;
                const bool in = c0 + u < chunks && row < a.nvS;
                p[u][i] = in ? parent[row] : 0ull;          // the epoch is never zero: an untagged word
                sib[u][i] = in ? sibling[row] : 0u;
            }
        }
#pragma unroll
        for (int u = 0; u < kTotalsAhead; ++u) {
#pragma unroll
            for (int i = 0; i < kBuildPer; ++i) {
                const bool opens = Tagged(p[u][i], a.epoch) && (sib[u][i] & 0xffffu) == 0;
                *open += opens ? 1 : 0;
                *size += opens ? static_cast<int>(sib[u][i] >> 16) : 0;
            }
        }
    }
}

// Groups and slice starts of one chunk of destination rank `rank` (see above).
// SELF: the workgroup adds up the chunks before its own from the row records themselves -- when the chunks are few, and
// when it runs as an extra workgroup of the scatter launch, where nothing waits for it; otherwise from the totals that a
// launch of moon_dedup_totals_kernel left.
template <bool SELF>
__device__ __forceinline__ void DedupGroupsOfChunk(const DispatchWorld &a, int rank, int chunk, bool lastChunk,
    int (*s_part)[kThreads / kWave], int *s_base)
{
    const int tid = threadIdx.x;
    // totals of the chunks before this one
    int beforeOpen = 0;
    int beforeSize = 0;
    if (SELF) {
        AddEarlierChunks(a, rank, chunk, &beforeOpen, &beforeSize);
    } else {
        const int32_t *totals = a.tables.chunkTotals + static_cast<int64_t>(rank) * a.tables.groupStride * 2;
        for (int c = tid; c < chunk; c += kThreads) {
            beforeOpen += totals[2 * c];
            beforeSize += totals[2 * c + 1];
        }
    }
    int exclOpen, exclSize, baseOpen, baseSize;
    ScanPair(beforeOpen, beforeSize, s_part, &exclOpen, &exclSize, &baseOpen, &baseSize);
    if (tid == 0) {
        s_base[0] = baseOpen;
        s_base[1] = baseSize;
    }
    __syncthreads();
    const ChunkRows c = LoadChunkRows(a, rank, static_cast<int64_t>(chunk) * kBuildRows);
    int totalOpen, totalSize;
    ScanPair(c.localOpen, c.localSize, s_part, &exclOpen, &exclSize, &totalOpen, &totalSize);
    int group = s_base[0] + exclOpen;
    int start = s_base[1] + exclSize;
    uint64_t *groupStart = a.tables.groupStart + static_cast<int64_t>(rank) * a.tables.stride;
#pragma unroll
    for (int i = 0; i < kBuildPer; ++i) {
        if (c.opens[i]) {
            // a plan in which duplicates of one token name the same row can claim more slots than there are rows
            if (group < a.nvS && static_cast<int64_t>(start) + c.sizes[i] <= a.nvS) {
                int32_t *g = a.dupGroups[rank] + static_cast<int64_t>(group) * 3;
                g[0] = c.primaries[i];
                g[1] = start;
                g[2] = c.sizes[i];
                groupStart[c.primaries[i]] = Tag(a.epoch, static_cast<uint32_t>(start));
            } else {
                RecordFailure(a.tables, rank, a.epoch, kDispatchInvalidRoute);
            }
            group += 1;
            start += c.sizes[i];
        }
    }
    if (lastChunk && tid == 0) {
        a.dupCounts[rank][0] = s_base[0] + totalOpen;
        a.dupCounts[rank][1] = s_base[1] + totalSize;
    }
}

template <bool SELF>
__global__ __launch_bounds__(kThreads) void moon_dedup_groups_kernel(DispatchWorld a)
{
    __shared__ int s_part[2][kThreads / kWave];
    __shared__ int s_base[2];
    DedupGroupsOfChunk<SELF>(a, blockIdx.y, blockIdx.x, blockIdx.x == gridDim.x - 1, s_part, s_base);
}

// ---------------------------------------------------------------------------------------------------------------
// saved duplicate plan -> records the later kernels follow (dispatch: parentTag per row; combine: per-slot tables)
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
    const int32_t *dstLocal;     // combine only
    int world;
    int64_t n;
};

// Slot (origin rank * stride + target) a receive row returns to, or -1 (reference: combine kernel :285-298).
__device__ __forceinline__ int64_t SlotOfRow(const WalkArgs &a, int32_t row)
{
    const int32_t encoded = a.dstLocal[row];
    if (encoded < 0) {
        return -1;
    }
    const int64_t peer = encoded / a.nvS;
    const int64_t target = encoded % a.nvS;
    if (peer >= a.world || target >= a.n) {
        return -1;
    }
    return peer * a.t.stride + target;
}

constexpr int kWalkBatch = 8;    // entries of a group a thread has in flight

// One thread per group.  Checks follow the reference (dispatch kernel :428-457, combine kernel :307-345).
__device__ __forceinline__ void WalkGroup(const WalkArgs &a, int64_t g)
{
    const int32_t groupCount = a.dupCounts[0];
    const int32_t duplicateCount = a.dupCounts[1];
    const int32_t invalid = a.combine ? kCombineInvalidRoute : kDispatchInvalidRoute;
    if (groupCount < 0 || groupCount > a.nvS || duplicateCount < 0 || duplicateCount > a.nvS) {
        if (g == 0) {
            RecordFailure(a.t, a.rank, a.epoch, invalid);
        }
        return;
    }
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
    // The group's entries are handled eight at a time with all loads of a batch issued together: a thread that took them
    // one by one would sit out two dependent round trips per duplicate (entry, then the entry's dstLocal word).
    // Nothing is recorded for a group with a bad entry: the kernels that follow these records do not check them again.
    bool bad = false;
    for (int32_t i0 = 0; i0 < count; i0 += kWalkBatch) {
        int32_t dup[kWalkBatch];
#pragma unroll
        for (int j = 0; j < kWalkBatch; ++j) {
            dup[j] = i0 + j < count ? a.dupLoffs[start + i0 + j] : 0;
        }
#pragma unroll
        for (int j = 0; j < kWalkBatch; ++j) {
            bad = bad || (i0 + j < count && (dup[j] < 0 || dup[j] >= a.nvS || (a.combine && dup[j] == primary)));
        }
    }
    if (bad) {
        RecordFailure(a.t, a.rank, a.epoch, invalid);
        return;
    }
    if (a.combine) {
        // the origin reads these per slot, next to the slot's row, so that one round trip tells it everything
        const int64_t slot = SlotOfRow(a, primary);
        if (slot >= 0) {
            a.t.slotCount[slot] = count;
            a.t.slotGroup[slot] = Tag(a.epoch, static_cast<uint32_t>(start));
        }
    }
    for (int32_t i0 = 0; i0 < count; i0 += kWalkBatch) {
        int32_t dup[kWalkBatch];
#pragma unroll
        for (int j = 0; j < kWalkBatch; ++j) {
            dup[j] = i0 + j < count ? a.dupLoffs[start + i0 + j] : -1;
        }
        if (a.combine) {
            int64_t slot[kWalkBatch];
#pragma unroll
            for (int j = 0; j < kWalkBatch; ++j) {
                slot[j] = dup[j] >= 0 ? SlotOfRow(a, dup[j]) : -1;
            }
#pragma unroll
            for (int j = 0; j < kWalkBatch; ++j) {
                if (slot[j] >= 0) {
                    a.t.slotDup[slot[j]] = Tag(a.epoch, 1u);
                }
            }
        } else {
#pragma unroll
            for (int j = 0; j < kWalkBatch; ++j) {
                if (dup[j] >= 0) {
                    a.t.parentTag[base + dup[j]] = Tag(a.epoch, static_cast<uint32_t>(primary) + 1u);
                }
            }
        }
    }
}

__global__ __launch_bounds__(kThreads) void moon_group_walk_kernel(DispatchWorld a)
{
    const int rank = blockIdx.y;
    WalkArgs w {a.nvS, rank, false, a.dupGroups[rank], a.dupLoffs[rank], a.dupCounts[rank], a.tables, a.epoch, nullptr, a.world, 0};
    WalkGroup(w, static_cast<int64_t>(blockIdx.x) * kThreads + threadIdx.x);
}

// ---------------------------------------------------------------------------------------------------------------
// dispatch: rows nobody wrote
// ---------------------------------------------------------------------------------------------------------------

// Work item of the finish kernel: row | kind << 30.
constexpr int32_t kFillZero = 0;
constexpr int32_t kFillCopy = 1;
constexpr int kFinishRows = 64;     // rows one workgroup looks after

// What is left to do once every source has scattered.  The first wave of a workgroup looks at 64 rows, one per lane:
// nothing (a route wrote the row), zeros (no route wrote it: the reference clears the whole window first, dispatch kernel
// :206-230), or -- saved plans -- a copy of its primary row (dispatch kernel :426-461); the weight of a row no route
// names is zero for the same reason; the duplicates of a fresh plan take their places in dupLoffs.  Then the whole
// workgroup writes the rows that need writing.  Workgroup 0 of every rank writes the rank's device status.
template <bool VEC>
__global__ __launch_bounds__(kThreads) void moon_finish_kernel(DispatchWorld a)
{
    __shared__ int32_t s_items[kFinishRows];
    __shared__ int s_count;
    const int rank = blockIdx.y;
    const int tid = threadIdx.x;
    const int64_t base = static_cast<int64_t>(rank) * a.tables.stride;
    if (tid < kWave) {
        const int64_t row = static_cast<int64_t>(blockIdx.x) * kFinishRows + tid;
        int32_t item = -1;
        if (row < a.nvS) {
            const uint64_t tag = a.tables.rowTag[base + row];
            const bool tagged = Tagged(tag, a.epoch);
            const bool named = tagged && (tag & kRowNamed) != 0;
            const bool written = tagged && (tag & kRowWritten) != 0;
            const bool direct = tagged && (tag & kRowDirect) != 0;
            const uint64_t p = a.tables.parentTag[base + row];
            if (!a.fresh && Tagged(p, a.epoch) && !direct) {
                item = static_cast<int32_t>(row) | (kFillCopy << 30);
            } else if (!written) {
                item = static_cast<int32_t>(row) | (kFillZero << 30);
            }
            if (!named && a.weightsNvs[rank] != nullptr) {
                a.weightsNvs[rank][row] = 0.0f;
            }
            if (a.fresh && Tagged(p, a.epoch)) {
                // slot of this duplicate in its group's slice (dispatch kernel :393-419)
                const uint64_t gs = a.tables.groupStart[base + static_cast<int64_t>(p & 0xffffffffu) - 1];
                if (Tagged(gs, a.epoch)) {
                    const int64_t at = static_cast<int64_t>(gs & 0xffffffffu) + (a.tables.sibling[base + row] & 0xffffu);
                    if (at < a.nvS) {
                        a.dupLoffs[rank][at] = static_cast<int32_t>(row);
                    } else {
                        RecordFailure(a.tables, rank, a.epoch, kDispatchInvalidRoute);
                    }
                }
            }
        }
        const uint64_t have = __ballot(item >= 0);
        if (item >= 0) {
            s_items[__popcll(have & ((1ull << tid) - 1ull))] = item;
        }
        if (tid == 0) {
            s_count = __popcll(have);
        }
    }
    if (blockIdx.x == 0 && tid == 0) {
        // own failure first, then the first failed peer walking upwards from this rank (dispatch kernel :559-574)
        int32_t status = kDispatchOk;
        const uint64_t own = __hip_atomic_load(&a.tables.fail[rank], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        if (Tagged(own, a.epoch)) {
            status = static_cast<int32_t>(own & 0xffffffffu);
        } else {
            for (int o = 1; o < a.world; ++o) {
                const int peer = (rank + o) % a.world;
                const uint64_t f = __hip_atomic_load(&a.tables.fail[peer], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                if (Tagged(f, a.epoch)) {
                    status = kDispatchRemoteFailureBase + peer;
                    break;
                }
            }
        }
        a.status[rank][0] = status;
    }
    __syncthreads();
    const int count = s_count;
    const int h = static_cast<int>(a.h);
    char *tensor = static_cast<char *>(a.hiddenNvsh[rank]);
    for (int i = 0; i < count; ++i) {
        const int32_t item = s_items[i];
        const int row = item & 0x3fffffff;
        bool copy = (item >> 30) == kFillCopy;
        int primary = 0;
        if (copy) {
            primary = static_cast<int>(a.tables.parentTag[base + row] & 0xffffffffu) - 1;
            // a primary no route wrote is all zeros in the reference too (the window was cleared)
            const uint64_t tag = a.tables.rowTag[base + primary];
            copy = Tagged(tag, a.epoch) && (tag & kRowWritten) != 0;
        }
        if (VEC) {
            const int vecs = h / 8;
            u32x4 *dstRow = reinterpret_cast<u32x4 *>(tensor + static_cast<int64_t>(row) * h * 2);
            const u32x4 *srcRow = reinterpret_cast<const u32x4 *>(tensor + static_cast<int64_t>(primary) * h * 2);
            for (int idx = tid; idx < vecs; idx += kThreads) {
                const u32x4 v = copy ? srcRow[idx] : u32x4{0u, 0u, 0u, 0u};
                __builtin_nontemporal_store(v, dstRow + idx);
            }
        } else {
            uint16_t *dstRow = reinterpret_cast<uint16_t *>(tensor) + static_cast<int64_t>(row) * h;
            const uint16_t *srcRow = reinterpret_cast<const uint16_t *>(tensor) + static_cast<int64_t>(primary) * h;
            for (int c = tid; c < h; c += kThreads) {
                dstRow[c] = copy ? srcRow[c] : static_cast<uint16_t>(0);
            }
        }
    }
}

// ---------------------------------------------------------------------------------------------------------------
// combine: prepare
// ---------------------------------------------------------------------------------------------------------------

// Thread i of expert rank blockIdx.y walks duplicate group i (marks the slots of its duplicates, leaves the group's extent
// at the slot of its primary) and files receive row i under the slot of the origin it returns to.
// reference: combine kernel :285-298 (decode), :350-366 (validation), :568-606 (which rows travel)
__global__ __launch_bounds__(kThreads) void moon_combine_prepare_kernel(CombineWorld a)
{
    const int rank = blockIdx.y;
    const int64_t row = static_cast<int64_t>(blockIdx.x) * kThreads + threadIdx.x;
    WalkArgs w {a.nvS, rank, true, a.dupGroups[rank], a.dupLoffs[rank], a.dupCounts[rank], a.tables, a.epoch, a.dstLocal[rank],
        a.world, a.s * a.k};
    const int32_t encoded = row < a.nvS ? a.dstLocal[rank][row] : -1;      // in flight while the group is walked
    WalkGroup(w, row);
    if (encoded == -1) {
        return;
    }
    const int64_t peer = encoded / a.nvS;
    const int64_t target = encoded % a.nvS;
    if (encoded < 0 || peer >= a.world || target >= a.s * a.k) {
        RecordFailure(a.tables, rank, a.epoch, kCombineInvalidRoute);
        return;
    }
    a.tables.slotSrc[peer * a.tables.stride + target] = Tag(a.epoch, static_cast<uint32_t>(rank * a.nvS + row));
}

// ---------------------------------------------------------------------------------------------------------------
// combine: reduce
// ---------------------------------------------------------------------------------------------------------------

// Device status of combine: own failure, else the first failed peer in rank order (combine kernel :391-411), else 0.
__device__ __forceinline__ void WriteCombineStatus(const CombineWorld &a, int rank)
{
    int32_t value = kCombineOk;
    const uint64_t own = __hip_atomic_load(&a.tables.fail[rank], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    if (Tagged(own, a.epoch)) {
        value = static_cast<int32_t>(own & 0xffffffffu);
    } else {
        for (int peer = 0; peer < a.world; ++peer) {
            const uint64_t f = __hip_atomic_load(&a.tables.fail[peer], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            if (Tagged(f, a.epoch)) {
                value = kCombineRemoteFailureBase + peer;
                break;
            }
        }
    }
    a.status[rank][0] = value;
}

// The lane's kRowVecs vectors of a row slice.  Lanes beyond the row's end read its last vector (and store nothing
// later): every lane issues every load, unconditionally.
__device__ __forceinline__ void LoadRowSlice(const void *tensor, int64_t row, int h, int vecs, int colBase, int lane, int lanes,
    u32x4 (&v)[kRowVecs])
{
    const u32x4 *p = reinterpret_cast<const u32x4 *>(static_cast<const char *>(tensor) + row * h * 2);
#pragma unroll
    for (int j = 0; j < kRowVecs; ++j) {
        const int idx = colBase + j * lanes + lane;
        v[j] = __builtin_nontemporal_load(p + (idx < vecs ? idx : vecs - 1));
    }
}

// What the reduce kernels need to know about the K slots of a token, gathered by K lanes at once so that the table
// lookups of all slots overlap (done slot after slot they would be K dependent round trips to memory).
struct TokenSlots {
    uint32_t where[kMaxTopK];   // expert rank * nvS + row of the slot's row; kNoRow when the slot contributes nothing
    int32_t start[kMaxTopK];    // first dupLoffs index of the row's duplicate group
    int32_t count[kMaxTopK];    // duplicates in the group; 0 for a row without duplicates
};
constexpr uint32_t kNoRow = 0xffffffffu;

// A slot contributes nothing when nothing was returned to it or when the row filed under it is a duplicate (a
// duplicate row does not travel: its values are part of its primary's slot, combine kernel :583-590).  Weights come
// back for every receive row, duplicates included (combine kernel :593-600).
__device__ __forceinline__ void LoadSlots(const CombineWorld &a, int rank, int token, bool writeWeights, TokenSlots *s)
{
    const int lane = threadIdx.x;
    const int K = static_cast<int>(a.k);
    if (lane >= K) {
        return;
    }
    const int64_t slot = static_cast<int64_t>(rank) * a.tables.stride + static_cast<int64_t>(token) * K + lane;
    const uint64_t w = a.tables.slotSrc[slot];
    const uint64_t dup = a.tables.slotDup[slot];
    const uint64_t group = a.tables.slotGroup[slot];
    const int32_t groupCount = a.tables.slotCount[slot];
    const bool present = Tagged(w, a.epoch);
    const uint32_t low = static_cast<uint32_t>(w);
    if (writeWeights && a.weightsSk[rank] != nullptr) {
        a.weightsSk[rank][static_cast<int64_t>(token) * K + lane] = present ? a.weightsNvs[low / a.nvS][low % a.nvS] : 0.0f;
    }
    const bool travels = present && !Tagged(dup, a.epoch);
    const bool grouped = travels && Tagged(group, a.epoch);
    s->where[lane] = travels ? low : kNoRow;
    s->start[lane] = grouped ? static_cast<int32_t>(group & 0xffffffffu) : 0;
    s->count[lane] = grouped ? groupCount : 0;
}

// What a lane of the reduce kernel knows about one of the rows its token slice sums: bits.  A row without duplicates is
// a group of one (rounding a bf16 value to bf16 changes nothing).
constexpr int kItemOpens = 1;       // the group's sum starts as this row (otherwise the row is added to it)
constexpr int kItemCloses = 2;      // after this row the group's sum is rounded to bf16 and joins the token's sum
constexpr int kItemValid = 4;       // clear: no item (the tail of a batch of loads)

// sub = row (opens: a uniform condition) or sub + row.  -0.0 + x is x for every x, zeros of either sign included.
__device__ __forceinline__ void StartOrAddRow(float (&sub)[kRowVecs][8], const u32x4 (&v)[kRowVecs], bool opens)
{
#pragma unroll
    for (int j = 0; j < kRowVecs; ++j) {
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            sub[j][2 * e] = __fadd_rn(opens ? -0.0f : sub[j][2 * e], __uint_as_float(v[j][e] << 16));
            sub[j][2 * e + 1] = __fadd_rn(opens ? -0.0f : sub[j][2 * e + 1], __uint_as_float(v[j][e] & 0xffff0000u));
        }
    }
}

__device__ __forceinline__ void AddRounded(float (&acc)[kRowVecs][8], const float (&sub)[kRowVecs][8])
{
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

// Slot sum of one token slice of origin rank blockIdx.y.  Slots are taken in slot order from zero (combine kernel
// :664-699); a slot that holds a primary with duplicates contributes bf16(fp32(primary) + fp32(dup) + ...) in the plan's
// list order (combine kernel :489-530); slots that contribute nothing leave the sum as it is (their receive row stays
// zero in the reference).
//
// One wave per slice.  Every row the slice reads -- primaries and the duplicates of their groups, in the order in which
// they are summed -- becomes an item of one lane (which tensor, which row, what to do with it), so that all look-ups
// (slot tables, then the duplicates' row numbers) are two round trips for the whole token whatever its groups look like,
// and the rows themselves are read four at a time.  Items are dealt to the lanes 64 at a time.
//
// `placed`: units are dealt by XCD (workgroup b runs on XCD b % 8 and takes a slice of a token t with t % 8 == b % 8, the
// XCD on which the scatter kernels run the token's routes), for worlds whose rows can still be in the XCDs' L2s when
// Combine follows Dispatch: rows written on one XCD and read on another travel through memory.  The tokens are padded
// to a multiple of eight.
template <int G>
__global__ __launch_bounds__(G) void moon_reduce_kernel(CombineWorld a, int colSlices, int placed)
{
    static_assert(G == kWave, "the items of a token are spread over the lanes of one wave");
    constexpr int kRowsInFlight = 4;
    __shared__ TokenSlots s_slots;
    const int rank = blockIdx.y;
    const int unit = blockIdx.x;
    int token = unit / colSlices;
    int slice = unit % colSlices;
    if (placed != 0) {
        const int j = unit / kXcds;
        token = (j / colSlices) * kXcds + unit % kXcds;
        slice = j % colSlices;
    }
    const int lane = threadIdx.x;
    if (unit == 0 && lane == 0) {
        WriteCombineStatus(a, rank);
    }
    if (token >= a.s) {
        return;
    }
    const int colBase = slice * (G * kRowVecs);
    const int h = static_cast<int>(a.h);
    const int vecs = h / 8;
    LoadSlots(a, rank, token, colBase == 0, &s_slots);
    TileXREp::LdsBarrier();
    float acc[kRowVecs][8];
#pragma unroll
    for (int j = 0; j < kRowVecs; ++j) {
#pragma unroll
        for (int e = 0; e < 8; ++e) {
            acc[j][e] = 0.0f;
        }
    }
    const int K = static_cast<int>(a.k);
    const uint32_t nvS = static_cast<uint32_t>(a.nvS);
    // lane k < K: slot k, the tensor and row of its primary, and how many items it makes
    uint32_t where = kNoRow;
    int slotStart = 0;
    int slotCount = 0;
    if (lane < K) {
        where = s_slots.where[lane];
        slotStart = s_slots.start[lane];
        slotCount = s_slots.count[lane];
    }
    const bool travels = where != kNoRow;
    const int slotQ = travels ? static_cast<int>(where / nvS) : 0;
    const int slotRow = travels ? static_cast<int>(where % nvS) : 0;
    const int slotItems = travels ? 1 + slotCount : 0;
    int slotFirst = slotItems;                       // inclusive prefix over the K <= 32 slot lanes, then exclusive
#pragma unroll
    for (int off = 1; off < kMaxTopK; off <<= 1) {
        const int below = __shfl_up(slotFirst, off);
        slotFirst += lane >= off ? below : 0;
    }
    const int total = __builtin_amdgcn_readlane(slotFirst, kMaxTopK - 1);      // lanes from K on add nothing
    slotFirst -= slotItems;
    float sub[kRowVecs][8];                          // sum of the group that is open (groups may span windows)
#pragma unroll
    for (int j = 0; j < kRowVecs; ++j) {
#pragma unroll
        for (int e = 0; e < 8; ++e) {
            sub[j][e] = 0.0f;
        }
    }
    // windows of 64 items (a token of a built plan has at most K; a saved plan may list any number of duplicates)
#pragma unroll 1
    for (int base = 0; base < total; base += kWave) {
        const int here = total - base < kWave ? total - base : kWave;
        // lane i < here: item base + i
        int itemQ = 0;
        int itemRow = 0;
        int itemKind = 0;
        const int32_t *listed = nullptr;             // where a duplicate's row number stands in its rank's dupLoffs
#pragma unroll 1
        for (int k = 0; k < K; ++k) {
            const int items = __builtin_amdgcn_readlane(slotItems, k);
            if (items == 0) {
                continue;
            }
            const int q = __builtin_amdgcn_readlane(slotQ, k);
            const int row = __builtin_amdgcn_readlane(slotRow, k);
            const int at = base + lane - __builtin_amdgcn_readlane(slotFirst, k);
            if (at >= 0 && at < items) {
                itemQ = q;
                itemRow = row;
                itemKind = kItemValid | (at == 0 ? kItemOpens : 0) | (at == items - 1 ? kItemCloses : 0);
            }
            if (items > 1) {
                const int32_t *list = a.dupLoffs[q] + __builtin_amdgcn_readlane(slotStart, k);
                if (at >= 1 && at < items) {
                    listed = list + (at - 1);
                }
            }
        }
        if (listed != nullptr) {
            itemRow = *listed;
        }
#pragma unroll 1
        for (int i0 = 0; i0 < here; i0 += kRowsInFlight) {
            u32x4 v[kRowsInFlight][kRowVecs];
            int kind[kRowsInFlight];
#pragma unroll
            for (int u = 0; u < kRowsInFlight; ++u) {
                // a batch that runs past the window reads its last row again and drops it: four loads are issued
                // whatever the count, so the sums below wait for exactly the load they need
                const int i = i0 + u < here ? i0 + u : here - 1;
                kind[u] = i0 + u < here ? __builtin_amdgcn_readlane(itemKind, i) : 0;
                const int q = __builtin_amdgcn_readlane(itemQ, i);
                const int row = __builtin_amdgcn_readlane(itemRow, i);
                LoadRowSlice(a.hiddenNvsh[q], row, h, vecs, colBase, lane, G, v[u]);
            }
#pragma unroll
            for (int u = 0; u < kRowsInFlight; ++u) {
                if ((kind[u] & kItemValid) != 0) {
                    StartOrAddRow(sub, v[u], (kind[u] & kItemOpens) != 0);
                    if ((kind[u] & kItemCloses) != 0) {
                        AddRounded(acc, sub);
                    }
                }
            }
        }
    }
    u32x4 *out = reinterpret_cast<u32x4 *>(static_cast<char *>(a.hiddenSh[rank]) + static_cast<int64_t>(token) * h * 2);
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
__global__ __launch_bounds__(kThreads) void moon_reduce_generic_kernel(CombineWorld a)
{
    __shared__ TokenSlots s_slots;
    const int rank = blockIdx.y;
    const int token = blockIdx.x;
    const int lane = threadIdx.x;
    if (token == 0 && lane == 0) {
        WriteCombineStatus(a, rank);
    }
    LoadSlots(a, rank, token, true, &s_slots);
    __syncthreads();
    const int K = static_cast<int>(a.k);
    const uint32_t nvS = static_cast<uint32_t>(a.nvS);
    for (int c = lane; c < a.h; c += kThreads) {
        float acc = 0.0f;
        for (int k = 0; k < K; ++k) {
            const uint32_t where = s_slots.where[k];
            if (where == kNoRow) {
                continue;
            }
            const int q = static_cast<int>(where / nvS);
            const int64_t row = where % nvS;
            const uint16_t *tensor = static_cast<const uint16_t *>(a.hiddenNvsh[q]);
            float value = __uint_as_float(static_cast<uint32_t>(tensor[row * a.h + c]) << 16);
            const int count = s_slots.count[k];
            if (count != 0) {
                const int start = s_slots.start[k];
                for (int i = 0; i < count; ++i) {
                    const int64_t dup = a.dupLoffs[q][start + i];
                    value = __fadd_rn(value, __uint_as_float(static_cast<uint32_t>(tensor[dup * a.h + c]) << 16));
                }
                value = __uint_as_float(TileXREp::FloatToBf16Rne(value) << 16);
            }
            acc = __fadd_rn(acc, value);
        }
        static_cast<uint16_t *>(a.hiddenSh[rank])[static_cast<int64_t>(token) * a.h + c] =
            static_cast<uint16_t>(TileXREp::FloatToBf16Rne(acc));
    }
}

hipError_t RecordIf(hipEvent_t e, hipStream_t stream)
{
    return e == nullptr ? hipSuccess : hipEventRecord(e, stream);
}

#define MOON_LAUNCH_CHECK()                \
    do {                                   \
        const hipError_t launchErr = hipGetLastError(); \
        if (launchErr != hipSuccess) {     \
            return launchErr;              \
        }                                  \
    } while (0)

} // namespace

// One device status word, written in stream order (a call that was dropped because a peer's call disagreed with it).
__global__ void moon_status_kernel(int32_t *status, int32_t value)
{
    if (threadIdx.x == 0 && blockIdx.x == 0) {
        status[0] = value;
    }
}

hipError_t LaunchMoonStatus(int32_t *status, int32_t value, hipStream_t stream)
{
    hipLaunchKernelGGL(moon_status_kernel, dim3(1), dim3(kWave), 0, stream, status, value);
    return hipGetLastError();
}

int64_t SetCachedRowBytes(int64_t bytes)
{
    return gCachedRowBytes.exchange(bytes < 0 ? 0 : bytes);
}

const char *MoonScatterKernelName()
{
    return gScatterName;
}

const char *MoonReduceKernelName()
{
    return gReduceName;
}

// What follows the routes' records: the duplicate plan of a fresh Dispatch, then the rows and weights no route wrote.
hipError_t LaunchPlanAndFinish(const DispatchWorld &w, hipStream_t stream, bool vec, bool plan)
{
    const unsigned R = static_cast<unsigned>(w.world);
    if (w.fresh && plan) {
        const unsigned chunks = static_cast<unsigned>((w.nvS + kBuildRows - 1) / kBuildRows);
        if (chunks <= kSelfTotalChunks) {
            hipLaunchKernelGGL(moon_dedup_groups_kernel<true>, dim3(chunks, R), dim3(kThreads), 0, stream, w);
        } else {
            hipLaunchKernelGGL(moon_dedup_totals_kernel, dim3(chunks, R), dim3(kThreads), 0, stream, w);
            MOON_LAUNCH_CHECK();
            hipLaunchKernelGGL(moon_dedup_groups_kernel<false>, dim3(chunks, R), dim3(kThreads), 0, stream, w);
        }
        MOON_LAUNCH_CHECK();
    }
    const unsigned groups = static_cast<unsigned>((w.nvS + kFinishRows - 1) / kFinishRows);
    if (vec) {
        hipLaunchKernelGGL(moon_finish_kernel<true>, dim3(groups, R), dim3(kThreads), 0, stream, w);
    } else {
        hipLaunchKernelGGL(moon_finish_kernel<false>, dim3(groups, R), dim3(kThreads), 0, stream, w);
    }
    return hipGetLastError();
}

hipError_t LaunchMoonDispatch(const DispatchWorld &w, hipStream_t stream, const LaunchTiming &timing)
{
    const unsigned R = static_cast<unsigned>(w.world);
    const unsigned rowBlocks = static_cast<unsigned>((w.nvS + kThreads - 1) / kThreads);
    bool vec = w.h % 8 == 0;
    for (int r = 0; r < w.world; ++r) {
        vec = vec && TileXREp::Aligned16(w.hiddenSh[r]) && TileXREp::Aligned16(w.hiddenNvsh[r]);
    }
    const int64_t vecs = w.h / 8;
    const int colSlices = static_cast<int>((vecs + kRowVecs * kThreads - 1) / (kRowVecs * kThreads));
    const int64_t blocks = (w.s + kXcds - 1) / kXcds * kXcds * w.k * colSlices;
    const int tokenSlices = static_cast<int>((vecs + kTokenThreads - 1) / kTokenThreads);
    // token rows that cannot all stay in the memory-side cache from one call to the next: the kernel that keeps its speed
    // when they come from HBM
    const int64_t worldRowBytes = static_cast<int64_t>(w.world) * w.s * w.h * 2;
    const bool uncachedRows = worldRowBytes > gCachedRowBytes.load();
    const int64_t rowVecs = w.s * vecs;
    const bool perToken = vec && uncachedRows && w.s * tokenSlices <= 0x7fffffff;
    const bool perRoute = vec && !perToken && blocks <= 0x7fffffff;
    // up to half the memory-side cache of token rows: read them once so that the per-route kernel finds them there
    // (one rank's share of 4096 x 7168: 257 -> about 210 us per layer on rows that were not cached, a few us more
    // on rows that were)
    const bool warm = perRoute && worldRowBytes <= kWarmRowBytes;
    const unsigned warmBlocks = warm ? static_cast<unsigned>((rowVecs + kThreads * kWarmLoads - 1) / (kThreads * kWarmLoads)) : 0u;
    const unsigned routeBlocks = static_cast<unsigned>((w.s * w.k + kThreads - 1) / kThreads);
    // A fresh plan of a world whose rows are copied per route and come to at most kFusedPlanRowBytes: what the routes
    // record is written ahead of the scatter, by the launch that reads the token rows ahead, and the plan is built by
    // extra workgroups of the scatter launch; only the finish kernel follows the scatter.  Three launches instead of five
    // while a rank has at most kSelfPlanChunks chunks, four (the chunk totals need one) beyond: 128 tokens x 7168 x top-8
    // 36.6 -> 34.2 us per layer, 384 tokens 47.8 -> 41.6, 1024 tokens 77.5 -> 71.8, 4096 tokens x 2048 99.8 -> 93.6.  The
    // scatter kernel that holds the plan's code has 50 registers per lane instead of 16, and its short-lived workgroups
    // then start more slowly: from about 256 MB of rows on that costs more than the launches saved (4096 tokens x 7168
    // 201 -> 204 us, 8192 tokens 365 -> 386 us), so larger worlds keep the plain kernel and the launches after it.
    const int planChunks = static_cast<int>((w.nvS + kBuildRows - 1) / kBuildRows);
    const bool planInScatter = w.fresh && perRoute && planChunks <= kFusedPlanChunks &&
        static_cast<int64_t>(w.world) * w.s * w.k * w.h * 2 <= kFusedPlanRowBytes;
    const bool planSelf = planChunks <= kSelfPlanChunks;
    const unsigned planBlocks = planInScatter ? static_cast<unsigned>((planChunks + kXcds - 1) / kXcds * kXcds) : 0u;
    if (planInScatter) {
        hipLaunchKernelGGL(moon_records_kernel, dim3(routeBlocks + warmBlocks, R), dim3(kThreads), 0, stream, w, routeBlocks,
            warm ? rowVecs : int64_t{0});
        MOON_LAUNCH_CHECK();
        if (!planSelf) {
            hipLaunchKernelGGL(moon_dedup_totals_kernel, dim3(static_cast<unsigned>(planChunks), R), dim3(kThreads), 0, stream, w);
            MOON_LAUNCH_CHECK();
        }
    } else if (!w.fresh) {
        hipLaunchKernelGGL(moon_group_walk_kernel, dim3(rowBlocks, R), dim3(kThreads), 0, stream, w);
        MOON_LAUNCH_CHECK();
        hipLaunchKernelGGL(moon_agree_kernel, dim3(routeBlocks + warmBlocks, R), dim3(kThreads), 0, stream, w, routeBlocks,
            warm ? rowVecs : int64_t{0});
        MOON_LAUNCH_CHECK();
    } else if (warm) {
        hipLaunchKernelGGL(moon_warm_rows_kernel, dim3(warmBlocks, R), dim3(kThreads), 0, stream, w, rowVecs);
        MOON_LAUNCH_CHECK();
    }
    hipError_t err = RecordIf(timing.start, stream);
    if (err != hipSuccess) {
        return err;
    }
    if (perToken) {
        gScatterName = "moon_scatter_token_kernel";
        const dim3 grid(static_cast<unsigned>(w.s * tokenSlices), R);
        if (w.fresh) {
            hipLaunchKernelGGL(moon_scatter_token_kernel<true>, grid, dim3(kTokenThreads), 0, stream, w, tokenSlices);
        } else {
            hipLaunchKernelGGL(moon_scatter_token_kernel<false>, grid, dim3(kTokenThreads), 0, stream, w, tokenSlices);
        }
    } else if (perRoute) {
        gScatterName = "moon_scatter_kernel";
        const dim3 grid(static_cast<unsigned>(blocks) + planBlocks, R);
        if (planInScatter) {
            hipLaunchKernelGGL((moon_scatter_kernel<true, true>), grid, dim3(kThreads), 0, stream, w, colSlices, planBlocks,
                planChunks, planSelf ? 1 : 0);
        } else if (w.fresh) {
            hipLaunchKernelGGL((moon_scatter_kernel<true, false>), grid, dim3(kThreads), 0, stream, w, colSlices, 0u, 0, 0);
        } else {
            hipLaunchKernelGGL((moon_scatter_kernel<false, false>), grid, dim3(kThreads), 0, stream, w, colSlices, 0u, 0, 0);
        }
    } else {
        gScatterName = "moon_scatter_generic_kernel";
        const unsigned grid = static_cast<unsigned>(w.s * w.k);
        if (w.fresh) {
            hipLaunchKernelGGL(moon_scatter_generic_kernel<true>, dim3(grid, R), dim3(kThreads), 0, stream, w);
        } else {
            hipLaunchKernelGGL(moon_scatter_generic_kernel<false>, dim3(grid, R), dim3(kThreads), 0, stream, w);
        }
    }
    MOON_LAUNCH_CHECK();
    err = RecordIf(timing.stop, stream);
    if (err != hipSuccess) {
        return err;
    }
    return LaunchPlanAndFinish(w, stream, vec, !planInScatter);
}

hipError_t LaunchMoonCombine(const CombineWorld &w, hipStream_t stream, const LaunchTiming &timing)
{
    const unsigned R = static_cast<unsigned>(w.world);
    const unsigned rowBlocks = static_cast<unsigned>((w.nvS + kThreads - 1) / kThreads);
    hipLaunchKernelGGL(moon_combine_prepare_kernel, dim3(rowBlocks, R), dim3(kThreads), 0, stream, w);
    MOON_LAUNCH_CHECK();
    bool vec = w.h % 8 == 0;
    for (int r = 0; r < w.world; ++r) {
        vec = vec && TileXREp::Aligned16(w.hiddenSh[r]) && TileXREp::Aligned16(w.hiddenNvsh[r]);
    }
    const int64_t vecs = w.h / 8;
    constexpr int G = kWave;
    const int colSlices = static_cast<int>((vecs + G * kRowVecs - 1) / (G * kRowVecs));
    // up to three times the L2s' 32 MB of receive rows in the world: the slices of a token go to the XCD that wrote its rows
    const bool placed = static_cast<int64_t>(w.world) * w.nvS * w.h * 2 <= (int64_t{96} << 20);
    const int64_t units = (placed ? (w.s + kXcds - 1) / kXcds * kXcds : w.s) * colSlices;
    hipError_t err = RecordIf(timing.start, stream);
    if (err != hipSuccess) {
        return err;
    }
    if (vec && units <= 0x7fffffff) {
        gReduceName = "moon_reduce_kernel";
        hipLaunchKernelGGL(moon_reduce_kernel<G>, dim3(static_cast<unsigned>(units), R), dim3(G), 0, stream, w, colSlices,
            placed ? 1 : 0);
    } else {
        gReduceName = "moon_reduce_generic_kernel";
        hipLaunchKernelGGL(moon_reduce_generic_kernel, dim3(static_cast<unsigned>(w.s), R), dim3(kThreads), 0, stream, w);
    }
    MOON_LAUNCH_CHECK();
    return RecordIf(timing.stop, stream);
}

} // namespace TileXRMoon
