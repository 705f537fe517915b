// Readiness-tile bookkeeping shared by the scatter kernels (device atomics) and a host-side hook that runs the same
// code on CPU threads, so the counting logic can be stressed without a GPU.
//
// A tile's readiness word is stored exactly once per dispatch, by whoever lands the last part of the tile's last
// row, and only after every part of every row of the tile has been counted.  Counters return to zero.  Tiles wider
// than kTileSubRows rows are counted in two levels (groups of kTileSubRows rows, then completed groups), because
// atomics on one address complete at only about three per microsecond on gfx950.
//
// `Ops` supplies the three memory operations: FetchAdd(uint32_t *, 1) -> previous value, Store(uint32_t *, v),
// Store(uint64_t *, v).  A caller makes its part of the row complete in memory before it calls PublishLanded.
#ifndef TILEXR_AMD_EP_TILE_PUBLISH_H
#define TILEXR_AMD_EP_TILE_PUBLISH_H

#include <cstdint>

#include "tilexr_ep_publish.hip.h"

#if defined(__HIPCC__)
#define TILEXR_EP_HD __host__ __device__ inline __attribute__((always_inline))
#else
#define TILEXR_EP_HD inline
#endif

namespace TileXREp {

constexpr int kTileSubRows = 16;

// Words of counter scratch for up to maxRows rows: one per tile, then one per group of a wide tile.
inline int64_t TileCounterWords(int64_t maxRows, int64_t tileRows)
{
    const int64_t tiles = (maxRows + tileRows - 1) / tileRows;
    const int64_t groupsPerTile = tileRows > kTileSubRows ? (tileRows + kTileSubRows - 1) / kTileSubRows : 0;
    return tiles * (1 + groupsPerTile);
}

struct TilePublishArgs {
    uint64_t *flags;         // readiness words, one per tile
    uint32_t *counters;      // TileCounterWords(maxRows, tileRows) words, all zero between dispatches
    int tileRows;
    int maxTiles;            // tiles of the largest possible row count: the group counters start there
    int totalRows;           // rows this dispatch keeps (size of the last tile)
    uint64_t epoch;
};

// The word a complete tile is published with, and the consumer's test of a polled word: ready means "published for
// exactly this epoch".  A word of an older epoch, a word of a newer one and a zero-filled word all read as not ready.
// (One definition, in the installed header that producers and consumers outside the library include.)
TILEXR_EP_HD uint64_t TileReadyWord(uint64_t epoch, int rowsInTile)
{
    return TileXREpTileReadyWord(epoch, rowsInTile);
}

TILEXR_EP_HD bool TileWordReady(uint64_t word, uint64_t epoch)
{
    return TileXREpTileWordReady(word, epoch);
}

template <typename Ops>
TILEXR_EP_HD bool CountLanded(Ops &ops, uint32_t *counter, int target)
{
    const uint32_t before = ops.FetchAdd(counter);
    if (static_cast<int>(before) + 1 != target) {
        return false;
    }
    ops.Store(counter, 0u);      // nobody else touches it until the next dispatch
    return true;
}

// One of the `parts` callers that publish row `row` reports its part as landed.
template <typename Ops>
TILEXR_EP_HD void PublishLanded(Ops &ops, const TilePublishArgs &a, int row, int parts)
{
    const int tile = row / a.tileRows;
    int rowsInTile = 1;
    if (a.tileRows > 1 || parts > 1) {
        const int left = a.totalRows - tile * a.tileRows;
        rowsInTile = left < a.tileRows ? left : a.tileRows;
        if (a.tileRows <= kTileSubRows) {
            if (!CountLanded(ops, &a.counters[tile], rowsInTile * parts)) {
                return;
            }
        } else {
            const int groupsPerTile = (a.tileRows + kTileSubRows - 1) / kTileSubRows;
            const int group = (row - tile * a.tileRows) / kTileSubRows;
            const int leftInTile = rowsInTile - group * kTileSubRows;
            const int rowsInGroup = leftInTile < kTileSubRows ? leftInTile : kTileSubRows;
            if (!CountLanded(ops, &a.counters[a.maxTiles + tile * groupsPerTile + group], rowsInGroup * parts)) {
                return;
            }
            if (!CountLanded(ops, &a.counters[tile], (rowsInTile + kTileSubRows - 1) / kTileSubRows)) {
                return;
            }
        }
    }
    ops.Store(&a.flags[tile], TileReadyWord(a.epoch, rowsInTile));
}

} // namespace TileXREp

#endif // TILEXR_AMD_EP_TILE_PUBLISH_H
