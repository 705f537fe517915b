// Entry points of the test- and bench-only companion library libtilexr-ep-probes.so (ep_probe.hip): memory-system
// yardsticks and a stand-in expert stage.  Not part of the product library and not installed: nothing on the dispatch /
// combine path calls these, and libtilexr-ep.so does not export them.
#ifndef TILEXR_AMD_EP_PROBE_H
#define TILEXR_AMD_EP_PROBE_H

#include <cstdint>

#include "tilexr_ep.h"

extern "C" {
#pragma GCC visibility push(default)

// Measurement aid without a reference counterpart: one launch of a kernel that does nothing but the memory traffic of
// a given pattern, so that a harness can time what this device's memory system delivers for the read : write mix of
// the scatter and reduce kernels.  `bytes` is the size of the larger side and a multiple of 128; pointers are device
// memory, 16-byte aligned.
//   READ     reads `bytes` of src                     (dst: at least 4 bytes, not written in practice)
//   WRITE    writes `bytes` of dst                    (src unused)
//   COPY     reads `bytes` of src, writes `bytes` of dst
//   FAN_OUT  reads bytes / 8 of src, writes `bytes` of dst as eight copies   (the scatter's 1 : 8 mix)
//   FAN_IN   reads `bytes` of src as eight regions, writes bytes / 8 of dst  (the reduce's 8 : 1 mix)
//   GATHER_ROWS  the same mix with the reduce's addresses: src is rows of 14336 bytes, every output row combines
//            eight source rows at unrelated positions; `bytes` a multiple of 8 * 14336; writes bytes / 8 of dst
//   GATHER_ROWS_2K_X8 / GATHER_ROWS_4K_X6  the quantised reduce's mix and addresses: src is rows of 2048 (4096) one-byte
//            payloads, every output row of twice that many bytes combines eight (six) source rows at unrelated
//            positions; `bytes` a multiple of 8 * 2048 (6 * 4096), fewer than 2^17 rows; writes bytes / 4 (bytes / 3)
//            of dst
// Asynchronous on `stream`; returns 0, -3 for bad arguments, -2 when the launch fails.
enum TileXREpProbePattern {
    TILEXR_EP_PROBE_READ = 0,
    TILEXR_EP_PROBE_WRITE = 1,
    TILEXR_EP_PROBE_COPY = 2,
    TILEXR_EP_PROBE_FAN_OUT = 3,
    TILEXR_EP_PROBE_FAN_IN = 4,
    TILEXR_EP_PROBE_GATHER_ROWS = 5,
    TILEXR_EP_PROBE_GATHER_ROWS_2K_X8 = 6,
    TILEXR_EP_PROBE_GATHER_ROWS_4K_X6 = 7
};
int TileXREpMemoryProbe(int pattern, const void *src, void *dst, int64_t bytes, aclrtStream stream);

// Measurement aid without a reference counterpart: a stand-in for an expert stage between dispatch and combine, so
// that a harness can time (and a test can check) a combine that follows a producer which is slower than memory and
// publishes tiles as it goes.  `workgroups` workgroups copy rows [0, rows) of `rowBytes` bytes (a multiple of 16) from
// `src` to `dst`, tile by tile (workgroup w takes tiles w, w + workgroups, ...), spend at least `minTileNs` on a tile
// (workgroup w starting w * staggerNs / workgroups late: with staggerNs = minTileNs tiles complete at a steady rate
// instead of `workgroups` at a time),
// and publish it the way any producer outside this library has to: rows complete, one release at agent scope, then
// tileFlags[tile] = (epoch << 32) | rows in the tile.  `rows` is a host value (the kept rows of the dispatch).
// Asynchronous on `stream`; returns 0, -3 for bad arguments, -2 when the launch fails.
int TileXREpTileProducerProbe(const void *src, void *dst, int64_t rows, int64_t rowBytes, uint64_t *tileFlags,
    int64_t tileRows, int64_t epoch, int64_t workgroups, int64_t minTileNs, int64_t staggerNs, aclrtStream stream);

#pragma GCC visibility pop
}

#endif // TILEXR_AMD_EP_PROBE_H
