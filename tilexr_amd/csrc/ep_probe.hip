// Memory-system yardsticks for gfx950: the access patterns of the dispatch / combine data kernels with everything but
// the memory traffic taken out, so that a harness can price those kernels against what this device's memory system
// delivers for their mix of reads and writes rather than against the nominal HBM peak alone.
//
//   read      every byte of src once (two 16-byte non-temporal loads per lane)
//   write     every byte of dst once (one 16-byte non-temporal store per lane)
//   copy      src -> dst, two loads then two stores per lane
//   fan-out   the scatter's mix: a block of src is loaded once and stored to eight regions of dst (1 read : 8 writes)
//   fan-in    the reduce's mix: eight regions of src are loaded and one region of dst is stored (8 reads : 1 write)
//   gather    the same mix with the reduce's addresses: every output row of 14 KiB combines eight rows of src that lie
//             at unrelated positions
//
//   tile producer   a stand-in for an expert stage between dispatch and combine: a few workgroups copy rows tile by tile,
//             spend a set time per tile, and publish every tile's readiness word the way any producer outside this
//             library has to: rows complete, release at agent scope, then the word
//
// No reference counterpart; nothing on the dispatch / combine path calls these.
#include <hip/hip_runtime.h>

#include "ep_kernel_common.hip.h"
#include "ep_numerics.hip.h"
#include "ep_probe.h"
#include "tilexr_ep_publish.hip.h"
#include "tilexr_types.h"

namespace TileXREp {
namespace {

__global__ __launch_bounds__(kThreads) void ep_probe_read_kernel(const u32x4 *src, int64_t vecs, uint32_t *sink)
{
    const int64_t base = static_cast<int64_t>(blockIdx.x) * (2 * kThreads) + threadIdx.x;
    uint32_t acc = 0;
#pragma unroll
    for (int i = 0; i < 2; ++i) {
        const int64_t at = base + static_cast<int64_t>(i) * kThreads;
        if (at < vecs) {
            const u32x4 v = __builtin_nontemporal_load(src + at);
            acc |= v[0] & v[1] & v[2] & v[3];
        }
    }
    if (acc == 0x9e3779b9u) {       // keeps the loads alive; all but never true
        *sink = acc;
    }
}

__global__ __launch_bounds__(kThreads) void ep_probe_write_kernel(u32x4 *dst, int64_t vecs)
{
    const int64_t at = static_cast<int64_t>(blockIdx.x) * kThreads + threadIdx.x;
    if (at < vecs) {
        __builtin_nontemporal_store(u32x4{1u, 2u, 3u, 4u}, dst + at);
    }
}

__global__ __launch_bounds__(kThreads) void ep_probe_copy_kernel(const u32x4 *src, u32x4 *dst, int64_t vecs)
{
    const int64_t base = static_cast<int64_t>(blockIdx.x) * (2 * kThreads) + threadIdx.x;
    u32x4 v[2];
#pragma unroll
    for (int i = 0; i < 2; ++i) {
        const int64_t at = base + static_cast<int64_t>(i) * kThreads;
        v[i] = at < vecs ? __builtin_nontemporal_load(src + at) : u32x4{0u, 0u, 0u, 0u};
    }
#pragma unroll
    for (int i = 0; i < 2; ++i) {
        const int64_t at = base + static_cast<int64_t>(i) * kThreads;
        if (at < vecs) {
            __builtin_nontemporal_store(v[i], dst + at);
        }
    }
}

// one wave per workgroup: a 1 KiB block of src, stored at the same offset of each of the eight regions of dst
__global__ __launch_bounds__(kWave) void ep_probe_fan_out_kernel(const u32x4 *src, u32x4 *dst, int64_t regionVecs)
{
    const int64_t at = static_cast<int64_t>(blockIdx.x) * kWave + threadIdx.x;
    if (at >= regionVecs) {
        return;
    }
    const u32x4 v = src[at];
#pragma unroll
    for (int k = 0; k < 8; ++k) {
        __builtin_nontemporal_store(v, dst + static_cast<int64_t>(k) * regionVecs + at);
    }
}

// one wave per workgroup: the same 1 KiB block of each of the eight regions of src, combined into one block of dst
__global__ __launch_bounds__(kWave) void ep_probe_fan_in_kernel(const u32x4 *src, u32x4 *dst, int64_t regionVecs)
{
    const int64_t at = static_cast<int64_t>(blockIdx.x) * kWave + threadIdx.x;
    if (at >= regionVecs) {
        return;
    }
    u32x4 v[8];
#pragma unroll
    for (int k = 0; k < 8; ++k) {
        v[k] = __builtin_nontemporal_load(src + static_cast<int64_t>(k) * regionVecs + at);
    }
    u32x4 acc = v[0];
#pragma unroll
    for (int k = 1; k < 8; ++k) {
        acc ^= v[k];
    }
    __builtin_nontemporal_store(acc, dst + at);
}

// The reduce's mix with the reduce's addresses: src is rows of kProbeRowBytes; output row t is combined from eight rows
// at unrelated positions ((t * stride_k + k) mod rows, a bijection per k because the strides are coprime to the row
// count chosen by the launcher).  One wave per 1 KiB slice of an output row, as in the reduce kernel.
constexpr int kProbeRowBytes = 14336;
constexpr int kProbeRowVecs = kProbeRowBytes / 16;
__global__ __launch_bounds__(kWave) void ep_probe_gather_rows_kernel(const u32x4 *src, u32x4 *dst, int64_t rows)
{
    constexpr int kSlices = kProbeRowVecs / kWave;
    const uint32_t t = blockIdx.x / kSlices;
    const int at = (blockIdx.x % kSlices) * kWave + threadIdx.x;
    const uint32_t strides[8] = {1u, 7919u, 10007u, 12289u, 15013u, 17389u, 20011u, 22291u};   // primes; rows < 2^17
    u32x4 v[8];
#pragma unroll
    for (int k = 0; k < 8; ++k) {
        const uint32_t row = (t * strides[k] + static_cast<uint32_t>(k) * 977u) % static_cast<uint32_t>(rows);
        v[k] = __builtin_nontemporal_load(src + static_cast<int64_t>(row) * kProbeRowVecs + at);
    }
    u32x4 acc = v[0];
#pragma unroll
    for (int k = 1; k < 8; ++k) {
        acc ^= v[k];
    }
    __builtin_nontemporal_store(acc, dst + static_cast<int64_t>(t) * kProbeRowVecs + at);
}

// The quantised reduce's mix with its addresses: src is rows of ROW_BYTES one-byte payloads, output row t (two bytes per
// column) is combined from K rows at unrelated positions.  One wave per 1 KiB slice of the input rows: K 16-byte loads
// and two 16-byte stores per lane.
template <int ROW_BYTES, int K>
__global__ __launch_bounds__(kWave) void ep_probe_gather_narrow_kernel(const u32x4 *src, u32x4 *dst, int64_t rows)
{
    constexpr int kRowVecs = ROW_BYTES / 16;
    constexpr int kSlices = kRowVecs / kWave;
    const uint32_t t = blockIdx.x / kSlices;
    const int at = (blockIdx.x % kSlices) * kWave + threadIdx.x;
    const uint32_t strides[8] = {1u, 7919u, 10007u, 12289u, 15013u, 17389u, 20011u, 22291u};
    u32x4 v[K];
#pragma unroll
    for (int k = 0; k < K; ++k) {
        const uint32_t row = (t * strides[k] + static_cast<uint32_t>(k) * 977u) % static_cast<uint32_t>(rows);
        v[k] = __builtin_nontemporal_load(src + static_cast<int64_t>(row) * kRowVecs + at);
    }
    u32x4 acc = v[0];
#pragma unroll
    for (int k = 1; k < K; ++k) {
        acc ^= v[k];
    }
    u32x4 *out = dst + (static_cast<int64_t>(t) * kRowVecs + at) * 2;
    __builtin_nontemporal_store(acc, out);
    __builtin_nontemporal_store(acc ^ v[K - 1], out + 1);
}

// Tiles t = blockIdx.x, blockIdx.x + gridDim.x, ... in turn.  Ordinary loads and stores (the rows may sit dirty in this
// XCD's L2), then per tile: every wave waits for its stores, the barrier collects the waves, one lane writes the L2 back
// with a release fence at agent scope and stores the word.  One such fence per tile of tens of rows is cheap; one per row
// is not (the scatter kernels therefore write rows through instead).
__global__ __launch_bounds__(kThreads) void ep_probe_tile_producer_kernel(const char *src, char *dst, int rows,
    int64_t rowBytes, uint64_t *tileFlags, int tileRows, uint64_t epoch, int64_t minTileTicks, int64_t staggerTicks)
{
    const int tiles = (rows + tileRows - 1) / tileRows;
    if (staggerTicks > 0) {
        // workgroups that do not move in step: workgroup w starts w / gridDim.x of the stagger late
        const uint64_t launch = wall_clock64();
        const int64_t late = staggerTicks * static_cast<int64_t>(blockIdx.x) / static_cast<int64_t>(gridDim.x);
        while (static_cast<int64_t>(wall_clock64() - launch) < late) {
            __builtin_amdgcn_s_sleep(32);
        }
    }
    const int64_t vecsPerRow = rowBytes / 16;
    for (int tile = blockIdx.x; tile < tiles; tile += gridDim.x) {
        const uint64_t begin = wall_clock64();
        const int first = tile * tileRows;
        const int count = min(tileRows, rows - first);
        const u32x4 *in = reinterpret_cast<const u32x4 *>(src + static_cast<int64_t>(first) * rowBytes);
        u32x4 *out = reinterpret_cast<u32x4 *>(dst + static_cast<int64_t>(first) * rowBytes);
        const int64_t vecs = vecsPerRow * count;
        for (int64_t at = threadIdx.x; at < vecs; at += 4 * kThreads) {
            u32x4 v[4];
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const int64_t idx = at + static_cast<int64_t>(i) * kThreads;
                v[i] = idx < vecs ? in[idx] : u32x4{0u, 0u, 0u, 0u};
            }
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const int64_t idx = at + static_cast<int64_t>(i) * kThreads;
                if (idx < vecs) {
                    out[idx] = v[i];
                }
            }
        }
        // the time an expert stage would spend computing the tile
        while (static_cast<int64_t>(wall_clock64() - begin) < minTileTicks) {
            __builtin_amdgcn_s_sleep(32);
        }
        // the publishing rule of tilexr_ep_publish.hip.h, with that header's functions and nothing else, as a producer
        // outside the library would write it
        TileXREpWaitOwnStores();
        __syncthreads();
        if (threadIdx.x == 0) {
            TileXREpReleaseRowsToAgent();
            TileXREpPublishTile(tileFlags, tile, epoch, count);
        }
    }
}

} // namespace
} // namespace TileXREp

extern "C" int TileXREpTileProducerProbe(const void *src, void *dst, int64_t rows, int64_t rowBytes, uint64_t *tileFlags,
    int64_t tileRows, int64_t epoch, int64_t workgroups, int64_t minTileNs, int64_t staggerNs, aclrtStream stream)
{
    using namespace TileXREp;
    if (src == nullptr || dst == nullptr || tileFlags == nullptr || stream == nullptr || !Aligned16(src) || !Aligned16(dst) ||
        rows <= 0 || rows > 0x7fffffff || rowBytes <= 0 || rowBytes % 16 != 0 || tileRows <= 0 || tileRows > 0x7fffffff ||
        epoch <= 0 || epoch > 0xffffffffll || workgroups <= 0 || workgroups > 65535 || minTileNs < 0 ||
        minTileNs > 1000000000ll || staggerNs < 0 || staggerNs > 1000000000ll) {
        return TileXR::TILEXR_ERROR_PARA_CHECK_FAIL;
    }
    const int64_t ticks = minTileNs / 10;       // wall_clock64() counts at 100 MHz
    hipLaunchKernelGGL(ep_probe_tile_producer_kernel, dim3(static_cast<unsigned>(workgroups)), dim3(kThreads), 0,
        static_cast<hipStream_t>(stream), static_cast<const char *>(src), static_cast<char *>(dst), static_cast<int>(rows),
        rowBytes, tileFlags, static_cast<int>(tileRows), static_cast<uint64_t>(epoch), ticks, staggerNs / 10);
    return hipGetLastError() == hipSuccess ? TileXR::TILEXR_SUCCESS : TileXR::TILEXR_ERROR_MKIRT;
}

extern "C" int TileXREpMemoryProbe(int pattern, const void *src, void *dst, int64_t bytes, aclrtStream stream)
{
    using namespace TileXREp;
    const bool needSrc = pattern != TILEXR_EP_PROBE_WRITE;
    const bool needDst = true;      // the read probe uses dst as a 4-byte sink
    if (pattern == TILEXR_EP_PROBE_GATHER_ROWS && (bytes % (8 * kProbeRowBytes) != 0 || bytes / kProbeRowBytes >= (1 << 17))) {
        return TileXR::TILEXR_ERROR_PARA_CHECK_FAIL;
    }
    if (pattern == TILEXR_EP_PROBE_GATHER_ROWS_2K_X8 && (bytes % (8 * 2048) != 0 || bytes / 2048 >= (1 << 17))) {
        return TileXR::TILEXR_ERROR_PARA_CHECK_FAIL;
    }
    if (pattern == TILEXR_EP_PROBE_GATHER_ROWS_4K_X6 && (bytes % (6 * 4096) != 0 || bytes / 4096 >= (1 << 17))) {
        return TileXR::TILEXR_ERROR_PARA_CHECK_FAIL;
    }
    if (pattern < TILEXR_EP_PROBE_READ || pattern > TILEXR_EP_PROBE_GATHER_ROWS_4K_X6 || bytes < 128 || bytes % 128 != 0 ||
        bytes > (int64_t{1} << 40) || (needSrc && (src == nullptr || !Aligned16(src))) ||
        (needDst && (dst == nullptr || !Aligned16(dst)))) {
        return TileXR::TILEXR_ERROR_PARA_CHECK_FAIL;
    }
    hipStream_t s = static_cast<hipStream_t>(stream);
    const int64_t vecs = bytes / 16;
    const u32x4 *in = static_cast<const u32x4 *>(src);
    u32x4 *out = static_cast<u32x4 *>(dst);
    auto blocks = [](int64_t items, int64_t perBlock) { return dim3(static_cast<unsigned>((items + perBlock - 1) / perBlock)); };
    switch (pattern) {
        case TILEXR_EP_PROBE_READ:
            hipLaunchKernelGGL(ep_probe_read_kernel, blocks(vecs, 2 * kThreads), dim3(kThreads), 0, s, in, vecs,
                static_cast<uint32_t *>(dst));
            break;
        case TILEXR_EP_PROBE_WRITE:
            hipLaunchKernelGGL(ep_probe_write_kernel, blocks(vecs, kThreads), dim3(kThreads), 0, s, out, vecs);
            break;
        case TILEXR_EP_PROBE_COPY:
            hipLaunchKernelGGL(ep_probe_copy_kernel, blocks(vecs, 2 * kThreads), dim3(kThreads), 0, s, in, out, vecs);
            break;
        case TILEXR_EP_PROBE_FAN_OUT:
            hipLaunchKernelGGL(ep_probe_fan_out_kernel, blocks(vecs / 8, kWave), dim3(kWave), 0, s, in, out, vecs / 8);
            break;
        case TILEXR_EP_PROBE_FAN_IN:
            hipLaunchKernelGGL(ep_probe_fan_in_kernel, blocks(vecs / 8, kWave), dim3(kWave), 0, s, in, out, vecs / 8);
            break;
        case TILEXR_EP_PROBE_GATHER_ROWS_2K_X8: {
            const int64_t rows = bytes / 2048;
            hipLaunchKernelGGL((ep_probe_gather_narrow_kernel<2048, 8>), blocks(vecs / 8, kWave), dim3(kWave), 0, s, in, out, rows);
            break;
        }
        case TILEXR_EP_PROBE_GATHER_ROWS_4K_X6: {
            const int64_t rows = bytes / 4096;
            hipLaunchKernelGGL((ep_probe_gather_narrow_kernel<4096, 6>), blocks(vecs / 6, kWave), dim3(kWave), 0, s, in, out, rows);
            break;
        }
        default: {
            const int64_t rows = bytes / kProbeRowBytes;
            hipLaunchKernelGGL(ep_probe_gather_rows_kernel, blocks(vecs / 8, kWave), dim3(kWave), 0, s, in, out, rows);
            break;
        }
    }
    return hipGetLastError() == hipSuccess ? TileXR::TILEXR_SUCCESS : TileXR::TILEXR_ERROR_MKIRT;
}
