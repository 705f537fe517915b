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
// No reference counterpart; nothing on the dispatch / combine path calls these.
#include <hip/hip_runtime.h>

#include "ep_kernel_common.hip.h"
#include "ep_numerics.hip.h"
#include "tilexr_ep.h"
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

} // namespace
} // namespace TileXREp

extern "C" int TileXREpMemoryProbe(int pattern, const void *src, void *dst, int64_t bytes, aclrtStream stream)
{
    using namespace TileXREp;
    const bool needSrc = pattern != TILEXR_EP_PROBE_WRITE;
    const bool needDst = true;      // the read probe uses dst as a 4-byte sink
    if (pattern == TILEXR_EP_PROBE_GATHER_ROWS && (bytes % (8 * kProbeRowBytes) != 0 || bytes / kProbeRowBytes >= (1 << 17))) {
        return TileXR::TILEXR_ERROR_PARA_CHECK_FAIL;
    }
    if (pattern < TILEXR_EP_PROBE_READ || pattern > TILEXR_EP_PROBE_GATHER_ROWS || bytes < 128 || bytes % 128 != 0 ||
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
        default: {
            const int64_t rows = bytes / kProbeRowBytes;
            hipLaunchKernelGGL(ep_probe_gather_rows_kernel, blocks(vecs / 8, kWave), dim3(kWave), 0, s, in, out, rows);
            break;
        }
    }
    return hipGetLastError() == hipSuccess ? TileXR::TILEXR_SUCCESS : TileXR::TILEXR_ERROR_MKIRT;
}
