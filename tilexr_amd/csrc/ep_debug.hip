// Debug aids of the dispatch / combine path (no reference counterpart as an API; the reference's kernels leave
// breadcrumbs of the same kind: RunPosRecord, src/ep/kernels/tilexr_ep_dispatch_memory_kernel.h:1319-1328, run
// positions :28-30).
//
//   phase stamps   a one-thread kernel ahead of and behind every kernel of a call writes {call magic, kernel id, edge,
//                  device clock} into a caller-owned ring, so that after a wait that expired (or a run that never came
//                  back) the ring says which phase was reached and how long each one took on the device's own clock
//   poison         the rows a dispatch may write are filled with 0x7f bytes first (bf16 3.4e38, int8 127, the e4m3 NaN
//                  code, int32 2139062143), so a row that was counted but never written cannot pass for data
#include <hip/hip_runtime.h>

#include "ep_debug.h"
#include "ep_kernel_common.hip.h"

namespace TileXREp {
namespace {

__global__ void ep_debug_stamp_kernel(uint64_t *record, uint64_t magic, uint64_t kernelId, uint64_t edge)
{
    record[0] = magic;
    record[1] = kernelId;
    record[2] = edge;
    record[3] = wall_clock64();
}

__global__ __launch_bounds__(kThreads) void ep_debug_fill_kernel(uint32_t *words, int64_t count, uint32_t pattern)
{
    const int64_t stride = static_cast<int64_t>(gridDim.x) * kThreads;
    for (int64_t i = static_cast<int64_t>(blockIdx.x) * kThreads + threadIdx.x; i < count; i += stride) {
        words[i] = pattern;
    }
}

} // namespace

hipError_t LaunchDebugStamp(uint64_t *record, uint64_t magic, int kernelId, int edge, hipStream_t stream)
{
    hipLaunchKernelGGL(ep_debug_stamp_kernel, dim3(1), dim3(1), 0, stream, record, magic, static_cast<uint64_t>(kernelId),
        static_cast<uint64_t>(edge));
    return hipGetLastError();
}

hipError_t LaunchDebugPoison(void *base, int64_t bytes, hipStream_t stream)
{
    if (base == nullptr || bytes < 4) {
        return hipSuccess;
    }
    // whole 32-bit words; a buffer the caller aligned to less than four bytes is left alone (the data kernels do not
    // take such buffers through their vector paths either)
    if ((reinterpret_cast<uintptr_t>(base) & 3u) != 0) {
        return hipSuccess;
    }
    const int64_t words = bytes / 4;
    const int64_t blocks = (words + kThreads * 8 - 1) / (kThreads * 8);
    hipLaunchKernelGGL(ep_debug_fill_kernel, dim3(static_cast<unsigned>(blocks > 65536 ? 65536 : blocks)), dim3(kThreads), 0,
        stream, static_cast<uint32_t *>(base), words, kDebugPoisonWord);
    return hipGetLastError();
}

} // namespace TileXREp
