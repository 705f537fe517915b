// Scratch for the entry point that allocates nothing: one file-scope device array per GPU instead of hipMalloc.
//
// Some callers cannot allocate device memory at call time (a stream under graph capture, a serving loop that has
// handed all memory to its own pool, a harness that forbids hipMalloc).  TileXRMoeEpDispatchMemoryNoAlloc gives its
// count / place / scatter kernels this array where the ordinary entry point gives them a buffer from hipMalloc.
//
// The array's name is only a host-side stand-in for the device symbol, not a device address: every GPU the library
// runs on holds its own copy at its own address, which hipGetSymbolAddress reports for the current device.  That
// address -- never the name -- is what kernels, fills and copies are given.  It is resolved once per device, when a
// communicator is created on that device (the library's set-up call), with that device current.
//
// All calls on one GPU share the one array: it keeps the previous call's contents, and two calls that overlap in time
// on one GPU would race on it.
#include <hip/hip_runtime.h>

#include <mutex>

#include "ep_static_scratch.h"

namespace TileXREp {
namespace {

static __device__ __align__(256) unsigned char scratch[kStaticScratchBytes];

constexpr int kMaxDevices = 64;
std::mutex gMutex;
void *gScratchOnDevice[kMaxDevices] = {};

__global__ void ep_clear_word_kernel(uint32_t *word)
{
    *word = 0u;
}

} // namespace

hipError_t ResolveStaticScratch(int device)
{
    if (device < 0 || device >= kMaxDevices) {
        return hipErrorInvalidDevice;
    }
    std::lock_guard<std::mutex> lock(gMutex);
    if (gScratchOnDevice[device] != nullptr) {
        return hipSuccess;
    }
    int current = -1;
    hipError_t err = hipGetDevice(&current);
    if (err != hipSuccess) {
        return err;
    }
    if (current != device) {
        return hipErrorInvalidDevice;       // the address is the current device's: the caller makes `device` current
    }
    void *ptr = nullptr;
    err = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch));
    if (err != hipSuccess) {
        return err;
    }
    gScratchOnDevice[device] = ptr;
    return hipSuccess;
}

void *StaticScratchOnDevice(int device)
{
    if (device < 0 || device >= kMaxDevices) {
        return nullptr;
    }
    std::lock_guard<std::mutex> lock(gMutex);
    return gScratchOnDevice[device];
}

hipError_t ClearScratchWord(void *word, hipStream_t stream)
{
    // a kernel, not hipMemsetAsync: the call may be recorded into a graph, where memset nodes are best avoided
    hipLaunchKernelGGL(ep_clear_word_kernel, dim3(1), dim3(1), 0, stream, static_cast<uint32_t *>(word));
    return hipGetLastError();
}

} // namespace TileXREp
