// Per-GPU static scratch of the entry point that allocates nothing (internal header, see ep_static_scratch.hip).
#ifndef TILEXR_AMD_EP_STATIC_SCRATCH_H
#define TILEXR_AMD_EP_STATIC_SCRATCH_H

#include <cstddef>
#include <cstdint>

#include <hip/hip_runtime_api.h>

namespace TileXREp {

// Size of the array every GPU holds from the moment the library is loaded until the process ends.  It covers the
// count scratch of 131 072 routes (bs * topK) over up to 2048 experts (8.3 bytes per route + 264 bytes per expert and
// 1024-route chunk + a few hundred bytes); larger calls are rejected, not served from elsewhere.
constexpr size_t kStaticScratchBytes = size_t{2} << 20;

// Resolves the device address of the array on `device`, which must be the current device.  Once per device; later
// calls return at once.
hipError_t ResolveStaticScratch(int device);

// The address resolved for `device`, or nullptr when ResolveStaticScratch has not succeeded there.
void *StaticScratchOnDevice(int device);

// Stores 0 to one 32-bit word of the scratch with a one-thread kernel on `stream`.
hipError_t ClearScratchWord(void *word, hipStream_t stream);

} // namespace TileXREp

#endif // TILEXR_AMD_EP_STATIC_SCRATCH_H
