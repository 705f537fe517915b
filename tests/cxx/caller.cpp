// A C++ caller written against the installed headers only, the way the reference's demo is
// (reference: tests/ep/demo/tilexr_ep_dispatch_demo.cpp:1289-1300, 1463-1496): create a communicator, make the
// calls, destroy it.  It runs without a GPU: every call below must be turned away by the host-side checks, in the
// reference's order (arguments, communicator, configuration) and with the reference's status codes, before anything
// could reach a device.  Exit status 0 = all expectations held.
#include <cstdint>
#include <cstdio>

#include "tilexr_api.h"
#include "tilexr_ep.h"

namespace {

int failures = 0;

void Expect(int got, int want, const char *what)
{
    if (got != want) {
        std::printf("FAIL %s: got %d, want %d\n", what, got, want);
        ++failures;
    }
}

} // namespace

int main()
{
    using TileXR::TILEXR_DATA_TYPE_BFP16;
    using TileXR::TILEXR_DATA_TYPE_RESERVED;
    TileXRCommPtr comm = nullptr;
    Expect(TileXRCommInitRankLocal(1, 0, &comm), TileXR::TILEXR_SUCCESS, "TileXRCommInitRankLocal");
    int64_t magic = 0;
    Expect(TileXRCommNextMagic(comm, &magic), TileXR::TILEXR_SUCCESS, "TileXRCommNextMagic");
    Expect(static_cast<int>(magic), 1, "first magic");

    void *fake = reinterpret_cast<void *>(0x1000);
    int32_t *fakeI32 = reinterpret_cast<int32_t *>(0x1000);
    int64_t *fakeI64 = reinterpret_cast<int64_t *>(0x1000);
    aclrtStream stream = fake;

    // null tensor -> parameter check, whatever else is wrong
    Expect(TileXRMoeEpDispatch(nullptr, fakeI32, comm, 4, 8, 2, 8, fake, fakeI64, fakeI32, fakeI32, TILEXR_DATA_TYPE_BFP16,
               stream), TileXR::TILEXR_ERROR_PARA_CHECK_FAIL, "dispatch: null x");
    Expect(TileXRMoeEpDispatchMemory(fake, fakeI32, comm, 0, 8, 2, 8, fake, fakeI64, fakeI32, fakeI32,
               TILEXR_DATA_TYPE_BFP16, stream), TileXR::TILEXR_ERROR_PARA_CHECK_FAIL, "memory dispatch: bs = 0");
    Expect(TileXRMoeEpCombine(fake, fakeI32, fakeI32, comm, 4, 8, 2, 8, fake, TILEXR_DATA_TYPE_BFP16, nullptr),
        TileXR::TILEXR_ERROR_PARA_CHECK_FAIL, "combine: null stream");
    Expect(TileXRMoeEpCombineMemory(fake, fakeI32, fakeI32, nullptr, 4, 8, 2, 8, fake, TILEXR_DATA_TYPE_BFP16, stream),
        TileXR::TILEXR_ERROR_PARA_CHECK_FAIL, "memory combine: null comm");
    // a handle nobody created
    Expect(TileXRMoeEpDispatchMemoryV2(fake, fakeI32, nullptr, nullptr, 0, nullptr, fake, 4, 8, 2, 8, 0, 0, 1, 0, 0, 0, 0,
               0, 0, 1, fake, nullptr, fakeI32, fakeI64, fakeI32, nullptr, nullptr, TILEXR_DATA_TYPE_BFP16,
               TILEXR_DATA_TYPE_RESERVED, stream), TileXR::TILEXR_ERROR_NOT_INITIALIZED, "memory dispatch V2: unknown comm");
    Expect(TileXRMoeEpCombineMemoryV2(fake, fakeI32, fakeI32, nullptr, nullptr, 0, nullptr, fake, 4, 8, 2, 8, 0, 0, 1, 0,
               0, 0, 0, 0, 0, fake, TILEXR_DATA_TYPE_BFP16, stream), TileXR::TILEXR_ERROR_NOT_INITIALIZED,
        "memory combine V2: unknown comm");
    Expect(TileXRMoeEpDispatchV2(fake, fakeI32, nullptr, nullptr, nullptr, fake, 4, 8, 2, 8, 0, 0, 0, 0, 0, 0, 0, 0, 0, 1,
               fake, nullptr, fakeI32, fakeI64, fakeI32, nullptr, nullptr, nullptr, TILEXR_DATA_TYPE_BFP16, stream),
        TileXR::TILEXR_ERROR_NOT_INITIALIZED, "dispatch V2: unknown comm");
    Expect(TileXRMoeEpCombineV2(fake, fakeI32, fakeI32, fake, 4, 8, 2, 8, fake, nullptr, TILEXR_DATA_TYPE_BFP16, stream),
        TileXR::TILEXR_ERROR_NOT_INITIALIZED, "combine V2: unknown comm");
    // rejected calls draw no magic
    Expect(TileXRCommNextMagic(comm, &magic), TileXR::TILEXR_SUCCESS, "TileXRCommNextMagic");
    Expect(static_cast<int>(magic), 2, "second magic");
    Expect(TileXRCommDestroy(comm), TileXR::TILEXR_SUCCESS, "TileXRCommDestroy");
    Expect(TileXRCommDestroy(comm), TileXR::TILEXR_ERROR_PARA_CHECK_FAIL, "TileXRCommDestroy twice");
    std::printf("%s\n", failures == 0 ? "caller ok" : "caller FAILED");
    return failures == 0 ? 0 : 1;
}
