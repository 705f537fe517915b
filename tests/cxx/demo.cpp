// A caller of libtilexr-ep written the way the reference's own demo is (tests/ep/demo/tilexr_ep_dispatch_demo.cpp:
// allocate, dispatch, identity expert, combine, compare with a host model): plain C++ against include/ and the HIP
// runtime, no Python and no torch anywhere.  Test infrastructure: built by tilexr_amd/csrc/Makefile into
// tests/cxx/bin/demo and run by tests/test_gpu_cxx_demo.py.
//
//   demo <bs> <h> <topK> <experts>
//
// Routing: token t picks experts (t + k * (experts / topK)) % experts, k = 0 .. topK-1 (distinct).  x[t][c] is a small
// integer, exact in bf16, so that the unweighted combine of the memory route has to return topK * x exactly.
#include <chrono>
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <vector>

#include <hip/hip_runtime_api.h>

#include "tilexr_api.h"
#include "tilexr_ep.h"

namespace {

#define HIP_OK(call)                                                                                  \
    do {                                                                                              \
        hipError_t e_ = (call);                                                                       \
        if (e_ != hipSuccess) {                                                                       \
            std::fprintf(stderr, "%s failed: %s\n", #call, hipGetErrorString(e_));                    \
            std::exit(2);                                                                             \
        }                                                                                             \
    } while (0)

uint16_t Bf16OfSmallInt(int v)
{
    const float f = static_cast<float>(v);
    uint32_t bits;
    static_assert(sizeof(bits) == sizeof(f), "float is 32 bits");
    __builtin_memcpy(&bits, &f, 4);
    return static_cast<uint16_t>(bits >> 16);      // |v| <= 128: the low 16 bits are zero
}

int Fail(const char *what, long long at, long long got, long long want)
{
    std::fprintf(stderr, "MISMATCH %s at %lld: got %lld, want %lld\n", what, at, got, want);
    return 1;
}

} // namespace

int main(int argc, char **argv)
{
    if (argc != 5 && argc != 6) {
        std::fprintf(stderr, "usage: demo <bs> <h> <topK> <experts> [layers timed back to back after the check]\n");
        return 2;
    }
    const int64_t timedLayers = argc == 6 ? std::atoll(argv[5]) : 0;
    const int64_t bs = std::atoll(argv[1]);
    const int64_t h = std::atoll(argv[2]);
    const int64_t topK = std::atoll(argv[3]);
    const int64_t experts = std::atoll(argv[4]);
    if (bs <= 0 || h <= 0 || topK <= 0 || experts < topK || topK > 15) {
        std::fprintf(stderr, "bad shape\n");
        return 2;
    }
    const int64_t n = bs * topK;
    const int64_t step = experts / topK;

    std::vector<uint16_t> x(static_cast<size_t>(bs * h));
    std::vector<int32_t> ids(static_cast<size_t>(n));
    for (int64_t t = 0; t < bs; ++t) {
        for (int64_t c = 0; c < h; ++c) {
            x[static_cast<size_t>(t * h + c)] = Bf16OfSmallInt(static_cast<int>((t * 3 + c * 5) % 17) - 8);
        }
        for (int64_t k = 0; k < topK; ++k) {
            ids[static_cast<size_t>(t * topK + k)] = static_cast<int32_t>((t + k * step) % experts);
        }
    }

    HIP_OK(hipSetDevice(0));
    hipStream_t stream;
    HIP_OK(hipStreamCreate(&stream));
    TileXRCommPtr comm = nullptr;
    if (TileXRCommInitRankLocal(1, 0, &comm) != 0 || comm == nullptr) {
        std::fprintf(stderr, "TileXRCommInitRankLocal failed\n");
        return 2;
    }

    void *dX, *dIds, *dExpand, *dTokenNums, *dCounts, *dAssist, *dY;
    HIP_OK(hipMalloc(&dX, x.size() * 2));
    HIP_OK(hipMalloc(&dIds, ids.size() * 4));
    HIP_OK(hipMalloc(&dExpand, static_cast<size_t>(n * h * 2)));
    HIP_OK(hipMalloc(&dTokenNums, static_cast<size_t>(experts * 8)));
    HIP_OK(hipMalloc(&dCounts, static_cast<size_t>(experts * 4)));
    HIP_OK(hipMalloc(&dAssist, static_cast<size_t>(n * 16)));
    HIP_OK(hipMalloc(&dY, x.size() * 2));
    HIP_OK(hipMemcpy(dX, x.data(), x.size() * 2, hipMemcpyHostToDevice));
    HIP_OK(hipMemcpy(dIds, ids.data(), ids.size() * 4, hipMemcpyHostToDevice));
    HIP_OK(hipMemset(dExpand, 0x5a, static_cast<size_t>(n * h * 2)));
    HIP_OK(hipMemset(dY, 0x5a, x.size() * 2));

    int st = TileXRMoeEpDispatchMemory(dX, static_cast<int32_t *>(dIds), comm, bs, h, topK, experts, dExpand,
        static_cast<int64_t *>(dTokenNums), static_cast<int32_t *>(dCounts), static_cast<int32_t *>(dAssist),
        TileXR::TILEXR_DATA_TYPE_BFP16, stream);
    if (st != 0) {
        std::fprintf(stderr, "TileXRMoeEpDispatchMemory returned %d\n", st);
        return 1;
    }
    // identity expert: combine reads the rows dispatch wrote
    st = TileXRMoeEpCombineMemory(dExpand, static_cast<int32_t *>(dAssist), static_cast<int32_t *>(dCounts), comm, bs, h,
        topK, experts, dY, TileXR::TILEXR_DATA_TYPE_BFP16, stream);
    if (st != 0) {
        std::fprintf(stderr, "TileXRMoeEpCombineMemory returned %d\n", st);
        return 1;
    }
    HIP_OK(hipStreamSynchronize(stream));

    std::vector<int32_t> counts(static_cast<size_t>(experts));
    std::vector<int64_t> tokenNums(static_cast<size_t>(experts));
    std::vector<int32_t> assist(static_cast<size_t>(n * 4));
    std::vector<uint16_t> expand(static_cast<size_t>(n * h));
    std::vector<uint16_t> y(x.size());
    HIP_OK(hipMemcpy(counts.data(), dCounts, counts.size() * 4, hipMemcpyDeviceToHost));
    HIP_OK(hipMemcpy(tokenNums.data(), dTokenNums, tokenNums.size() * 8, hipMemcpyDeviceToHost));
    HIP_OK(hipMemcpy(assist.data(), dAssist, assist.size() * 4, hipMemcpyDeviceToHost));
    HIP_OK(hipMemcpy(expand.data(), dExpand, expand.size() * 2, hipMemcpyDeviceToHost));
    HIP_OK(hipMemcpy(y.data(), dY, y.size() * 2, hipMemcpyDeviceToHost));

    // host model of the memory route (reference: tests/ep/demo/tilexr_ep_dispatch_demo.cpp:745-792): rows ordered by
    // expert, within an expert by flat route index; sendCounts is the inclusive running total
    std::vector<int64_t> perExpert(static_cast<size_t>(experts), 0);
    for (int64_t i = 0; i < n; ++i) {
        ++perExpert[static_cast<size_t>(ids[static_cast<size_t>(i)])];
    }
    std::vector<int64_t> firstRow(static_cast<size_t>(experts), 0);
    int64_t run = 0;
    for (int64_t e = 0; e < experts; ++e) {
        firstRow[static_cast<size_t>(e)] = run;
        run += perExpert[static_cast<size_t>(e)];
        if (counts[static_cast<size_t>(e)] != run) {
            return Fail("sendCounts", e, counts[static_cast<size_t>(e)], run);
        }
        // expertTokenNums: the count per expert (reference: tilexr_ep_dispatch_memory_kernel.h:1159-1168, type 1)
        if (tokenNums[static_cast<size_t>(e)] != perExpert[static_cast<size_t>(e)]) {
            return Fail("expertTokenNums", e, tokenNums[static_cast<size_t>(e)], perExpert[static_cast<size_t>(e)]);
        }
    }
    std::vector<int64_t> next = firstRow;
    for (int64_t i = 0; i < n; ++i) {
        const int64_t e = ids[static_cast<size_t>(i)];
        const int64_t row = next[static_cast<size_t>(e)]++;
        const int32_t *tuple = &assist[static_cast<size_t>(row * 4)];
        const int64_t want[4] = {0, i / topK, i % topK, e};
        for (int f = 0; f < 4; ++f) {
            if (tuple[f] != want[f]) {
                return Fail("assist tuple", row * 4 + f, tuple[f], want[f]);
            }
        }
        for (int64_t c = 0; c < h; ++c) {
            const uint16_t got = expand[static_cast<size_t>(row * h + c)];
            const uint16_t src = x[static_cast<size_t>((i / topK) * h + c)];
            if (got != src) {
                return Fail("expandX", row * h + c, got, src);
            }
        }
    }
    for (int64_t t = 0; t < bs; ++t) {
        for (int64_t c = 0; c < h; ++c) {
            const int v = (static_cast<int>((t * 3 + c * 5) % 17) - 8) * static_cast<int>(topK);
            // |v| <= 120: exact in bf16; -0 and +0 both stand for zero
            const uint16_t want = Bf16OfSmallInt(v);
            const uint16_t got = y[static_cast<size_t>(t * h + c)];
            if (got != want && !(v == 0 && (got & 0x7fffu) == 0)) {
                return Fail("y", t * h + c, got, want);
            }
        }
    }

    // the same two calls per layer as a serving loop makes them: no synchronisation between layers, so a layer costs
    // whichever is longer, the host's two calls or the device's kernels
    double usPerLayer = 0.0;
    if (timedLayers > 0) {
        for (int pass = 0; pass < 2; ++pass) {     // the first pass warms up
            HIP_OK(hipStreamSynchronize(stream));
            const auto t0 = std::chrono::steady_clock::now();
            for (int64_t l = 0; l < timedLayers; ++l) {
                st = TileXRMoeEpDispatchMemory(dX, static_cast<int32_t *>(dIds), comm, bs, h, topK, experts, dExpand,
                    static_cast<int64_t *>(dTokenNums), static_cast<int32_t *>(dCounts), static_cast<int32_t *>(dAssist),
                    TileXR::TILEXR_DATA_TYPE_BFP16, stream);
                if (st == 0) {
                    st = TileXRMoeEpCombineMemory(dExpand, static_cast<int32_t *>(dAssist), static_cast<int32_t *>(dCounts),
                        comm, bs, h, topK, experts, dY, TileXR::TILEXR_DATA_TYPE_BFP16, stream);
                }
                if (st != 0) {
                    std::fprintf(stderr, "timed layer %lld returned %d\n", static_cast<long long>(l), st);
                    return 1;
                }
            }
            HIP_OK(hipStreamSynchronize(stream));
            const auto t1 = std::chrono::steady_clock::now();
            usPerLayer = std::chrono::duration<double, std::micro>(t1 - t0).count() / static_cast<double>(timedLayers);
        }
    }

    TileXRCommDestroy(comm);
    HIP_OK(hipFree(dX));
    HIP_OK(hipFree(dIds));
    HIP_OK(hipFree(dExpand));
    HIP_OK(hipFree(dTokenNums));
    HIP_OK(hipFree(dCounts));
    HIP_OK(hipFree(dAssist));
    HIP_OK(hipFree(dY));
    HIP_OK(hipStreamDestroy(stream));
    std::printf("OK bs=%lld h=%lld topK=%lld experts=%lld rows=%lld", static_cast<long long>(bs), static_cast<long long>(h),
        static_cast<long long>(topK), static_cast<long long>(experts), static_cast<long long>(n));
    if (timedLayers > 0) {
        std::printf(" layers=%lld us_per_layer=%.2f", static_cast<long long>(timedLayers), usPerLayer);
    }
    std::printf("\n");
    return 0;
}
