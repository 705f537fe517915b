// Exhaustive check of DivideByShared (tilexr_amd/csrc/ep_numerics.hip.h) against the correctly rounded division, on the
// pairs the block fp8 quantiser of the scatter can meet: every 16-bit element pattern x (bf16 or fp16, NaNs and
// infinities included) with every non-negative block maximum amax of the same type, scale = amax / 448 (1 for amax = 0)
// as the quantiser forms it.  Test infrastructure: built by tilexr_amd/csrc/Makefile into
// tests/cxx/bin/shared_division_check and run by tests/test_gpu_shared_division.py.
//
//   shared_division_check <bf16|fp16> [all]
//
// Prints, per exponent field of the scale, the pairs on which the e4m3 codes differ and those on which the quotients
// differ in any bit (NaNs count as equal when their signs agree: the encoder that follows looks at nothing else).
// Passes when no code differs: the quotient feeds the encoder and nothing else.  (The short form leaves out the second
// correction of the long one, so a quotient can be off in its last place; the run shows that no such quotient sits close
// enough to a rounding boundary of e4m3 to change a code.)  Without "all" only divisors that SharedReciprocalHolds accepts
// are tried with the short form, as in the kernel; with "all" the short form is tried on every divisor, which is how the
// accepted range was found.
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <cstring>

#include <hip/hip_runtime.h>

#include "ep_numerics.hip.h"

namespace {

using namespace TileXREp;

struct Tally {
    unsigned long long pairs[256];
    unsigned long long quotient[256];
    unsigned long long code[256];
    unsigned int firstX;
    unsigned int firstMax;
    unsigned int haveFirst;
    unsigned int largestMissedBits;      // bits of the largest |correct quotient| the short form did not reproduce
};

template <bool BF16>
__global__ __launch_bounds__(256) void check_kernel(Tally *tally, int tryAll)
{
    const uint32_t maxBits = blockIdx.x;                 // 0 .. 0x7fff: sign bit clear
    const float amax = Decode16<BF16>(maxBits);
    // the quantiser's block maximum comes out of fmaxf over |x|: never a NaN
    if (amax != amax) {
        return;
    }
    const float sc = amax > 0.0f ? __fdiv_rn(amax, 448.0f) : 1.0f;
    const uint32_t exponent = (__float_as_uint(sc) >> 23) & 0xffu;
    const bool shortForm = tryAll != 0 || SharedReciprocalHolds(sc);
    const float y = SharedReciprocal(sc);
    unsigned long long pairs = 0, badQ = 0, badCode = 0;
    for (uint32_t xBits = threadIdx.x; xBits < 0x10000u; xBits += blockDim.x) {
        const float x = Decode16<BF16>(xBits);
        // within a block no |x| exceeds the maximum; a NaN does not take part in it
        if (x == x && fabsf(x) > amax) {
            continue;
        }
        const float want = __fdiv_rn(x, sc);
        const float got = shortForm ? DivideByShared(x, sc, y) : want;
        ++pairs;
        const uint32_t wb = __float_as_uint(want);
        const uint32_t gb = __float_as_uint(got);
        const bool bothNan = want != want && got != got;
        const bool sameQ = bothNan ? ((wb ^ gb) >> 31) == 0u : wb == gb;
        const bool sameCode = (Fp8E4m3EncodePairSat(want, 0.0f) & 0xffu) == (Fp8E4m3EncodePairSat(got, 0.0f) & 0xffu);
        if (!sameQ) {
            ++badQ;
            atomicMax(&tally->largestMissedBits, want != want ? 0x7fc00000u : (wb & 0x7fffffffu));
        }
        if (!sameCode) {
            ++badCode;
            if (atomicExch(&tally->haveFirst, 1u) == 0u) {
                tally->firstX = xBits;
                tally->firstMax = maxBits;
            }
        }
    }
    atomicAdd(&tally->pairs[exponent], pairs);
    atomicAdd(&tally->quotient[exponent], badQ);
    atomicAdd(&tally->code[exponent], badCode);
}

#define HIP_OK(call)                                                                                  \
    do {                                                                                              \
        hipError_t e_ = (call);                                                                       \
        if (e_ != hipSuccess) {                                                                       \
            std::fprintf(stderr, "%s failed: %s\n", #call, hipGetErrorString(e_));                    \
            std::exit(2);                                                                             \
        }                                                                                             \
    } while (0)

} // namespace

int main(int argc, char **argv)
{
    if (argc < 2 || (std::strcmp(argv[1], "bf16") != 0 && std::strcmp(argv[1], "fp16") != 0)) {
        std::fprintf(stderr, "usage: shared_division_check <bf16|fp16> [all]\n");
        return 2;
    }
    const bool bf16 = std::strcmp(argv[1], "bf16") == 0;
    const int tryAll = argc > 2 && std::strcmp(argv[2], "all") == 0 ? 1 : 0;
    HIP_OK(hipSetDevice(0));
    Tally *dev = nullptr;
    HIP_OK(hipMalloc(&dev, sizeof(Tally)));
    HIP_OK(hipMemset(dev, 0, sizeof(Tally)));
    if (bf16) {
        hipLaunchKernelGGL(check_kernel<true>, dim3(0x8000), dim3(256), 0, nullptr, dev, tryAll);
    } else {
        hipLaunchKernelGGL(check_kernel<false>, dim3(0x8000), dim3(256), 0, nullptr, dev, tryAll);
    }
    HIP_OK(hipGetLastError());
    HIP_OK(hipDeviceSynchronize());
    Tally host;
    HIP_OK(hipMemcpy(&host, dev, sizeof(Tally), hipMemcpyDeviceToHost));
    HIP_OK(hipFree(dev));
    unsigned long long pairs = 0, badQ = 0, badCode = 0;
    for (int e = 0; e < 256; ++e) {
        pairs += host.pairs[e];
        badQ += host.quotient[e];
        badCode += host.code[e];
        if (host.quotient[e] != 0 || host.code[e] != 0) {
            std::printf("scale exponent field %3d: %llu pairs, %llu quotients differ, %llu codes differ\n", e, host.pairs[e],
                host.quotient[e], host.code[e]);
        }
    }
    if (host.haveFirst != 0) {
        std::printf("first differing code: x bits 0x%04x, maximum bits 0x%04x\n", host.firstX, host.firstMax);
    }
    float largestMissed;
    std::memcpy(&largestMissed, &host.largestMissedBits, sizeof(float));
    const bool ok = badCode == 0;
    std::printf("%s %s: %llu pairs, %llu codes differ, %llu quotients differ (largest %.9g)\n", ok ? "OK" : "DIFF", argv[1], pairs,
        badCode, badQ, static_cast<double>(largestMissed));
    return ok ? 0 : 1;
}
