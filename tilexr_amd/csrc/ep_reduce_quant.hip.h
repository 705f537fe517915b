// reduce of quantised rows (int8 with a scale per row, fp8 e4m3 with a scale per 128 columns): ep_reduce.hip says what
// is computed.  Compiled once per (element type, readiness flags): the including file sets TILEXR_REDUCE_BF16,
// TILEXR_REDUCE_FLAGS and TILEXR_REDUCE_ENTRY.  TILEXR_REDUCE_FLAGS: 0 no flags; 1 flags that may still be pending
// (the launch can wait: tokens are claimed, rows and scales are read past the L2); 2 flags that were all published
// before the launch began (a dispatch earlier on the same stream): nothing waits, every wave only looks at the words
// of its token's tiles, and the kernel carries none of the waiting code -- with it in the same kernel the registers
// of the claim loop cost the fp8 kernel a wave per SIMD and the settled case ran 4 us behind the kernel without flags.
#if !defined(TILEXR_REDUCE_BF16) || !defined(TILEXR_REDUCE_FLAGS) || !defined(TILEXR_REDUCE_ENTRY)
#error "include from ep_reduce_quant_*.hip"
#endif

#include "ep_reduce_common.hip.h"

namespace TileXREp {
namespace {

// Quantised expert output: int8 rows with one fp32 scale per row, or fp8 e4m3 rows with one fp32 scale per 128
// columns.  Each value is dequantised, rounded to the output element type, then accumulated exactly like an ordinary
// row (fp32, k order, separate multiply and add).  Rows are a quarter the bytes of bf16 rows, so a lane owns 16
// consecutive columns per vector (one 16-byte load) and KB rows are kept in flight at once.
constexpr int kFlagsNone = 0;
constexpr int kFlagsMayWait = 1;
constexpr int kFlagsSettled = 2;

template <int G, int V, int INQ, bool BF16, int FL>
__global__ __launch_bounds__(kThreads, (V == 1 && BF16) ? ((FL == kFlagsMayWait && INQ == TILEXR_EP_QUANT_FP8_BLOCK128) ? 6 : 7) : 1) void ep_reduce_quant_kernel(ReduceArgs a)
{
    constexpr int kTokens = kThreads / G;
    constexpr int KB = V >= 4 ? 2 : 4;
    __shared__ int s_row[kTokens][kMaxTopK];
    __shared__ float s_w[kTokens][kMaxTopK];

    const int tg = threadIdx.x / G;
    const int lane = threadIdx.x % G;
    const int vecs = a.h / 16;
    const int groups = (a.bs + kTokens - 1) / kTokens;
    const int b128 = (a.h + 127) / 128;

    auto tokenAt = [&](int group, int t) {
        const int token = group * kTokens + t;
        return token < a.bs ? token : -1;
    };
    auto load = [&](int group, int mode) {
        const int token = group * kTokens + tg;
        return LoadRoutes<false>(a, token, token < a.bs, lane, G, s_row[tg], s_w[tg], mode);
    };
    auto reduceUnit = [&](int group) {
        const int token = group * kTokens + tg;
        const bool tokOk = token < a.bs;
        // Lane k of every wave keeps slot k's row and weight; the K loop takes the slots that have a row, in k order,
        // KB at a time.  Where tokens lose rows to an expert's capacity that is often one trip to memory, not two
        // (absent rows are skipped by the sum anyway, so the order of the additions is the same).
        static_assert(G % kWave == 0, "a wave works on one token");
        const int waveLane = threadIdx.x % kWave;
        int slotRow = -1;
        float myWeight = 0.0f;
        if (waveLane < a.slots) {
            slotRow = s_row[tg][waveLane];
            myWeight = s_w[tg][waveLane];
        }
        constexpr bool checkWords = FL == kFlagsSettled;
        const bool expired = FL == kFlagsMayWait && __ballot(slotRow == kRowExpired) != 0;
        const bool active = tokOk && (a.tokenMask == nullptr || a.tokenMask[token] != 0) && !expired;
        const int myRow = active ? slotRow : -1;
        // (an inactive token's output is zeros whatever its words say: only the rows that are read are asked about)
        const uint32_t tileWord = checkWords ? SettledWordLoad(a, myRow) : 0u;
        const uint64_t live = __ballot(myRow >= 0);

        float acc[V][16];
        // The K loop.  fp8 rows are decoded by the hardware convert alone, which differs from the reference decode in
        // one respect only (the sign of the NaN it returns for code 0x7f); a NaN code always surfaces as a NaN in the
        // sum, so a wave that finds a NaN among its sums runs the loop once more with the exact decode.  That keeps a
        // test of every word (four instructions and a branch per four values) out of the loop that everything else
        // shares.
        // throughMemory: rows and scales are read past this XCD's L2, as they must be while their producer may still
        // be writing neighbours of theirs.  Once the producer has finished (flagsSettled) the L2 is as good as memory,
        // and the scales, which the lanes of a token share, are worth keeping there (4096 x int8 rows: 58 -> 49 us).
        auto accumulate = [&](auto exactDecode, auto throughMemory) {
            constexpr bool kExactDecode = decltype(exactDecode)::value;
            constexpr bool kThroughMemory = decltype(throughMemory)::value;
#pragma unroll
            for (int j = 0; j < V; ++j) {
#pragma unroll
                for (int e = 0; e < 16; ++e) {
                    acc[j][e] = 0.0f;
                }
            }
            uint64_t todo = live;
            while (todo != 0) {
                u32x4 q[KB][V];
                float sc[KB][V];
                int rowOfK[KB];
                float weightOfK[KB];
#pragma unroll
                for (int u = 0; u < KB; ++u) {
                    const bool any = todo != 0;
                    const int k = any ? __builtin_ctzll(todo) : 0;
                    todo &= todo - 1;
                    const int row = any ? __builtin_amdgcn_readlane(myRow, k) : -1;
                    rowOfK[u] = row;
                    weightOfK[u] = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(myWeight), k));
                    // Bounds are the buffer resources' business: an absent row gets resources of zero bytes, so its loads, like
                    // those of the lanes past the end of a row, return zeros without a branch (and without the register
                    // clears a branch would need).
                    const int64_t rowAt = row < 0 ? 0 : row;
                    const char *base = static_cast<const char *>(a.expertOut) + rowAt * a.rowBytes;
                    const __amdgpu_buffer_rsrc_t rsrc = RowResource(base, row < 0 ? 0 : vecs * 16);
                    const bool perRow = INQ == TILEXR_EP_QUANT_TOKEN_INT8;
                    const float *scaleBase = a.inScales + (perRow ? rowAt : rowAt * b128);
                    const __amdgpu_buffer_rsrc_t scaleRsrc = RowResource(scaleBase, row < 0 ? 0 : (perRow ? 4 : b128 * 4));
#pragma unroll
                    for (int j = 0; j < V; ++j) {
                        const int idx = j * G + lane;
                        q[u][j] = __builtin_amdgcn_raw_buffer_load_b128(rsrc, idx * 16, 0,
                            kThroughMemory ? kAuxAgentScope : kAuxNonTemporal);
                        sc[u][j] = __uint_as_float(__builtin_amdgcn_raw_buffer_load_b32(scaleRsrc, perRow ? 0 : (idx >> 3) * 4, 0,
                            kThroughMemory ? kAuxAgentScope : 0));
                    }
                }
#pragma unroll
                for (int u = 0; u < KB; ++u) {
                    if (rowOfK[u] < 0) {
                        continue;                       // uniform across the lanes of a token
                    }
                    const float w = weightOfK[u];
#pragma unroll
                    for (int j = 0; j < V; ++j) {
#pragma unroll
                        for (int d = 0; d < 4; ++d) {
                            const uint32_t word = q[u][j][d];
                            float f[4];
                            if (INQ == TILEXR_EP_QUANT_TOKEN_INT8) {
#pragma unroll
                                for (int e = 0; e < 4; ++e) {
                                    f[e] = static_cast<float>(static_cast<int>(static_cast<int8_t>((word >> (8 * e)) & 0xffu)));
                                }
                            } else if (kExactDecode) {
                                Fp8E4m3DecodeWord(word, f);
                            } else {
                                Fp8E4m3DecodeWordFast(word, f);
                            }
#pragma unroll
                            for (int e = 0; e < 4; e += 2) {
                                const float d0 = __fmul_rn(f[e], sc[u][j]);
                                const float d1 = __fmul_rn(f[e + 1], sc[u][j]);
                                float r0;
                                float r1;
                                if (BF16) {
                                    r0 = FloatRoundedToBf16(d0);
                                    r1 = FloatRoundedToBf16(d1);
                                } else {
                                    r0 = __half2float(__ushort_as_half(static_cast<unsigned short>(FloatToHalfRneSat(d0))));
                                    r1 = __half2float(__ushort_as_half(static_cast<unsigned short>(FloatToHalfRneSat(d1))));
                                }
                                acc[j][4 * d + e] = __fadd_rn(acc[j][4 * d + e], __fmul_rn(r0, w));
                                acc[j][4 * d + e + 1] = __fadd_rn(acc[j][4 * d + e + 1], __fmul_rn(r1, w));
                            }
                        }
                    }
                }
            }
        };
        constexpr bool throughMemory = FL == kFlagsMayWait;
        if (throughMemory) {
            accumulate(std::false_type {}, std::true_type {});
        } else {
            accumulate(std::false_type {}, std::false_type {});
        }
        if (INQ == TILEXR_EP_QUANT_FP8_BLOCK128) {
            bool sawNan = false;
#pragma unroll
            for (int j = 0; j < V; ++j) {
#pragma unroll
                for (int e = 0; e < 16; ++e) {
                    sawNan |= acc[j][e] != acc[j][e];
                }
            }
            if (__any(sawNan ? 1 : 0)) {
                if (throughMemory) {
                    accumulate(std::true_type {}, std::true_type {});
                } else {
                    accumulate(std::true_type {}, std::false_type {});
                }
            }
        }
        if (a.sharedExpertX != nullptr && active) {
            const u32x4 *sx = reinterpret_cast<const u32x4 *>(static_cast<const char *>(a.sharedExpertX) +
                static_cast<int64_t>(token) * a.h * 2);
#pragma unroll
            for (int j = 0; j < V; ++j) {
                const int idx = j * G + lane;
                if (idx < vecs) {
#pragma unroll
                    for (int half = 0; half < 2; ++half) {
                        const u32x4 v = sx[idx * 2 + half];
#pragma unroll
                        for (int q2 = 0; q2 < 4; ++q2) {
                            float &lo = acc[j][half * 8 + 2 * q2];
                            float &hi = acc[j][half * 8 + 2 * q2 + 1];
                            lo = __fadd_rn(lo, Decode16<BF16>(v[q2] & 0xffffu));
                            hi = __fadd_rn(hi, Decode16<BF16>(v[q2] >> 16));
                        }
                    }
                }
            }
        }
        const bool keep = active && !(checkWords && SettledWordMissing(a, myRow, tileWord, waveLane));
        if (tokOk) {
            u32x4 *dst = reinterpret_cast<u32x4 *>(static_cast<char *>(a.y) + static_cast<int64_t>(token) * a.h * 2);
            // the lane index once more, from the thread index and out of the optimiser's sight: values derived from it
            // for these stores are then computed here instead of being kept (or spilled) across the K loop, where every
            // register counts towards the seventh wave per SIMD
            int storeThread = threadIdx.x;
            asm volatile("" : "+v"(storeThread));
            const int storeLane = storeThread % G;
#pragma unroll
            for (int j = 0; j < V; ++j) {
                const int idx = j * G + storeLane;
                if (idx < vecs) {
#pragma unroll
                    for (int half = 0; half < 2; ++half) {
                        u32x4 o;
#pragma unroll
                        for (int q2 = 0; q2 < 4; ++q2) {
                            o[q2] = keep ? EncodePair16Sat<BF16>(acc[j][half * 8 + 2 * q2], acc[j][half * 8 + 2 * q2 + 1]) : 0u;
                        }
                        // An ordinary store, not a streaming one: a lane's 32 bytes go out as two 16-byte stores, each
                        // of which fills every other 16 bytes of the lines it touches; the L2 puts the halves together
                        // before they go to memory (4096-column int8 rows: 46.3 us, 48.4 us with streaming stores;
                        // trading halves between lanes so that each store covers whole lines: 46.8 us).
                        dst[idx * 2 + half] = o;
                    }
                }
            }
        }
    };
    ForEachGroup<FL == kFlagsMayWait>(a, groups, kTokens, tokenAt, load, reduceUnit);
}


template <int G, int V, bool BF16, int FL>
void LaunchQuant(const ReduceLaunch &l, const ReduceArgs &a, int gridLimit)
{
    constexpr int kTokens = kThreads / G;
    int grid = (a.bs + kTokens - 1) / kTokens;
    if (gridLimit > 0 && grid > gridLimit) {
        grid = gridLimit;
    }
    const dim3 g(grid);
    const dim3 b(kThreads);
    if (l.inQuant == TILEXR_EP_QUANT_TOKEN_INT8) {
        hipLaunchKernelGGL((ep_reduce_quant_kernel<G, V, TILEXR_EP_QUANT_TOKEN_INT8, BF16, FL>), g, b, 0, l.stream, a);
    } else {
        hipLaunchKernelGGL((ep_reduce_quant_kernel<G, V, TILEXR_EP_QUANT_FP8_BLOCK128, BF16, FL>), g, b, 0, l.stream, a);
    }
}

} // namespace

void TILEXR_REDUCE_ENTRY(int g, int v, const ReduceLaunch &l, const ReduceArgs &a, int gridLimit)
{
    constexpr bool kBf16 = TILEXR_REDUCE_BF16;
    constexpr int kFlags = TILEXR_REDUCE_FLAGS;
    if (g == kWave && v == 1) {
        LaunchQuant<kWave, 1, kBf16, kFlags>(l, a, gridLimit);
    } else if (g == 2 * kWave && v == 1) {
        LaunchQuant<2 * kWave, 1, kBf16, kFlags>(l, a, gridLimit);
    } else if (g == kThreads && v == 1) {
        LaunchQuant<kThreads, 1, kBf16, kFlags>(l, a, gridLimit);
    } else if (g == kThreads && v == 2) {
        LaunchQuant<kThreads, 2, kBf16, kFlags>(l, a, gridLimit);
    } else if (g == kThreads && v == 4) {
        LaunchQuant<kThreads, 4, kBf16, kFlags>(l, a, gridLimit);
    }
}

} // namespace TileXREp
