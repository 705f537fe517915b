// reduce: y[token] = sum over the token's rows, gathered through the inverse map (gfx950, wave64).
//
// HBM-bound: topK row reads per output row, < 0.5 FLOP per byte, no MFMA.  G lanes cooperate on one token and keep
// V x 8 fp32 accumulators in registers; for each route in k order a lane issues all V of its 128-bit non-temporal
// loads of that row before touching the accumulators, so 64-128 bytes per lane are in flight while the previous
// row is being summed.  Measured on MI355X this moves 4096 x 7168 bf16 x top-8 (529 MB) at about 6 TB/s.
//
//   KIND fp32     sum = 0; for k = 0..K-1: sum = sum + (w_k * row_k) in fp32 (separate multiply and add), then the
//                 shared-expert row, then one round-to-nearest-even (saturating for fp16) to the output type;
//                 an inactive token (mask) gives zeros
//                 (reference: src/ep/kernels/tilexr_ep_combine_memory_kernel.h:505-553, 555-571, 573-601, 632-662)
//   KIND per-add  rows in ascending row index; y = T(float(y) + float(row)) after every add
//                 (reference: src/ep/kernels/tilexr_ep_combine_kernel.cpp:15-26, 54-101)
//   COMMQ 3/4     every row first takes the MXFP8 e5m2 / e4m3 round trip and is accumulated as
//                 ((fp8 * 2^(s-127)) * w) (reference: src/ep/kernels/tilexr_ep_mxfp8_quant.h:286-352)
//   INQ 2/5       rows hold int8 / fp8 payloads that are dequantised with their scales and rounded to the element
//                 type first (no reference counterpart)
//
// This file holds the register-resident kernel for 16-bit rows and is compiled once per (element type, with / without
// readiness flags): the including file sets TILEXR_REDUCE_BF16, TILEXR_REDUCE_FLAGS and TILEXR_REDUCE_ENTRY.
#if !defined(TILEXR_REDUCE_BF16) || !defined(TILEXR_REDUCE_FLAGS) || !defined(TILEXR_REDUCE_ENTRY)
#error "include from ep_reduce_vec_*.hip"
#endif

#include <algorithm>

#include "ep_reduce_common.hip.h"

namespace TileXREp {
namespace {

// WIDE: eight rows in flight per lane instead of four.  For launches with fewer waves than the device has SIMDs
// (decode): a wave that has a SIMD to itself gains nothing from small registers, and a token's rows arrive in one
// round trip instead of two.
//
// Launches with sliced rows (single-wave workgroups) that do not wait place their units by XCD: workgroup b runs on
// XCD b % 8 and takes a slice of a token t with t % 8 == b % 8, as the dispatch kernels do with a token's routes, so that
// rows which still sit in the L2 of the XCD that wrote them are read there (the eight L2s are not one cache: rows
// written on one XCD and read on another travel through memory).  128 tokens x 7168 x top-8, dispatch and combine in
// turn: 8.4 + 6.3 us without the placement, 5.7 + 3.2 us with it; a layer of 384 tokens 26.6 -> 21.5 us; from 1024 tokens
// on (117 MB of rows against 32 MB of L2) it makes no difference, and the launch keeps the plain order.
template <bool FL>
__host__ __device__ inline bool PlacesByXcd(const ReduceArgs &a, int lanesPerUnit)
{
    // sliced rows are launched with one wave per workgroup and one unit per wave; a launch that may wait has whole
    // workgroups per token and claims them as they become ready.  Up to three times the L2s' 32 MB of rows: beyond that
    // nothing is left to find there, and consecutive workgroups that read consecutive slices of the same rows are the
    // better order for memory (4096 tokens x 7168 x top-8: 88.7 us against 90.3 us placed by XCD)
    constexpr int64_t kPlacedRowBytes = int64_t{96} << 20;
    return lanesPerUnit == kWave && a.colSlices > 1 && (!FL || a.flagsSettled != 0) &&
        static_cast<int64_t>(a.bs) * a.slots * a.rowBytes <= kPlacedRowBytes;
}

template <int G, int V, int KIND, bool BF16, int COMMQ, bool FL, bool WIDE = false>
__global__ __launch_bounds__(kThreads) void ep_reduce_vec_kernel(ReduceArgs a)
{
    constexpr int kTokens = kThreads / G;
    constexpr bool kMx = COMMQ != 0;
    constexpr bool kCommE5m2 = COMMQ == TILEXR_EP_QUANT_COMM_MXFP8_E5M2;
    __shared__ int s_row[kTokens][kMaxTopK];
    __shared__ float s_w[kTokens][kMaxTopK];

    const int tg = threadIdx.x / G;
    const int lane = threadIdx.x % G;
    // Rows in flight per lane.  A whole workgroup per token is the geometry of launches that may wait on flags: at most two
    // such workgroups run per compute unit, so a wave may use half a SIMD's registers and keeps four rows in flight
    // whatever the row width; the other geometries run many more waves and trade rows in flight for occupancy.
    constexpr int KB = WIDE ? 8 : (G == kThreads ? 4 : (V <= 2 ? 4 : (V <= 4 ? 2 : 1)));
    const int vecs = a.h / 8;
    // a unit is one token, or -- for wide rows -- one slice of G * V vectors of a token
    // the launch may use fewer waves per workgroup than kThreads / kWave (single-wave workgroups for sliced rows)
    const int unitsPerGroup = static_cast<int>(blockDim.x) / G;
    const bool byXcd = PlacesByXcd<FL>(a, G);
    const int units = byXcd ? XcdPlacedUnits(a.bs, a.colSlices) : a.bs * a.colSlices;
    const int groups = (units + unitsPerGroup - 1) / unitsPerGroup;

    // token and slice of a unit; the token is -1 when the unit is padding
    auto placeOf = [&](int unit, int *slice) {
        int token = unit / a.colSlices;
        *slice = unit % a.colSlices;
        if (byXcd) {
            const int j = unit / kXcdCount;
            token = (j / a.colSlices) * kXcdCount + unit % kXcdCount;
            *slice = j % a.colSlices;
        }
        return unit < units && token < a.bs ? token : -1;
    };
    auto tokenAt = [&](int group, int t) {
        int slice;
        return placeOf(group * unitsPerGroup + t, &slice);
    };
    auto load = [&](int group, int mode) {
        int slice;
        const int token = placeOf(group * unitsPerGroup + tg, &slice);
        return LoadRoutes<false>(a, token < 0 ? 0 : token, token >= 0, lane, G, s_row[tg], s_w[tg], mode);
    };
    auto reduceUnit = [&](int group) {
        int slice;
        const int placed = placeOf(group * unitsPerGroup + tg, &slice);
        const bool tokOk = placed >= 0;
        const int token = tokOk ? placed : 0;
        const int colBase = slice * (G * V);
        if (KIND == kReducePerAdd) {
            if (lane == 0) {
                SortRows(s_row[tg], a.slots, a.orderKeys);
            }
            __syncthreads();
        }
        // Lane k of every wave keeps slot k's row and weight (the lanes of a wave share one token); the K loop takes the
        // slots that have a row, in k order, KB at a time, so a token that lost rows (capacity, masks) makes fewer trips
        // to memory.  Absent rows are skipped by the sum anyway: the order of the additions is the same.
        static_assert(G % kWave == 0, "a wave works on one token");
        const int waveLane = threadIdx.x % kWave;
        int slotRow = -1;
        float myWeight = 0.0f;
        if (waveLane < a.slots) {
            slotRow = s_row[tg][waveLane];
            myWeight = s_w[tg][waveLane];
        }
        const bool checkWords = FL && a.flagsSettled != 0;
        const uint32_t tileWord = checkWords ? SettledWordLoad(a, slotRow) : 0u;
        const bool expired = FL && __ballot(slotRow == kRowExpired) != 0;
        const bool active = tokOk && (a.tokenMask == nullptr || a.tokenMask[token] != 0) && !expired;
        const int myRow = active ? slotRow : -1;

        float acc[V][8];
#pragma unroll
        for (int j = 0; j < V; ++j) {
#pragma unroll
            for (int e = 0; e < 8; ++e) {
                acc[j][e] = 0.0f;
            }
        }
        // WIDE takes the slots as they stand, eight per trip (lane numbers known when the code is built: no chain of
        // scalar instructions from one slot to the next); the others compact the slots that have a row
        uint64_t todo = WIDE ? (a.slots > 0 ? 1ull : 0ull) : __ballot(myRow >= 0);
        int firstSlot = 0;
        // control flow below is uniform across the lanes that share a token (the MXFP8 round trip shuffles)
        while (todo != 0) {
            u32x4 v16[KB][V];
            int rowOfK[KB];
            float weightOfK[KB];
#pragma unroll
            for (int u = 0; u < KB; ++u) {
                const bool any = WIDE ? firstSlot + u < a.slots : todo != 0;
                const int k = WIDE ? firstSlot + u : (any ? __builtin_ctzll(todo) : 0);
                if (!WIDE) {
                    todo &= todo - 1;
                }
                const int row = any ? __builtin_amdgcn_readlane(myRow, k) : -1;
                rowOfK[u] = row;
                weightOfK[u] = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(myWeight), k));
                const char *base = static_cast<const char *>(a.expertOut) + static_cast<int64_t>(row < 0 ? 0 : row) * a.rowBytes;
                // WIDE: a slot without a row gets a resource of no bytes, and a lane beyond the row's end is beyond the
                // resource's: both read as zeros without a test per load (at this size the kernel is paid in
                // instructions)
                const __amdgpu_buffer_rsrc_t rsrc = RowResource(base, WIDE && row < 0 ? 0 : vecs * 16);
#pragma unroll
                for (int j = 0; j < V; ++j) {
                    const int idx = colBase + j * G + lane;
                    if (WIDE) {
                        v16[u][j] = __builtin_amdgcn_raw_buffer_load_b128(rsrc, idx * 16, 0, kAuxNonTemporal);
                    } else {
                        v16[u][j] = (row >= 0 && idx < vecs) ? RowLoad<FL>(base, rsrc, idx * 16) : u32x4{0u, 0u, 0u, 0u};
                    }
                }
            }
#pragma unroll
            for (int u = 0; u < KB; ++u) {
                if (rowOfK[u] < 0) {
                    continue;
                }
                const float w = weightOfK[u];
#pragma unroll
                for (int j = 0; j < V; ++j) {
                    float f[8];
#pragma unroll
                    for (int q = 0; q < 4; ++q) {
                        f[2 * q] = Decode16<BF16>(v16[u][j][q] & 0xffffu);
                        f[2 * q + 1] = Decode16<BF16>(v16[u][j][q] >> 16);
                    }
                    if (kMx) {
                        float amax = 0.0f;
#pragma unroll
                        for (int e = 0; e < 8; ++e) {
                            amax = fmaxf(amax, fabsf(f[e]));
                        }
                        amax = fmaxf(amax, __shfl_xor(amax, 1));
                        amax = fmaxf(amax, __shfl_xor(amax, 2));
                        const int se = MxSharedExponent<kCommE5m2>(amax);
                        const float up = Exp2Int(se);
#pragma unroll
                        for (int e = 0; e < 8; ++e) {
                            const float back = Fp8Decode<kCommE5m2>(Fp8Encode<kCommE5m2>(ldexpf(f[e], -se)));
                            f[e] = __fmul_rn(back, up);
                        }
                    }
                    if (KIND == kReducePerAdd) {
#pragma unroll
                        for (int e = 0; e < 8; ++e) {
                            acc[j][e] = RoundTo16<BF16>(__fadd_rn(acc[j][e], f[e]));
                        }
                    } else {
#pragma unroll
                        for (int e = 0; e < 8; ++e) {
                            acc[j][e] = __fadd_rn(acc[j][e], __fmul_rn(f[e], w));
                        }
                    }
                }
            }
            if (WIDE) {
                firstSlot += KB;
                todo = firstSlot < a.slots ? 1ull : 0ull;
            }
        }
        if (a.sharedExpertX != nullptr && active) {
            const u32x4 *sx = reinterpret_cast<const u32x4 *>(static_cast<const char *>(a.sharedExpertX) +
                static_cast<int64_t>(token) * a.h * 2);
#pragma unroll
            for (int j = 0; j < V; ++j) {
                const int idx = colBase + j * G + lane;
                if (idx < vecs) {
                    const u32x4 v = sx[idx];
#pragma unroll
                    for (int q = 0; q < 4; ++q) {
                        acc[j][2 * q] = __fadd_rn(acc[j][2 * q], Decode16<BF16>(v[q] & 0xffffu));
                        acc[j][2 * q + 1] = __fadd_rn(acc[j][2 * q + 1], Decode16<BF16>(v[q] >> 16));
                    }
                }
            }
        }
        const bool keep = active && !(checkWords && SettledWordMissing(a, slotRow, tileWord, waveLane));
        if (tokOk) {
            u32x4 *dst = reinterpret_cast<u32x4 *>(static_cast<char *>(a.y) + static_cast<int64_t>(token) * a.h * 2);
#pragma unroll
            for (int j = 0; j < V; ++j) {
                const int idx = colBase + j * G + lane;
                if (idx < vecs) {
                    u32x4 o;
#pragma unroll
                    for (int q = 0; q < 4; ++q) {
                        o[q] = keep ? EncodePair16Sat<BF16>(acc[j][2 * q], acc[j][2 * q + 1]) : 0u;
                    }
                    __builtin_nontemporal_store(o, dst + idx);
                }
            }
        }
    };
    ForEachGroup<FL>(a, groups, unitsPerGroup, tokenAt, load, reduceUnit);
}


constexpr int64_t kWideReduceUnits = 2048;      // token slices (waves) up to which a launch takes the WIDE kernel

template <int G, int V, int KIND, bool BF16, int COMMQ, bool FL>
void LaunchVec(const ReduceArgs &a, int gridLimit, hipStream_t stream)
{
    if constexpr (G == kThreads) {
        // whole-workgroup tokens are only used for rows published through readiness flags
        static_assert(FL, "one workgroup per token is the geometry of launches that wait on flags");
        int grid = a.bs;
        if (gridLimit > 0 && grid > gridLimit) {
            grid = gridLimit;
        }
        hipLaunchKernelGGL((ep_reduce_vec_kernel<G, V, KIND, BF16, COMMQ, true>), dim3(grid), dim3(kThreads), 0, stream, a);
    } else {
        // sliced rows: one wave per workgroup, so that no wave waits at a barrier for another slice's rows
        const int threads = a.colSlices > 1 ? G : kThreads;
        const int perGroup = threads / G;
        int64_t units = static_cast<int64_t>(a.bs) * a.colSlices;
        bool wide = false;
        if constexpr (G == kWave && V == 2 && KIND == kReduceFp32 && COMMQ == 0 && !FL) {
            wide = units <= kWideReduceUnits;
        }
        if (PlacesByXcd<FL>(a, G)) {
            units = XcdPlacedUnits(a.bs, a.colSlices);
        }
        int grid = static_cast<int>((units + perGroup - 1) / perGroup);
        if (gridLimit > 0 && grid > gridLimit * (kThreads / threads)) {
            // a multiple of eight, so that a workgroup's later units (blockIdx.x + i * gridDim.x) stay on its XCD
            grid = std::max(gridLimit * (kThreads / threads) / kXcdCount * kXcdCount, kXcdCount);
        }
        if constexpr (G == kWave && V == 2 && KIND == kReduceFp32 && COMMQ == 0 && !FL) {
            if (wide) {
                hipLaunchKernelGGL((ep_reduce_vec_kernel<G, V, KIND, BF16, COMMQ, FL, true>), dim3(grid), dim3(threads), 0, stream, a);
                return;
            }
        }
        hipLaunchKernelGGL((ep_reduce_vec_kernel<G, V, KIND, BF16, COMMQ, FL>), dim3(grid), dim3(threads), 0, stream, a);
    }
}

template <int G, int V, bool BF16, bool FL>
void LaunchByMode(const ReduceLaunch &l, const ReduceArgs &a, int gridLimit)
{
    if (l.reduceKind == kReducePerAdd) {
        LaunchVec<G, V, kReducePerAdd, BF16, 0, FL>(a, gridLimit, l.stream);
    } else if (l.commQuant == TILEXR_EP_QUANT_COMM_MXFP8_E5M2) {
        LaunchVec<G, V, kReduceFp32, BF16, TILEXR_EP_QUANT_COMM_MXFP8_E5M2, FL>(a, gridLimit, l.stream);
    } else if (l.commQuant == TILEXR_EP_QUANT_MXFP8) {
        LaunchVec<G, V, kReduceFp32, BF16, TILEXR_EP_QUANT_MXFP8, FL>(a, gridLimit, l.stream);
    } else {
        LaunchVec<G, V, kReduceFp32, BF16, 0, FL>(a, gridLimit, l.stream);
    }
}

} // namespace

void TILEXR_REDUCE_ENTRY(int g, int v, const ReduceLaunch &l, const ReduceArgs &a, int gridLimit)
{
    constexpr bool kBf16 = TILEXR_REDUCE_BF16;
    constexpr bool kFlags = TILEXR_REDUCE_FLAGS;
    if (g == kWave && v == 2) {
        LaunchByMode<kWave, 2, kBf16, kFlags>(l, a, gridLimit);
    } else if (g == kWave && v == 4) {
        LaunchByMode<kWave, 4, kBf16, kFlags>(l, a, gridLimit);
    }
    if constexpr (kFlags) {
        if (g == kThreads && v == 2) {
            LaunchByMode<kThreads, 2, kBf16, true>(l, a, gridLimit);
        } else if (g == kThreads && v == 4) {
            LaunchByMode<kThreads, 4, kBf16, true>(l, a, gridLimit);
        } else if (g == kThreads && v == 8) {
            LaunchByMode<kThreads, 8, kBf16, true>(l, a, gridLimit);
        }
    }
}

} // namespace TileXREp
