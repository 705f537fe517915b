// scatter: each token row is read once and written to the rows its routes were placed at (gfx950, wave64).
//
// HBM-bound byte movement, no MFMA.  Three kernels share the work:
//   ep_scatter_route_kernel    plain copies of wide rows in batches of 1024 tokens and more: one workgroup per
//                              (token, k, slice of 512 vectors; 1024 when readiness flags are published), two 16-byte
//                              loads and two 16-byte stores per lane
//   ep_scatter_vec_kernel      everything else that is 16-byte aligned (quantised payloads, narrow rows, small
//                              batches): G lanes cooperate on one token (a wave for narrow rows, the whole workgroup
//                              for wide ones); a lane keeps V 16-byte vectors of the row in registers, so every load of
//                              the row is in flight before the first store, then writes them to each destination row
//   ep_scatter_generic_kernel  any width and alignment, element by element
// Rows are written with non-temporal stores (they are not read again by this kernel; the input row is loaded with the
// default policy so that the sibling workgroups of a token find it in L2), or with agent-scope write-through stores
// when readiness flags are published.  Destination order (sorted or random rows) makes no difference.
//
//   QMODE 0  byte copy             (reference: src/ep/kernels/tilexr_ep_dispatch_helpers.h:104-112)
//   QMODE 1  static int8           (reference: tilexr_ep_dispatch_helpers.h:114-136)
//   QMODE 2  per-token int8        (reference: tilexr_ep_dispatch_helpers.h:153-191; BF16 decode has no counterpart)
//   QMODE 4  MXFP8, 32-wide blocks (reference: tests/ep/demo/mxfp8_golden.h:116-152)
//   QMODE 5  fp8 e4m3, fp32 scale per 128 columns (no reference counterpart)
#include <hip/hip_runtime.h>

#include "ep_kernel_common.hip.h"
#include "ep_launch.h"
#include "ep_numerics.hip.h"
#include "ep_place.hip.h"
#include "ep_tile_publish.h"
#include "tilexr_ep.h"

namespace TileXREp {
namespace {

struct ScatterArgs {
    const void *x;
    const int32_t *rowOf;
    PlaceArgs place;             // place.ids != nullptr: resolve the rows here instead of reading rowOf
    int bs;
    int h;
    int topK;
    const float *staticScale;
    void *out;
    void *scalesOut;
    uint64_t *tileFlags;
    uint32_t *tileCounters;
    int maxTiles;                // tiles of the largest possible row count: the group counters start there
    int tileRows;
    uint64_t epoch;
    const int32_t *totalRowsPtr;
    int colSlices;               // route kernel: workgroups a row is cut into
};

__device__ __forceinline__ int RowOfRoute(const ScatterArgs &a, int route)
{
    return a.place.ids != nullptr ? PlaceRoute(a.place, route) : a.rowOf[route];
}

template <int G>
__device__ __forceinline__ float GroupMax(float v, float *red, int lane)
{
#pragma unroll
    for (int off = kWave / 2; off >= 1; off >>= 1) {
        v = fmaxf(v, __shfl_xor(v, off));
    }
    if (G > kWave) {
        if ((lane & (kWave - 1)) == 0) {
            red[lane / kWave] = v;
        }
        __syncthreads();
        v = fmaxf(fmaxf(red[0], red[1]), fmaxf(red[2], red[3]));
        __syncthreads();
    }
    return v;
}

// Row stores of the register-resident kernels.  WT = false: non-temporal stores (the rows are not read again by this
// kernel).  WT = true: agent-scope write-through stores, used when readiness flags are published: such a store is
// complete for every XCD once the issuing wave's vmcnt is zero, so publishing needs no L2 write-back.
template <bool WT>
__device__ __forceinline__ void RowStore(const u32x4 &v, char *rowBase, __amdgpu_buffer_rsrc_t rsrc, int byteOffset)
{
    if (WT) {
        __builtin_amdgcn_raw_buffer_store_b128(v, rsrc, byteOffset, 0, kAuxAgentScope);
    } else {
        __builtin_nontemporal_store(v, reinterpret_cast<u32x4 *>(rowBase + byteOffset));
    }
}

template <bool WT>
__device__ __forceinline__ void RowStore(const u32x2 &v, char *rowBase, __amdgpu_buffer_rsrc_t rsrc, int byteOffset)
{
    if (WT) {
        __builtin_amdgcn_raw_buffer_store_b64(v, rsrc, byteOffset, 0, kAuxAgentScope);
    } else {
        __builtin_nontemporal_store(v, reinterpret_cast<u32x2 *>(rowBase + byteOffset));
    }
}

template <bool WT, typename T>
__device__ __forceinline__ void ScalarStore(T *p, T v)
{
    if (WT) {
        __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    } else {
        *p = v;
    }
}

__device__ __forceinline__ void PublishRow(const ScatterArgs &a, int row, int parts)
{
    TilePublishArgs t;
    t.flags = a.tileFlags;
    t.counters = a.tileCounters;
    t.tileRows = a.tileRows;
    t.maxTiles = a.maxTiles;
    t.totalRows = (a.tileRows > 1 || parts > 1) ? *a.totalRowsPtr : 0;
    t.epoch = a.epoch;
    DeviceTileOps ops;
    PublishLanded(ops, t, row, parts);
}

// Publishes the rows of one token.  Each wave waits for its own stores and the barrier collects the waves.
// WT = true: the rows were written through and are then complete.  WT = false: the rows may still sit dirty in this
// XCD's L2 and one release fence per publishing wave writes them back (slow under load; element-granular fallback only).
template <bool WT>
__device__ __forceinline__ void PublishRows(const ScatterArgs &a, const int *pos, int lane, int G)
{
    WaitOwnStores();
    if (G > kWave) {
        __syncthreads();
    }
    if (lane < a.topK) {
        if (!WT) {
            ReleaseRowsToAgent();
        }
        for (int k = lane; k < a.topK; k += G) {
            const int row = pos[k];
            if (row >= 0) {
                PublishRow(a, row, 1);
            }
        }
    }
}

// Plain copy of wide rows, one workgroup per (route, slice of 512 vectors): the workgroup loads its part of the token's
// row and writes it to the destination row of route (token, k).  The workgroups of a token are given block indices that
// the dispatcher places on the same XCD (block b runs on XCD b % 8), so the row comes from HBM once and from that
// XCD's L2 the other topK - 1 times.  Two 16-byte loads then two 16-byte stores per lane is what this memory system
// rewards, whatever the workgroup size: measured on 4096 x 7168 x top-8, 83-85 us with two vectors per lane (128 to
// 448 lanes per workgroup), 92-95 us with three to fourteen, 105-130 us with one; 93 us for "one workgroup writes all
// topK rows", and 132 us when the workgroups of a token are spread over the XCDs.
constexpr int kRouteVecs = 2;
constexpr unsigned kRouteCapLdsBytes = 27 * 1024;    // 160 KiB of LDS per compute unit: five workgroups fit
template <int THREADS, int V, bool WT>
__global__ __launch_bounds__(THREADS) void ep_scatter_route_kernel(ScatterArgs a)
{
    constexpr int kXcds = 8;
    __shared__ int s_row;
    // grid = (8 * slices, topK, groups of eight tokens): the hardware hands out the three indices, so no workgroup
    // starts with a division (this kernel runs at the rate its resident workgroups allow: a prologue of sixty scalar
    // instructions ahead of the first load was a tenth of a workgroup's life).  Workgroups are dealt to the XCDs in
    // linear order, x fastest, and gridDim.x is a multiple of eight: the XCD is blockIdx.x % 8.
    const int token = static_cast<int>(blockIdx.z) * kXcds + static_cast<int>(blockIdx.x % kXcds);
    const int k = blockIdx.y;
    const int colBase = static_cast<int>(blockIdx.x / kXcds) * (V * THREADS);
    if (token >= a.bs) {
        return;
    }
    const int lane = threadIdx.x;
    const int vecs = a.h / 8;
    if (lane == 0) {
        s_row = RowOfRoute(a, token * a.topK + k);
    }
    const u32x4 *src = reinterpret_cast<const u32x4 *>(static_cast<const char *>(a.x) + static_cast<int64_t>(token) * a.h * 2);
    u32x4 v[V];
#pragma unroll
    for (int i = 0; i < V; ++i) {
        const int idx = colBase + i * THREADS + lane;
        v[i] = idx < vecs ? src[idx] : u32x4{0u, 0u, 0u, 0u};
    }
    __syncthreads();
    const int row = __builtin_amdgcn_readfirstlane(s_row);
    if (row < 0) {
        return;
    }
    char *dst = static_cast<char *>(a.out) + static_cast<int64_t>(row) * a.h * 2;
    const __amdgpu_buffer_rsrc_t rsrc = RowResource(dst, vecs * 16);
#pragma unroll
    for (int i = 0; i < V; ++i) {
        const int idx = colBase + i * THREADS + lane;
        if (idx < vecs) {
            RowStore<WT>(v[i], dst, rsrc, idx * 16);
        }
    }
    if (WT && a.tileFlags != nullptr) {
        WaitOwnStores();
        __syncthreads();
        if (lane == 0) {
            PublishRow(a, row, a.colSlices);
        }
    }
}

template <int G, int V, int QMODE, bool BF16, bool E5M2, bool WT>
__global__ __launch_bounds__(kThreads) void ep_scatter_vec_kernel(ScatterArgs a)
{
    constexpr int kTokens = kThreads / G;
    __shared__ int s_pos[kTokens][kMaxTopK];
    __shared__ float s_red[kTokens][kWavesPerBlock];

    const int tg = threadIdx.x / G;
    const int lane = threadIdx.x % G;
    const int token = blockIdx.x * kTokens + tg;
    const bool tokOk = token < a.bs;
    const int vecs = a.h / 8;

    for (int k = lane; k < a.topK; k += G) {
        s_pos[tg][k] = tokOk ? RowOfRoute(a, token * a.topK + k) : -1;
    }
    const u32x4 *src = reinterpret_cast<const u32x4 *>(static_cast<const char *>(a.x) +
        static_cast<int64_t>(tokOk ? token : 0) * a.h * 2);
    u32x4 v[V];
#pragma unroll
    for (int j = 0; j < V; ++j) {
        const int idx = j * G + lane;
        v[j] = (tokOk && idx < vecs) ? src[idx] : u32x4{0u, 0u, 0u, 0u};
    }
    __syncthreads();

    if (QMODE == TILEXR_EP_QUANT_NONE) {
        for (int k = 0; k < a.topK; ++k) {
            // the lanes of a wave share one token, so the row is wave-uniform
            const int row = __builtin_amdgcn_readfirstlane(s_pos[tg][k]);
            if (row < 0) {
                continue;
            }
            char *dst = static_cast<char *>(a.out) + static_cast<int64_t>(row) * a.h * 2;
            const __amdgpu_buffer_rsrc_t rsrc = RowResource(dst, vecs * 16);
#pragma unroll
            for (int j = 0; j < V; ++j) {
                const int idx = j * G + lane;
                if (idx < vecs) {
                    RowStore<WT>(v[j], dst, rsrc, idx * 16);
                }
            }
        }
    } else {
        // per-row / per-block scale, then 8 output bytes per input vector
        float rowScaleInv = 1.0f;
        float rowScale = 1.0f;
        if (QMODE == TILEXR_EP_QUANT_STATIC_INT8) {
            rowScaleInv = a.staticScale[0];
        }
        if (QMODE == TILEXR_EP_QUANT_TOKEN_INT8) {
            float amax = 0.0f;
#pragma unroll
            for (int j = 0; j < V; ++j) {
#pragma unroll
                for (int w = 0; w < 4; ++w) {
                    amax = fmaxf(amax, fabsf(Decode16<BF16>(v[j][w] & 0xffffu)));
                    amax = fmaxf(amax, fabsf(Decode16<BF16>(v[j][w] >> 16)));
                }
            }
            amax = GroupMax<G>(amax, s_red[tg], lane);
            rowScale = amax > 0.0f ? __fdiv_rn(amax, 127.0f) : 1.0f;
            rowScaleInv = rowScale > 0.0f ? __fdiv_rn(1.0f, rowScale) : 1.0f;
        }
        u32x2 q[V];
        float blockScale[V];
        int sharedExp[V];
#pragma unroll
        for (int j = 0; j < V; ++j) {
            float f[8];
#pragma unroll
            for (int w = 0; w < 4; ++w) {
                f[2 * w] = Decode16<BF16>(v[j][w] & 0xffffu);
                f[2 * w + 1] = Decode16<BF16>(v[j][w] >> 16);
            }
            uint32_t bytes[8];
            uint32_t fp8Words[2] = {0u, 0u};
            if (QMODE == TILEXR_EP_QUANT_MXFP8 || QMODE == TILEXR_EP_QUANT_FP8_BLOCK128) {
                float amax = 0.0f;
#pragma unroll
                for (int e = 0; e < 8; ++e) {
                    amax = fmaxf(amax, fabsf(f[e]));
                }
                // 32 columns = 4 neighbouring lanes, 128 columns = 16 neighbouring lanes
                constexpr int kSpan = QMODE == TILEXR_EP_QUANT_MXFP8 ? 4 : 16;
#pragma unroll
                for (int off = 1; off < kSpan; off <<= 1) {
                    amax = fmaxf(amax, __shfl_xor(amax, off));
                }
                if (QMODE == TILEXR_EP_QUANT_MXFP8) {
                    const int se = MxSharedExponent<E5M2>(amax);
                    sharedExp[j] = se;
#pragma unroll
                    for (int e = 0; e < 8; ++e) {
                        bytes[e] = Fp8Encode<E5M2>(ldexpf(f[e], -se));
                    }
                } else {
                    const float sc = amax > 0.0f ? __fdiv_rn(amax, 448.0f) : 1.0f;
                    blockScale[j] = sc;
                    // eight quotients by one divisor: what depends on the divisor alone is done once (ep_numerics.hip.h)
                    float quot[8];
                    const bool shortForm = __all(SharedReciprocalHolds(sc) ? 1 : 0) != 0;
                    if (shortForm) {
                        const float y = SharedReciprocal(sc);
#pragma unroll
                        for (int e = 0; e < 8; ++e) {
                            quot[e] = DivideByShared(f[e], sc, y);
                        }
                    } else {
#pragma unroll
                        for (int e = 0; e < 8; ++e) {
                            quot[e] = __fdiv_rn(f[e], sc);
                        }
                    }
                    bool anyNan = false;
#pragma unroll
                    for (int e = 0; e < 8; e += 2) {
                        anyNan |= __builtin_isunordered(quot[e], quot[e + 1]);
                    }
                    if (!anyNan) {
                        // four codes per word straight from the converts: the second one fills the word's upper half
                        fp8Words[0] = Fp8E4m3EncodeFourSat(quot[0], quot[1], quot[2], quot[3]);
                        fp8Words[1] = Fp8E4m3EncodeFourSat(quot[4], quot[5], quot[6], quot[7]);
                    } else {
#pragma unroll
                        for (int e = 0; e < 8; e += 4) {
                            fp8Words[e / 4] = Fp8E4m3EncodePairSat(quot[e], quot[e + 1]) |
                                (Fp8E4m3EncodePairSat(quot[e + 2], quot[e + 3]) << 16);
                        }
                    }
                }
            } else {
#pragma unroll
                for (int e = 0; e < 8; ++e) {
                    bytes[e] = static_cast<uint32_t>(ClampInt8(__fmul_rn(f[e], rowScaleInv))) & 0xffu;
                }
            }
            if (QMODE == TILEXR_EP_QUANT_FP8_BLOCK128) {
                q[j][0] = fp8Words[0];
                q[j][1] = fp8Words[1];
            } else {
                q[j][0] = bytes[0] | (bytes[1] << 8) | (bytes[2] << 16) | (bytes[3] << 24);
                q[j][1] = bytes[4] | (bytes[5] << 8) | (bytes[6] << 16) | (bytes[7] << 24);
            }
        }
        const int mxBlocks = (a.h + 31) / 32;
        const int mxScales = (mxBlocks + 1) / 2 * 2;
        const int b128 = (a.h + 127) / 128;
        for (int k = 0; k < a.topK; ++k) {
            const int row = __builtin_amdgcn_readfirstlane(s_pos[tg][k]);
            if (row < 0) {
                continue;
            }
            char *dst = static_cast<char *>(a.out) + static_cast<int64_t>(row) * a.h;
            const __amdgpu_buffer_rsrc_t rsrc = RowResource(dst, vecs * 8);
#pragma unroll
            for (int j = 0; j < V; ++j) {
                const int idx = j * G + lane;
                if (idx < vecs) {
                    RowStore<WT>(q[j], dst, rsrc, idx * 8);
                    if (QMODE == TILEXR_EP_QUANT_MXFP8 && (idx & 3) == 0) {
                        uint8_t *sc = static_cast<uint8_t *>(a.scalesOut) + static_cast<int64_t>(row) * mxScales;
                        ScalarStore<WT>(sc + (idx >> 2), static_cast<uint8_t>(sharedExp[j] + 127));
                        if ((idx >> 2) + 1 == mxBlocks && mxBlocks < mxScales) {
                            ScalarStore<WT>(sc + mxBlocks, static_cast<uint8_t>(0));    // padding byte of an odd block count
                        }
                    }
                    if (QMODE == TILEXR_EP_QUANT_FP8_BLOCK128 && (idx & 15) == 0) {
                        ScalarStore<WT>(static_cast<float *>(a.scalesOut) + static_cast<int64_t>(row) * b128 + (idx >> 4),
                            blockScale[j]);
                    }
                }
            }
            if (QMODE == TILEXR_EP_QUANT_TOKEN_INT8 && lane == 0) {
                ScalarStore<WT>(static_cast<float *>(a.scalesOut) + row, rowScale);
            }
        }
    }
    if (WT && a.tileFlags != nullptr) {
        PublishRows<true>(a, s_pos[tg], lane, G);
    }
}

// Any row width / alignment: one workgroup per token, element-granular.  Used when h is not a multiple of 8, a
// base pointer is not 16-byte aligned or the row does not fit the register-resident kernel.
template <bool BF16, bool E5M2>
__global__ __launch_bounds__(kThreads) void ep_scatter_generic_kernel(ScatterArgs a, int qmode)
{
    __shared__ int s_pos[kMaxTopK];
    __shared__ float s_red[kWavesPerBlock];
    const int token = blockIdx.x;
    const int tid = threadIdx.x;
    for (int k = tid; k < a.topK; k += kThreads) {
        s_pos[k] = RowOfRoute(a, token * a.topK + k);
    }
    const uint16_t *src = static_cast<const uint16_t *>(a.x) + static_cast<int64_t>(token) * a.h;
    float rowScale = 1.0f;
    float rowScaleInv = qmode == TILEXR_EP_QUANT_STATIC_INT8 ? a.staticScale[0] : 1.0f;
    if (qmode == TILEXR_EP_QUANT_TOKEN_INT8) {
        float amax = 0.0f;
        for (int i = tid; i < a.h; i += kThreads) {
            amax = fmaxf(amax, fabsf(Decode16<BF16>(src[i])));
        }
        amax = GroupMax<kThreads>(amax, s_red, tid);
        rowScale = amax > 0.0f ? __fdiv_rn(amax, 127.0f) : 1.0f;
        rowScaleInv = rowScale > 0.0f ? __fdiv_rn(1.0f, rowScale) : 1.0f;
    }
    __syncthreads();
    const int mxBlocks = (a.h + 31) / 32;
    const int mxScales = (mxBlocks + 1) / 2 * 2;
    const int b128 = (a.h + 127) / 128;
    for (int k = 0; k < a.topK; ++k) {
        const int row = s_pos[k];
        if (row < 0) {
            continue;
        }
        if (qmode == TILEXR_EP_QUANT_NONE) {
            uint16_t *dst = static_cast<uint16_t *>(a.out) + static_cast<int64_t>(row) * a.h;
            for (int i = tid; i < a.h; i += kThreads) {
                dst[i] = src[i];
            }
        } else if (qmode == TILEXR_EP_QUANT_STATIC_INT8 || qmode == TILEXR_EP_QUANT_TOKEN_INT8) {
            int8_t *dst = static_cast<int8_t *>(a.out) + static_cast<int64_t>(row) * a.h;
            for (int i = tid; i < a.h; i += kThreads) {
                dst[i] = static_cast<int8_t>(ClampInt8(__fmul_rn(Decode16<BF16>(src[i]), rowScaleInv)));
            }
            if (qmode == TILEXR_EP_QUANT_TOKEN_INT8 && tid == 0) {
                static_cast<float *>(a.scalesOut)[row] = rowScale;
            }
        } else if (qmode == TILEXR_EP_QUANT_MXFP8) {
            uint8_t *dst = static_cast<uint8_t *>(a.out) + static_cast<int64_t>(row) * a.h;
            uint8_t *sc = static_cast<uint8_t *>(a.scalesOut) + static_cast<int64_t>(row) * mxScales;
            for (int b = tid; b < mxScales; b += kThreads) {
                if (b >= mxBlocks) {
                    sc[b] = 0;
                    continue;
                }
                const int begin = b * 32;
                const int end = min(begin + 32, a.h);
                float amax = 0.0f;
                for (int i = begin; i < end; ++i) {
                    amax = fmaxf(amax, fabsf(Decode16<BF16>(src[i])));
                }
                const int se = MxSharedExponent<E5M2>(amax);
                sc[b] = static_cast<uint8_t>(se + 127);
                for (int i = begin; i < end; ++i) {
                    dst[i] = static_cast<uint8_t>(Fp8Encode<E5M2>(ldexpf(Decode16<BF16>(src[i]), -se)));
                }
            }
        } else {
            uint8_t *dst = static_cast<uint8_t *>(a.out) + static_cast<int64_t>(row) * a.h;
            float *sc = static_cast<float *>(a.scalesOut) + static_cast<int64_t>(row) * b128;
            for (int b = tid; b < b128; b += kThreads) {
                const int begin = b * 128;
                const int end = min(begin + 128, a.h);
                float amax = 0.0f;
                for (int i = begin; i < end; ++i) {
                    amax = fmaxf(amax, fabsf(Decode16<BF16>(src[i])));
                }
                const float scale = amax > 0.0f ? __fdiv_rn(amax, 448.0f) : 1.0f;
                sc[b] = scale;
                for (int i = begin; i < end; ++i) {
                    dst[i] = static_cast<uint8_t>(Fp8Encode<false>(__fdiv_rn(Decode16<BF16>(src[i]), scale)));
                }
            }
        }
    }
    if (a.tileFlags != nullptr) {
        PublishRows<false>(a, s_pos, tid, kThreads);
    }
}

// Rows move with write-through stores when readiness flags are published (see RowStore).
inline bool WriteThrough(const ScatterArgs &a)
{
    return a.tileFlags != nullptr;
}

template <int G, int V, int QMODE, bool BF16, bool E5M2>
void LaunchVec(const ScatterArgs &a, hipStream_t stream)
{
    constexpr int kTokens = kThreads / G;
    const int grid = (a.bs + kTokens - 1) / kTokens;
    if (WriteThrough(a)) {
        hipLaunchKernelGGL((ep_scatter_vec_kernel<G, V, QMODE, BF16, E5M2, true>), dim3(grid), dim3(kThreads), 0, stream, a);
    } else {
        hipLaunchKernelGGL((ep_scatter_vec_kernel<G, V, QMODE, BF16, E5M2, false>), dim3(grid), dim3(kThreads), 0, stream, a);
    }
}

template <int G, int V>
void LaunchByMode(const ScatterLaunch &l, const ScatterArgs &a)
{
    switch (l.quantMode) {
        case TILEXR_EP_QUANT_NONE:
            // small batches are latency-bound and gain nothing from the extra workgroups
            if (G == kThreads && ScatterCopiesPerRoute(l.x, l.out, l.bs, l.h, l.topK, l.quantMode)) {
                const dim3 blocks(static_cast<unsigned>(8 * a.colSlices), static_cast<unsigned>(a.topK),
                    static_cast<unsigned>((a.bs + 7) / 8));
                if (l.kernelNameOut != nullptr) {
                    *l.kernelNameOut = "ep_scatter_route_kernel";
                }
                if (WriteThrough(a) && a.colSlices > 1 && !l.consumerBeside) {
                    // A publishing workgroup stays until its stores have landed and then counts its part of the row
                    // towards the tile: worth doing once per row rather than once per half row, so rows wider than 512
                    // vectors get workgroups of 512 lanes (4096 x 7168 x top-8: 82.2 instead of 84.7 us; without
                    // flags the narrower workgroups are the faster ones, 81.9 against 82.5 us).  Not when a consumer
                    // is expected beside this launch: its waiting workgroups leave room for the narrower ones only
                    // (dispatch + combine on two streams: 272 us with the wide ones, 244 us with the narrow ones).
                    constexpr int kWide = 2 * kThreads;
                    ScatterArgs wide = a;
                    wide.colSlices = (a.h / 8 + kRouteVecs * kWide - 1) / (kRouteVecs * kWide);
                    const dim3 wideBlocks(static_cast<unsigned>(8 * wide.colSlices), static_cast<unsigned>(a.topK),
                        static_cast<unsigned>((a.bs + 7) / 8));
                    hipLaunchKernelGGL((ep_scatter_route_kernel<kWide, kRouteVecs, true>), wideBlocks, dim3(kWide), 0,
                        l.stream, wide);
                } else if (WriteThrough(a)) {
                    hipLaunchKernelGGL((ep_scatter_route_kernel<kThreads, kRouteVecs, true>), blocks, dim3(kThreads), 0,
                        l.stream, a);
                } else {
                    // Workgroups that only look their row up in the row map are short-lived, and eight of them per
                    // compute unit keep more stores in flight than this memory system digests (4096 x 7168 x top-8:
                    // 88.9 us; seven 86.5, five 81.7, four 85.3, three 98.2).  Unused dynamic LDS caps them at five.
                    // Workgroups that resolve their row themselves (three dependent loads) are slow enough as they are.
                    const unsigned capLds = a.place.ids == nullptr ? kRouteCapLdsBytes : 0u;
                    hipLaunchKernelGGL((ep_scatter_route_kernel<kThreads, kRouteVecs, false>), blocks, dim3(kThreads), capLds,
                        l.stream, a);
                }
            } else {
                LaunchVec<G, V, TILEXR_EP_QUANT_NONE, true, false>(a, l.stream);
            }
            break;
        case TILEXR_EP_QUANT_STATIC_INT8:
            LaunchVec<G, V, TILEXR_EP_QUANT_STATIC_INT8, false, false>(a, l.stream);
            break;
        case TILEXR_EP_QUANT_TOKEN_INT8:
            if (l.inputBf16) {
                LaunchVec<G, V, TILEXR_EP_QUANT_TOKEN_INT8, true, false>(a, l.stream);
            } else {
                LaunchVec<G, V, TILEXR_EP_QUANT_TOKEN_INT8, false, false>(a, l.stream);
            }
            break;
        case TILEXR_EP_QUANT_MXFP8:
            if (l.inputBf16) {
                if (l.fp8E5m2) {
                    LaunchVec<G, V, TILEXR_EP_QUANT_MXFP8, true, true>(a, l.stream);
                } else {
                    LaunchVec<G, V, TILEXR_EP_QUANT_MXFP8, true, false>(a, l.stream);
                }
            } else {
                if (l.fp8E5m2) {
                    LaunchVec<G, V, TILEXR_EP_QUANT_MXFP8, false, true>(a, l.stream);
                } else {
                    LaunchVec<G, V, TILEXR_EP_QUANT_MXFP8, false, false>(a, l.stream);
                }
            }
            break;
        default:
            if (l.inputBf16) {
                LaunchVec<G, V, TILEXR_EP_QUANT_FP8_BLOCK128, true, false>(a, l.stream);
            } else {
                LaunchVec<G, V, TILEXR_EP_QUANT_FP8_BLOCK128, false, false>(a, l.stream);
            }
            break;
    }
}

} // namespace

bool ScatterCopiesPerRoute(const void *x, const void *out, int64_t bs, int64_t h, int64_t topK, int quantMode)
{
    const int64_t vecs = h / 8;
    // token rows beyond half the memory-side cache (256 MiB) cannot be kept close by: the per-token kernel takes those
    return quantMode == TILEXR_EP_QUANT_NONE && h % 8 == 0 && Aligned16(x) && Aligned16(out) && vecs > 4 * kWave &&
        vecs <= 8 * kThreads && topK > 1 && bs >= 1024 && bs * h * 2 <= (int64_t{128} << 20) &&
        (bs + 7) / 8 <= 65535 && topK <= 65535;
}

hipError_t LaunchScatter(const ScatterLaunch &l)
{
    ScatterArgs a {};
    a.x = l.x;
    a.rowOf = l.rowOf;
    if (l.fusedPlace != nullptr) {
        a.place = MakePlaceArgs(*l.fusedPlace);
    }
    a.bs = static_cast<int>(l.bs);
    a.h = static_cast<int>(l.h);
    a.topK = static_cast<int>(l.topK);
    a.staticScale = l.staticScale;
    a.out = l.out;
    a.scalesOut = l.scalesOut;
    a.tileFlags = l.tileFlags;
    a.tileCounters = l.tileCounters;
    a.tileRows = static_cast<int>(l.tileRows);
    a.maxTiles = l.tileRows > 0 ? static_cast<int>((l.bs * l.topK + l.tileRows - 1) / l.tileRows) : 0;
    a.epoch = l.epoch;
    a.totalRowsPtr = l.totalRowsPtr;
    a.colSlices = static_cast<int>((l.h / 8 + kRouteVecs * kThreads - 1) / (kRouteVecs * kThreads));
    const int64_t vecs = l.h / 8;
    const bool vecOk = l.h % 8 == 0 && Aligned16(l.x) && vecs <= 8 * kThreads &&
        (l.quantMode == TILEXR_EP_QUANT_NONE ? Aligned16(l.out) : Aligned8(l.out));
    if (l.kernelNameOut != nullptr) {
        *l.kernelNameOut = vecOk ? "ep_scatter_vec_kernel" : "ep_scatter_generic_kernel";
    }
    if (vecOk) {
        // narrow rows: a wave per token (four tokens per workgroup); wide rows: the workgroup per token
        if (vecs <= 2 * kWave) {
            LaunchByMode<kWave, 2>(l, a);
        } else if (vecs <= 4 * kWave) {
            LaunchByMode<kWave, 4>(l, a);
        } else if (vecs <= 2 * kThreads) {
            LaunchByMode<kThreads, 2>(l, a);
        } else if (vecs <= 4 * kThreads) {
            LaunchByMode<kThreads, 4>(l, a);
        } else {
            LaunchByMode<kThreads, 8>(l, a);
        }
    } else {
        const dim3 grid(static_cast<unsigned>(l.bs));
        if (l.inputBf16) {
            if (l.fp8E5m2) {
                hipLaunchKernelGGL((ep_scatter_generic_kernel<true, true>), grid, dim3(kThreads), 0, l.stream, a, l.quantMode);
            } else {
                hipLaunchKernelGGL((ep_scatter_generic_kernel<true, false>), grid, dim3(kThreads), 0, l.stream, a, l.quantMode);
            }
        } else {
            if (l.fp8E5m2) {
                hipLaunchKernelGGL((ep_scatter_generic_kernel<false, true>), grid, dim3(kThreads), 0, l.stream, a, l.quantMode);
            } else {
                hipLaunchKernelGGL((ep_scatter_generic_kernel<false, false>), grid, dim3(kThreads), 0, l.stream, a, l.quantMode);
            }
        }
    }
    return hipGetLastError();
}

} // namespace TileXREp
