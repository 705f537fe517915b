// HIP kernels of the EP dispatch / combine data path for gfx950 (CDNA4, wave64).
//
// Everything here is HBM-bound integer / byte movement with a little fp32 arithmetic: no MFMA.  The design rules
// are: read each token row once (128-bit loads), write it topK times (128-bit non-temporal stores), keep every
// decision about WHERE a row goes out of the copy kernel (it is pre-computed by the count + place kernels), and
// give each copy workgroup enough independent loads in flight (8 x 16 B per lane) to cover HBM latency.
//
// Reference behaviour restated by each kernel is cited at the kernel.
#include <hip/hip_runtime.h>

#include "ep_launch.h"
#include "ep_numerics.cuh"
#include "tilexr_ep.h"

namespace TileXREp {
namespace {

constexpr int kThreads = 256;
constexpr int kWave = 64;
constexpr int kWavesPerBlock = kThreads / kWave;
constexpr int kVecMax = 8;              // 16-byte vectors a lane keeps in registers per row

__device__ __forceinline__ unsigned long long LaneMaskLt()
{
    return (1ull << (threadIdx.x & (kWave - 1))) - 1ull;
}

// Exclusive scan of vals[0..m) in place (LDS), m <= 2048, by all 256 threads.  part[] is 256 ints of LDS.
// Returns the total.
__device__ int BlockExclusiveScan(int *vals, int m, int *part)
{
    const int tid = threadIdx.x;
    const int per = (m + kThreads - 1) / kThreads;
    const int begin = tid * per;
    int local = 0;
    for (int i = begin; i < begin + per && i < m; ++i) {
        local += vals[i];
    }
    part[tid] = local;
    __syncthreads();
    for (int off = 1; off < kThreads; off <<= 1) {
        const int add = tid >= off ? part[tid - off] : 0;
        __syncthreads();
        part[tid] += add;
        __syncthreads();
    }
    int run = part[tid] - local;
    const int total = part[kThreads - 1];
    for (int i = begin; i < begin + per && i < m; ++i) {
        const int v = vals[i];
        vals[i] = run;
        run += v;
    }
    __syncthreads();
    return total;
}

// -------------------------------------------------------------------------------------------------------------
// count: stable rank of every live route within (chunk, key), per-chunk key histogram, and -- in the last
// workgroup to finish -- the scans that turn histograms into destinations and the count outputs.
//
// Replaces the reference's per-route O(n) pass (`CalTokenSendExpertCnt`, number of earlier routes with the same
// expert, src/ep/kernels/tilexr_ep_dispatch_memory_kernel.h:791-818), its count exchange and cumulative sum
// (:820-1089) and the count outputs (:1142-1168); for the MVP route the same machinery with a single key gives the
// token-major, k-minor compaction of src/ep/kernels/tilexr_ep_dispatch_kernel.cpp:501-571.
// Route liveness: ids outside [0, E) are skipped (:686-687); mask modes are described in ep_launch.h.
// -------------------------------------------------------------------------------------------------------------
struct RouteCountArgs {
    const int32_t *ids;
    const uint8_t *mask;
    int maskMode;
    int bs;
    int topK;
    int numExperts;
    int keyDiv;
    int numKeys;
    int keyBits;
    int capacity;
    int numChunks;
    CountScratch s;
    int32_t *sendCountsOut;
    int32_t *recvCountOut;
    int64_t *expertTokenNumsOut;
    int tokenNumsType;
};

__global__ __launch_bounds__(kThreads) void ep_route_count_kernel(RouteCountArgs a)
{
    __shared__ int s_cnt[kWavesPerBlock * kMaxKeys];
    __shared__ int s_exp[kMaxKeys];
    __shared__ int s_part[kThreads];
    __shared__ int s_misc[4];

    const int tid = threadIdx.x;
    const int wave = tid / kWave;
    const int lane = tid & (kWave - 1);
    const int n = a.bs * a.topK;
    const int chunk = blockIdx.x;
    const bool expHist = a.s.chunkExpHist != nullptr;

    for (int i = tid; i < kWavesPerBlock * a.numKeys; i += kThreads) {
        s_cnt[i] = 0;
    }
    if (expHist) {
        for (int i = tid; i < a.numExperts; i += kThreads) {
            s_exp[i] = 0;
        }
    }
    if (tid == 0) {
        s_misc[0] = 0;
    }
    __syncthreads();

    int liveLimit = n;
    if (a.maskMode == kMaskTokenPrefix) {
        // activeCnt = sum(mask); only the first activeCnt tokens are dispatched
        // (reference: tilexr_ep_dispatch_memory_kernel.h:1387-1410, 1538-1544)
        int local = 0;
        for (int t = tid; t < a.bs; t += kThreads) {
            local += a.mask[t] != 0 ? 1 : 0;
        }
        for (int off = kWave / 2; off >= 1; off >>= 1) {
            local += __shfl_xor(local, off);
        }
        if (lane == 0) {
            atomicAdd(&s_misc[0], local);
        }
        __syncthreads();
        liveLimit = s_misc[0] * a.topK;
    }

    // phase A: per-wave histogram of the wave's 256 consecutive routes
    int keys[kChunkRoutes / kThreads];
#pragma unroll
    for (int b = 0; b < kChunkRoutes / kThreads; ++b) {
        const int i = chunk * kChunkRoutes + wave * (kChunkRoutes / kWavesPerBlock) + b * kWave + lane;
        int key = -1;
        if (i < n && i < liveLimit) {
            const int e = a.ids[i];
            bool live = e >= 0 && e < a.numExperts;
            if (a.maskMode == kMaskPerToken) {
                live = live && a.mask[i / a.topK] != 0;
            } else if (a.maskMode == kMaskPerRoute) {
                live = live && a.mask[i] != 0;
            }
            if (live) {
                key = e / a.keyDiv;
                atomicAdd(&s_cnt[wave * a.numKeys + key], 1);
                if (expHist) {
                    atomicAdd(&s_exp[e], 1);
                }
            }
        }
        keys[b] = key;
    }
    __syncthreads();

    // phase B: exclusive sum over the four waves; chunk totals to HBM
    for (int key = tid; key < a.numKeys; key += kThreads) {
        int run = 0;
#pragma unroll
        for (int w = 0; w < kWavesPerBlock; ++w) {
            const int v = s_cnt[w * a.numKeys + key];
            s_cnt[w * a.numKeys + key] = run;
            run += v;
        }
        a.s.chunkHist[static_cast<int64_t>(chunk) * a.numKeys + key] = run;
    }
    if (expHist) {
        for (int e = tid; e < a.numExperts; e += kThreads) {
            a.s.chunkExpHist[static_cast<int64_t>(chunk) * a.numExperts + e] = s_exp[e];
        }
    }
    __syncthreads();

    // phase C: batches of 64 routes in order; lanes with equal keys find each other with one ballot per key bit
    volatile int *cnt = s_cnt + wave * a.numKeys;
    const unsigned long long lt = LaneMaskLt();
#pragma unroll
    for (int b = 0; b < kChunkRoutes / kThreads; ++b) {
        const int i = chunk * kChunkRoutes + wave * (kChunkRoutes / kWavesPerBlock) + b * kWave + lane;
        const int key = keys[b];
        const bool live = key >= 0;
        unsigned long long peers = __ballot(live);
        for (int bit = 0; bit < a.keyBits; ++bit) {
            const bool one = live && ((key >> bit) & 1);
            const unsigned long long bal = __ballot(one);
            peers &= one ? bal : ~bal;
        }
        const int before = __popcll(peers & lt);
        const int base = live ? cnt[key] : 0;
        if (i < n) {
            a.s.localRank[i] = live ? base + before : -1;
        }
        __builtin_amdgcn_wave_barrier();
        if (live && before == 0) {
            cnt[key] = base + __popcll(peers);
        }
        __builtin_amdgcn_wave_barrier();
    }

    // last workgroup to arrive performs the scans
    __threadfence();
    __syncthreads();
    if (tid == 0) {
        const unsigned prev = atomicAdd(a.s.ticket, 1u);
        s_misc[1] = prev == static_cast<unsigned>(a.numChunks - 1) ? 1 : 0;
    }
    __syncthreads();
    if (s_misc[1] == 0) {
        return;
    }
    __threadfence();

    // per key: exclusive sum over chunks (becomes the chunk's base rank within the key), total, kept
    int *kept = s_cnt;                 // reuse: [numKeys]
    for (int key = tid; key < a.numKeys; key += kThreads) {
        int run = 0;
        for (int c = 0; c < a.numChunks; ++c) {
            const int64_t at = static_cast<int64_t>(c) * a.numKeys + key;
            const int v = a.s.chunkHist[at];
            a.s.chunkHist[at] = run;
            run += v;
        }
        const int k = (a.capacity > 0 && run > a.capacity) ? a.capacity : run;
        kept[key] = k;
        a.s.keyKept[key] = k;
    }
    __syncthreads();
    int *offs = s_cnt + kMaxKeys;      // [numKeys] exclusive offsets
    for (int key = tid; key < a.numKeys; key += kThreads) {
        offs[key] = kept[key];
    }
    __syncthreads();
    const int totalRows = BlockExclusiveScan(offs, a.numKeys, s_part);
    for (int key = tid; key < a.numKeys; key += kThreads) {
        a.s.keyOffset[key] = offs[key];
        if (a.sendCountsOut != nullptr) {
            a.sendCountsOut[key] = offs[key] + kept[key];
        }
    }
    if (tid == 0) {
        a.s.keyOffset[a.numKeys] = totalRows;
        if (a.recvCountOut != nullptr) {
            a.recvCountOut[0] = totalRows;
        }
    }

    // per expert totals
    //   keys == experts: rows kept per expert (reference: tilexr_ep_dispatch_memory_kernel.h:1159-1168)
    //   coarser keys:    live routes per expert (reference: tilexr_ep_combine_helpers.h:49-80)
    int *etot = s_cnt + 2 * kMaxKeys;  // [numExperts]
    if (expHist) {
        for (int e = tid; e < a.numExperts; e += kThreads) {
            int run = 0;
            for (int c = 0; c < a.numChunks; ++c) {
                run += a.s.chunkExpHist[static_cast<int64_t>(c) * a.numExperts + e];
            }
            etot[e] = run;
        }
    } else {
        for (int e = tid; e < a.numExperts; e += kThreads) {
            etot[e] = e < a.numKeys ? kept[e] : 0;
        }
    }
    __syncthreads();
    for (int e = tid; e < a.numExperts; e += kThreads) {
        a.s.expertTotal[e] = etot[e];
    }
    if (a.expertTokenNumsOut != nullptr) {
        if (a.tokenNumsType == 0) {
            int *pref = s_cnt + 3 * kMaxKeys;
            for (int e = tid; e < a.numExperts; e += kThreads) {
                pref[e] = etot[e];
            }
            __syncthreads();
            BlockExclusiveScan(pref, a.numExperts, s_part);
            for (int e = tid; e < a.numExperts; e += kThreads) {
                a.expertTokenNumsOut[e] = static_cast<int64_t>(pref[e]) + etot[e];
            }
        } else {
            for (int e = tid; e < a.numExperts; e += kThreads) {
                a.expertTokenNumsOut[e] = etot[e];
            }
        }
    }
    if (tid == 0) {
        *a.s.ticket = 0u;
    }
}

// -------------------------------------------------------------------------------------------------------------
// place: destination row of every route + assist tuple + inverse map + tile-flag reset.
//   row   = keyOffset[key] + (rank of the route within its key), routes at or beyond `capacity` get none
//   tuple = {srcRank, token, k, expert id} (reference: src/ep/common/ep_window.h:47-52,
//           tilexr_ep_dispatch_memory_kernel.h:1240-1258)
// -------------------------------------------------------------------------------------------------------------
struct RoutePlaceArgs {
    const int32_t *ids;
    int n;
    int topK;
    int keyDiv;
    int numKeys;
    int capacity;
    CountScratch s;
    int32_t srcRank;
    int32_t expertIdBias;
    int32_t *rowOf;
    int32_t *assist;
    uint64_t *tileFlags;
    int numTiles;
    uint64_t epoch;
};

__global__ __launch_bounds__(kThreads) void ep_route_place_kernel(RoutePlaceArgs a)
{
    const int i = blockIdx.x * kThreads + threadIdx.x;
    if (a.tileFlags != nullptr) {
        for (int f = i; f < a.numTiles; f += gridDim.x * kThreads) {
            a.tileFlags[f] = a.epoch << 32;
        }
    }
    if (i >= a.n) {
        return;
    }
    const int lr = a.s.localRank[i];
    int row = -1;
    if (lr >= 0) {
        const int e = a.ids[i];
        const int key = e / a.keyDiv;
        const int within = a.s.chunkHist[static_cast<int64_t>(i / kChunkRoutes) * a.numKeys + key] + lr;
        if (a.capacity <= 0 || within < a.capacity) {
            row = a.s.keyOffset[key] + within;
            int32_t *tuple = a.assist + static_cast<int64_t>(row) * 4;
            tuple[0] = a.srcRank;
            tuple[1] = i / a.topK;
            tuple[2] = i % a.topK;
            tuple[3] = e + a.expertIdBias;
        }
    }
    a.rowOf[i] = row;
}

// -------------------------------------------------------------------------------------------------------------
// scatter: each token row is read once and written to the rows its routes were placed at.
// G lanes cooperate on one token (a wave for narrow rows, the whole workgroup for wide ones); a lane keeps up to
// kVecMax 16-byte vectors of the row in registers, so all loads of a row are in flight before the first store.
//   QMODE 0  byte copy             (reference: tilexr_ep_dispatch_helpers.h:104-112)
//   QMODE 1  static int8           (reference: tilexr_ep_dispatch_helpers.h:114-136)
//   QMODE 2  per-token int8        (reference: tilexr_ep_dispatch_helpers.h:153-191; BF16 decode has no counterpart)
//   QMODE 4  MXFP8, 32-wide blocks (reference: tests/ep/demo/mxfp8_golden.h:116-152)
//   QMODE 5  fp8 e4m3, fp32 scale per 128 columns (no reference counterpart)
// -------------------------------------------------------------------------------------------------------------
struct ScatterArgs {
    const void *x;
    const int32_t *rowOf;
    int bs;
    int h;
    int topK;
    const float *staticScale;
    void *out;
    void *scalesOut;
    uint64_t *tileFlags;
    int tileRows;
};

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

__device__ __forceinline__ void PublishRows(uint64_t *tileFlags, int tileRows, const int *pos, int topK, int lane, int G)
{
    // every lane's row stores are complete once the workgroup barrier has been passed; the release below makes
    // them visible at agent scope before the tile counter moves
    __syncthreads();
    for (int k = lane; k < topK; k += G) {
        const int row = pos[k];
        if (row >= 0) {
            __hip_atomic_fetch_add(&tileFlags[row / tileRows], 1ull, __ATOMIC_RELEASE, __HIP_MEMORY_SCOPE_AGENT);
        }
    }
}

template <int G, int QMODE, bool BF16, bool E5M2>
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
        s_pos[tg][k] = tokOk ? a.rowOf[static_cast<int64_t>(token) * a.topK + k] : -1;
    }
    const u32x4 *src = reinterpret_cast<const u32x4 *>(static_cast<const char *>(a.x) +
        static_cast<int64_t>(tokOk ? token : 0) * a.h * 2);
    u32x4 v[kVecMax];
#pragma unroll
    for (int j = 0; j < kVecMax; ++j) {
        const int idx = j * G + lane;
        if (tokOk && idx < vecs) {
            v[j] = __builtin_nontemporal_load(src + idx);
        } else {
            v[j] = u32x4{0u, 0u, 0u, 0u};
        }
    }
    __syncthreads();

    if (QMODE == TILEXR_EP_QUANT_NONE) {
        for (int k = 0; k < a.topK; ++k) {
            const int row = s_pos[tg][k];
            if (row < 0) {
                continue;
            }
            u32x4 *dst = reinterpret_cast<u32x4 *>(static_cast<char *>(a.out) + static_cast<int64_t>(row) * a.h * 2);
#pragma unroll
            for (int j = 0; j < kVecMax; ++j) {
                const int idx = j * G + lane;
                if (idx < vecs) {
                    __builtin_nontemporal_store(v[j], dst + idx);
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
            for (int j = 0; j < kVecMax; ++j) {
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
        u32x2 q[kVecMax];
        float blockScale[kVecMax];
        int sharedExp[kVecMax];
#pragma unroll
        for (int j = 0; j < kVecMax; ++j) {
            float f[8];
#pragma unroll
            for (int w = 0; w < 4; ++w) {
                f[2 * w] = Decode16<BF16>(v[j][w] & 0xffffu);
                f[2 * w + 1] = Decode16<BF16>(v[j][w] >> 16);
            }
            uint32_t bytes[8];
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
#pragma unroll
                    for (int e = 0; e < 8; ++e) {
                        bytes[e] = Fp8Encode<false>(__fdiv_rn(f[e], sc));
                    }
                }
            } else {
#pragma unroll
                for (int e = 0; e < 8; ++e) {
                    bytes[e] = static_cast<uint32_t>(ClampInt8(__fmul_rn(f[e], rowScaleInv))) & 0xffu;
                }
            }
            q[j][0] = bytes[0] | (bytes[1] << 8) | (bytes[2] << 16) | (bytes[3] << 24);
            q[j][1] = bytes[4] | (bytes[5] << 8) | (bytes[6] << 16) | (bytes[7] << 24);
        }
        const int mxScales = ((a.h + 31) / 32 + 1) / 2 * 2;
        const int b128 = (a.h + 127) / 128;
        for (int k = 0; k < a.topK; ++k) {
            const int row = s_pos[tg][k];
            if (row < 0) {
                continue;
            }
            u32x2 *dst = reinterpret_cast<u32x2 *>(static_cast<char *>(a.out) + static_cast<int64_t>(row) * a.h);
#pragma unroll
            for (int j = 0; j < kVecMax; ++j) {
                const int idx = j * G + lane;
                if (idx < vecs) {
                    __builtin_nontemporal_store(q[j], dst + idx);
                    if (QMODE == TILEXR_EP_QUANT_MXFP8 && (idx & 3) == 0) {
                        uint8_t *sc = static_cast<uint8_t *>(a.scalesOut) + static_cast<int64_t>(row) * mxScales;
                        sc[idx >> 2] = static_cast<uint8_t>(sharedExp[j] + 127);
                        if ((idx >> 2) + 1 == (a.h + 31) / 32 && ((idx >> 2) + 1) < mxScales) {
                            sc[(idx >> 2) + 1] = 0;     // padding byte of an odd block count
                        }
                    }
                    if (QMODE == TILEXR_EP_QUANT_FP8_BLOCK128 && (idx & 15) == 0) {
                        static_cast<float *>(a.scalesOut)[static_cast<int64_t>(row) * b128 + (idx >> 4)] = blockScale[j];
                    }
                }
            }
            if (QMODE == TILEXR_EP_QUANT_TOKEN_INT8 && lane == 0) {
                static_cast<float *>(a.scalesOut)[row] = rowScale;
            }
        }
    }
    if (a.tileFlags != nullptr) {
        PublishRows(a.tileFlags, a.tileRows, s_pos[tg], a.topK, lane, G);
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
        s_pos[k] = a.rowOf[static_cast<int64_t>(token) * a.topK + k];
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
        PublishRows(a.tileFlags, a.tileRows, s_pos, a.topK, tid, kThreads);
    }
}

// -------------------------------------------------------------------------------------------------------------
// invert: (token, k) -> row from the assist tuples, tagged with the call's epoch so the table never needs clearing.
//   memory route: rows [0, counts[last]) whose tuple names this rank and lies in range
//                 (reference: tilexr_ep_combine_memory_kernel.h:256-266, 329-342)
//   MVP route:    rows [0, sum of counts clamped to [0, maxCountPerEntry]); the tuple's rank field is not tested
//                 because the reference overwrites it while scattering (tilexr_ep_combine_kernel.cpp:28-52, 94-97)
// -------------------------------------------------------------------------------------------------------------
struct InvertArgs {
    const int32_t *assist;
    const int32_t *counts;
    int numCounts;
    int countsArePrefix;
    int maxRows;
    int maxCountPerEntry;
    int32_t rank;
    int bs;
    int topK;
    uint64_t epoch;
    uint64_t *inverse;
};

__global__ __launch_bounds__(kThreads) void ep_invert_kernel(InvertArgs a)
{
    __shared__ int s_rows;
    if (threadIdx.x == 0) {
        int rows = 0;
        if (a.countsArePrefix) {
            rows = a.counts[a.numCounts - 1];
        } else {
            for (int i = 0; i < a.numCounts; ++i) {
                const int c = a.counts[i];
                rows += (c < 0 || c > a.maxCountPerEntry) ? 0 : c;
            }
        }
        s_rows = rows < 0 ? 0 : (rows > a.maxRows ? a.maxRows : rows);
    }
    __syncthreads();
    const int row = blockIdx.x * kThreads + threadIdx.x;
    if (row >= s_rows) {
        return;
    }
    const int32_t *t = a.assist + static_cast<int64_t>(row) * 4;
    const int srcRank = t[0];
    const int token = t[1];
    const int k = t[2];
    if ((a.countsArePrefix && srcRank != a.rank) || token < 0 || token >= a.bs || k < 0 || k >= a.topK) {
        return;
    }
    a.inverse[static_cast<int64_t>(token) * a.topK + k] = (a.epoch << 32) | static_cast<uint32_t>(row);
}

// -------------------------------------------------------------------------------------------------------------
// reduce: y[token] = sum over the token's rows.
//   KIND fp32     sum = 0; for k = 0..K-1: sum = sum + (w_k * row_k) in fp32 (separate multiply and add), then the
//                 shared-expert row, then one round-to-nearest-even (saturating for fp16) to the output type;
//                 an inactive token (mask) gives zeros
//                 (reference: tilexr_ep_combine_memory_kernel.h:505-553, 555-571, 573-601, 632-662)
//   KIND per-add  rows in ascending row index; y = T(float(y) + float(row)) after every add
//                 (reference: tilexr_ep_combine_kernel.cpp:15-26, 54-101)
//   COMMQ 3/4     every row first takes the MXFP8 e5m2 / e4m3 round trip and is accumulated as
//                 ((fp8 * 2^(s-127)) * w) (reference: tilexr_ep_mxfp8_quant.h:286-352)
//   INQ 2/5       rows hold int8 / fp8 payloads that are dequantised with their scales and rounded to the element
//                 type first (no reference counterpart)
// -------------------------------------------------------------------------------------------------------------
struct ReduceArgs {
    const void *expertOut;
    int64_t rowBytes;
    const uint64_t *inverseTagged;
    uint64_t epoch;
    const int32_t *rowIndexMap;
    const float *expertScales;
    const uint8_t *tokenMask;
    const void *sharedExpertX;
    const float *inScales;
    int bs;
    int h;
    int topK;
    void *y;
    const uint64_t *tileFlags;
    int tileRows;
    const int32_t *totalRowsPtr;
    uint64_t flagEpoch;
    int64_t waitTimeoutTicks;
    int32_t *deviceStatus;
};

__device__ __forceinline__ int LookupRow(const ReduceArgs &a, int64_t slot)
{
    if (a.rowIndexMap != nullptr) {
        return a.rowIndexMap[slot];
    }
    const uint64_t e = a.inverseTagged[slot];
    return (e >> 32) == a.epoch ? static_cast<int>(e & 0xffffffffu) : -1;
}

// Bounded acquire-wait until the tile holding `row` has all its rows published for this epoch.
__device__ bool WaitTile(const ReduceArgs &a, int row)
{
    const int tile = row / a.tileRows;
    const int total = *a.totalRowsPtr;
    int need = total - tile * a.tileRows;
    need = need > a.tileRows ? a.tileRows : need;
    const uint64_t start = wall_clock64();
    while (true) {
        const uint64_t w = __hip_atomic_load(&a.tileFlags[tile], __ATOMIC_ACQUIRE, __HIP_MEMORY_SCOPE_AGENT);
        if ((w >> 32) == a.flagEpoch && static_cast<int>(w & 0xffffffffu) >= need) {
            return true;
        }
        if (static_cast<int64_t>(wall_clock64() - start) > a.waitTimeoutTicks) {
            return false;
        }
        __builtin_amdgcn_s_sleep(4);
    }
}

// Insertion sort of row indices, ascending, absent rows (-1) last.  K is small.
__device__ void SortRows(int *rows, int k)
{
    for (int i = 1; i < k; ++i) {
        const int v = rows[i];
        const unsigned kv = static_cast<unsigned>(v);      // -1 becomes the largest key
        int j = i - 1;
        while (j >= 0 && static_cast<unsigned>(rows[j]) > kv) {
            rows[j + 1] = rows[j];
            --j;
        }
        rows[j + 1] = v;
    }
}

template <int G, int KIND, int INQ, bool BF16, int COMMQ>
__global__ __launch_bounds__(kThreads) void ep_reduce_vec_kernel(ReduceArgs a)
{
    constexpr int kTokens = kThreads / G;
    constexpr bool kMx = COMMQ != 0;
    constexpr bool kCommE5m2 = COMMQ == TILEXR_EP_QUANT_COMM_MXFP8_E5M2;
    __shared__ int s_row[kTokens][kMaxTopK];
    __shared__ float s_w[kTokens][kMaxTopK];

    const int tg = threadIdx.x / G;
    const int lane = threadIdx.x % G;
    const int vecs = a.h / 8;
    const int groups = (a.bs + kTokens - 1) / kTokens;
    const int b128 = (a.h + 127) / 128;

    for (int group = blockIdx.x; group < groups; group += gridDim.x) {
        const int token = group * kTokens + tg;
        const bool tokOk = token < a.bs;
        __syncthreads();        // previous iteration's readers are done with s_row / s_w
        for (int k = lane; k < a.topK; k += G) {
            const int64_t slot = static_cast<int64_t>(tokOk ? token : 0) * a.topK + k;
            int row = tokOk ? LookupRow(a, slot) : -1;
            if (row >= 0 && a.tileFlags != nullptr && !WaitTile(a, row)) {
                if (a.deviceStatus != nullptr) {
                    atomicExch(a.deviceStatus, 1);
                }
                row = -1;
            }
            s_row[tg][k] = row;
            s_w[tg][k] = (tokOk && a.expertScales != nullptr) ? a.expertScales[slot] : 1.0f;
        }
        __syncthreads();
        if (KIND == kReducePerAdd) {
            if (lane == 0) {
                SortRows(s_row[tg], a.topK);
            }
            __syncthreads();
        }
        const bool active = tokOk && (a.tokenMask == nullptr || a.tokenMask[token] != 0);

#pragma unroll 1
        for (int j = 0; j < kVecMax; ++j) {
            const int idx = j * G + lane;
            if (j * G >= vecs) {
                break;                      // uniform across the group
            }
            const bool inRow = idx < vecs;
            float acc[8];
#pragma unroll
            for (int e = 0; e < 8; ++e) {
                acc[e] = 0.0f;
            }
            if (active || kMx) {
                for (int k = 0; k < a.topK; ++k) {
                    const int row = s_row[tg][k];
                    if (row < 0) {
                        continue;           // uniform across the group
                    }
                    const float w = s_w[tg][k];
                    float f[8];
                    if (INQ == 0) {
                        u32x4 v = u32x4{0u, 0u, 0u, 0u};
                        if (inRow && active) {
                            v = __builtin_nontemporal_load(reinterpret_cast<const u32x4 *>(
                                static_cast<const char *>(a.expertOut) + static_cast<int64_t>(row) * a.rowBytes) + idx);
                        }
#pragma unroll
                        for (int q = 0; q < 4; ++q) {
                            f[2 * q] = Decode16<BF16>(v[q] & 0xffffu);
                            f[2 * q + 1] = Decode16<BF16>(v[q] >> 16);
                        }
                    } else {
                        u32x2 v = u32x2{0u, 0u};
                        float sc = 0.0f;
                        if (inRow && active) {
                            v = __builtin_nontemporal_load(reinterpret_cast<const u32x2 *>(
                                static_cast<const char *>(a.expertOut) + static_cast<int64_t>(row) * a.rowBytes) + idx);
                            sc = INQ == TILEXR_EP_QUANT_TOKEN_INT8 ? a.inScales[row] :
                                a.inScales[static_cast<int64_t>(row) * b128 + (idx >> 4)];
                        }
#pragma unroll
                        for (int e = 0; e < 8; ++e) {
                            const uint32_t byte = (v[e >> 2] >> ((e & 3) * 8)) & 0xffu;
                            const float d = INQ == TILEXR_EP_QUANT_TOKEN_INT8 ?
                                __fmul_rn(static_cast<float>(static_cast<int>(static_cast<int8_t>(byte))), sc) :
                                __fmul_rn(Fp8Decode<false>(byte), sc);
                            f[e] = BF16 ? __uint_as_float(FloatToBf16Rne(d) << 16) :
                                          __half2float(__ushort_as_half(static_cast<unsigned short>(FloatToHalfRneSat(d))));
                        }
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
                            acc[e] = RoundTo16<BF16>(__fadd_rn(acc[e], f[e]));
                        }
                    } else {
#pragma unroll
                        for (int e = 0; e < 8; ++e) {
                            acc[e] = __fadd_rn(acc[e], __fmul_rn(f[e], w));
                        }
                    }
                }
                if (a.sharedExpertX != nullptr && inRow && active) {
                    const u32x4 v = *(reinterpret_cast<const u32x4 *>(static_cast<const char *>(a.sharedExpertX) +
                        static_cast<int64_t>(token) * a.h * 2) + idx);
#pragma unroll
                    for (int q = 0; q < 4; ++q) {
                        acc[2 * q] = __fadd_rn(acc[2 * q], Decode16<BF16>(v[q] & 0xffffu));
                        acc[2 * q + 1] = __fadd_rn(acc[2 * q + 1], Decode16<BF16>(v[q] >> 16));
                    }
                }
            }
            if (tokOk && inRow) {
                u32x4 o;
#pragma unroll
                for (int q = 0; q < 4; ++q) {
                    const uint32_t lo = active ? Encode16Sat<BF16>(acc[2 * q]) : 0u;
                    const uint32_t hi = active ? Encode16Sat<BF16>(acc[2 * q + 1]) : 0u;
                    o[q] = lo | (hi << 16);
                }
                __builtin_nontemporal_store(o, reinterpret_cast<u32x4 *>(static_cast<char *>(a.y) +
                    static_cast<int64_t>(token) * a.h * 2) + idx);
            }
        }
    }
}

// Element-granular reduce for any h / alignment.  One workgroup per token.
template <bool BF16>
__global__ __launch_bounds__(kThreads) void ep_reduce_generic_kernel(ReduceArgs a, int kind, int inq, int commq)
{
    __shared__ int s_row[kMaxTopK];
    __shared__ float s_w[kMaxTopK];
    const int tid = threadIdx.x;
    const int b128 = (a.h + 127) / 128;
    for (int token = blockIdx.x; token < a.bs; token += gridDim.x) {
        __syncthreads();
        for (int k = tid; k < a.topK; k += kThreads) {
            const int64_t slot = static_cast<int64_t>(token) * a.topK + k;
            int row = LookupRow(a, slot);
            if (row >= 0 && a.tileFlags != nullptr && !WaitTile(a, row)) {
                if (a.deviceStatus != nullptr) {
                    atomicExch(a.deviceStatus, 1);
                }
                row = -1;
            }
            s_row[k] = row;
            s_w[k] = a.expertScales != nullptr ? a.expertScales[slot] : 1.0f;
        }
        __syncthreads();
        if (kind == kReducePerAdd) {
            if (tid == 0) {
                SortRows(s_row, a.topK);
            }
            __syncthreads();
        }
        const bool active = a.tokenMask == nullptr || a.tokenMask[token] != 0;
        uint16_t *dst = static_cast<uint16_t *>(a.y) + static_cast<int64_t>(token) * a.h;
        // a thread owns whole 32-column blocks so that the MXFP8 round trip needs no cross-lane traffic
        const int blocks = (a.h + 31) / 32;
        for (int b = tid; b < blocks; b += kThreads) {
            const int begin = b * 32;
            const int end = min(begin + 32, a.h);
            float acc[32];
            for (int i = 0; i < 32; ++i) {
                acc[i] = 0.0f;
            }
            if (active) {
                for (int k = 0; k < a.topK; ++k) {
                    const int row = s_row[k];
                    if (row < 0) {
                        continue;
                    }
                    const float w = s_w[k];
                    const char *base = static_cast<const char *>(a.expertOut) + static_cast<int64_t>(row) * a.rowBytes;
                    float f[32];
                    float amax = 0.0f;
                    for (int i = begin; i < end; ++i) {
                        float v;
                        if (inq == 0) {
                            v = Decode16<BF16>(reinterpret_cast<const uint16_t *>(base)[i]);
                        } else {
                            const uint32_t byte = reinterpret_cast<const uint8_t *>(base)[i];
                            const float d = inq == TILEXR_EP_QUANT_TOKEN_INT8 ?
                                __fmul_rn(static_cast<float>(static_cast<int>(static_cast<int8_t>(byte))), a.inScales[row]) :
                                __fmul_rn(Fp8Decode<false>(byte), a.inScales[static_cast<int64_t>(row) * b128 + i / 128]);
                            v = BF16 ? __uint_as_float(FloatToBf16Rne(d) << 16) :
                                       __half2float(__ushort_as_half(static_cast<unsigned short>(FloatToHalfRneSat(d))));
                        }
                        f[i - begin] = v;
                        amax = fmaxf(amax, fabsf(v));
                    }
                    if (commq != 0) {
                        const bool e5 = commq == TILEXR_EP_QUANT_COMM_MXFP8_E5M2;
                        const int se = e5 ? MxSharedExponent<true>(amax) : MxSharedExponent<false>(amax);
                        const float up = Exp2Int(se);
                        for (int i = 0; i < end - begin; ++i) {
                            const float s = ldexpf(f[i], -se);
                            const float back = e5 ? Fp8Decode<true>(Fp8Encode<true>(s)) : Fp8Decode<false>(Fp8Encode<false>(s));
                            f[i] = __fmul_rn(back, up);
                        }
                    }
                    for (int i = 0; i < end - begin; ++i) {
                        if (kind == kReducePerAdd) {
                            acc[i] = RoundTo16<BF16>(__fadd_rn(acc[i], f[i]));
                        } else {
                            acc[i] = __fadd_rn(acc[i], __fmul_rn(f[i], w));
                        }
                    }
                }
                if (a.sharedExpertX != nullptr) {
                    const uint16_t *sx = static_cast<const uint16_t *>(a.sharedExpertX) + static_cast<int64_t>(token) * a.h;
                    for (int i = begin; i < end; ++i) {
                        acc[i - begin] = __fadd_rn(acc[i - begin], Decode16<BF16>(sx[i]));
                    }
                }
            }
            for (int i = begin; i < end; ++i) {
                dst[i] = active ? static_cast<uint16_t>(Encode16Sat<BF16>(acc[i - begin])) : static_cast<uint16_t>(0);
            }
        }
    }
}

inline bool Aligned16(const void *p)
{
    return (reinterpret_cast<uintptr_t>(p) & 15u) == 0;
}

int KeyBits(int64_t numKeys)
{
    int bits = 0;
    while ((1ll << bits) < numKeys) {
        ++bits;
    }
    return bits;
}

} // namespace

// -------------------------------------------------------------------------------------------------------------
// host-side launchers
// -------------------------------------------------------------------------------------------------------------
CountScratchLayout PlanCountScratch(int64_t routes, int64_t numKeys, int64_t numExperts, bool expertHist)
{
    auto align = [](int64_t v) { return (v + 255) / 256 * 256; };
    CountScratchLayout p {};
    p.chunks = (routes + kChunkRoutes - 1) / kChunkRoutes;
    int64_t off = 256;   // word 0 is the ticket
    p.localRankOff = off;
    off += align(routes * 4);
    p.rowOfOff = off;
    off += align(routes * 4);
    p.chunkHistOff = off;
    off += align(p.chunks * numKeys * 4);
    p.chunkExpHistOff = off;
    off += expertHist ? align(p.chunks * numExperts * 4) : 0;
    p.keyOffsetOff = off;
    off += align((numKeys + 1) * 4);
    p.keyKeptOff = off;
    off += align(numKeys * 4);
    p.expertTotalOff = off;
    off += align(numExperts * 4);
    p.totalBytes = off;
    return p;
}

hipError_t LaunchRouteCount(const RouteCountLaunch &l)
{
    RouteCountArgs a {};
    a.ids = l.ids;
    a.mask = l.mask;
    a.maskMode = l.maskMode;
    a.bs = static_cast<int>(l.bs);
    a.topK = static_cast<int>(l.topK);
    a.numExperts = static_cast<int>(l.numExperts);
    a.keyDiv = static_cast<int>(l.keyDiv);
    a.numKeys = static_cast<int>(l.numKeys);
    a.keyBits = KeyBits(l.numKeys);
    a.capacity = static_cast<int>(l.capacity);
    const int64_t n = l.bs * l.topK;
    a.numChunks = static_cast<int>((n + kChunkRoutes - 1) / kChunkRoutes);
    a.s = l.scratch;
    a.sendCountsOut = l.sendCountsOut;
    a.recvCountOut = l.recvCountOut;
    a.expertTokenNumsOut = l.expertTokenNumsOut;
    a.tokenNumsType = l.tokenNumsType;
    hipLaunchKernelGGL(ep_route_count_kernel, dim3(a.numChunks), dim3(kThreads), 0, l.stream, a);
    return hipGetLastError();
}

hipError_t LaunchRoutePlace(const RoutePlaceLaunch &l)
{
    RoutePlaceArgs a {};
    a.ids = l.ids;
    a.n = static_cast<int>(l.bs * l.topK);
    a.topK = static_cast<int>(l.topK);
    a.keyDiv = static_cast<int>(l.keyDiv);
    a.numKeys = static_cast<int>(l.numKeys);
    a.capacity = static_cast<int>(l.capacity);
    a.s = l.scratch;
    a.srcRank = l.srcRank;
    a.expertIdBias = l.expertIdBias;
    a.rowOf = l.rowOf;
    a.assist = l.assist;
    a.tileFlags = l.tileFlags;
    a.numTiles = static_cast<int>(l.numTiles);
    a.epoch = l.epoch;
    const int grid = (a.n + kThreads - 1) / kThreads;
    hipLaunchKernelGGL(ep_route_place_kernel, dim3(grid), dim3(kThreads), 0, l.stream, a);
    return hipGetLastError();
}

namespace {

template <int G, int QMODE, bool BF16, bool E5M2>
void LaunchScatterVec(const ScatterArgs &a, hipStream_t stream)
{
    constexpr int kTokens = kThreads / G;
    const int grid = (a.bs + kTokens - 1) / kTokens;
    hipLaunchKernelGGL((ep_scatter_vec_kernel<G, QMODE, BF16, E5M2>), dim3(grid), dim3(kThreads), 0, stream, a);
}

template <int G>
void DispatchScatterVec(const ScatterLaunch &l, const ScatterArgs &a)
{
    switch (l.quantMode) {
        case TILEXR_EP_QUANT_NONE:
            LaunchScatterVec<G, TILEXR_EP_QUANT_NONE, true, false>(a, l.stream);
            break;
        case TILEXR_EP_QUANT_STATIC_INT8:
            LaunchScatterVec<G, TILEXR_EP_QUANT_STATIC_INT8, false, false>(a, l.stream);
            break;
        case TILEXR_EP_QUANT_TOKEN_INT8:
            if (l.inputBf16) {
                LaunchScatterVec<G, TILEXR_EP_QUANT_TOKEN_INT8, true, false>(a, l.stream);
            } else {
                LaunchScatterVec<G, TILEXR_EP_QUANT_TOKEN_INT8, false, false>(a, l.stream);
            }
            break;
        case TILEXR_EP_QUANT_MXFP8:
            if (l.inputBf16) {
                if (l.fp8E5m2) {
                    LaunchScatterVec<G, TILEXR_EP_QUANT_MXFP8, true, true>(a, l.stream);
                } else {
                    LaunchScatterVec<G, TILEXR_EP_QUANT_MXFP8, true, false>(a, l.stream);
                }
            } else {
                if (l.fp8E5m2) {
                    LaunchScatterVec<G, TILEXR_EP_QUANT_MXFP8, false, true>(a, l.stream);
                } else {
                    LaunchScatterVec<G, TILEXR_EP_QUANT_MXFP8, false, false>(a, l.stream);
                }
            }
            break;
        default:
            if (l.inputBf16) {
                LaunchScatterVec<G, TILEXR_EP_QUANT_FP8_BLOCK128, true, false>(a, l.stream);
            } else {
                LaunchScatterVec<G, TILEXR_EP_QUANT_FP8_BLOCK128, false, false>(a, l.stream);
            }
            break;
    }
}

} // namespace

hipError_t LaunchScatter(const ScatterLaunch &l)
{
    ScatterArgs a {};
    a.x = l.x;
    a.rowOf = l.rowOf;
    a.bs = static_cast<int>(l.bs);
    a.h = static_cast<int>(l.h);
    a.topK = static_cast<int>(l.topK);
    a.staticScale = l.staticScale;
    a.out = l.out;
    a.scalesOut = l.scalesOut;
    a.tileFlags = l.tileFlags;
    a.tileRows = static_cast<int>(l.tileRows);
    const int64_t vecs = l.h / 8;
    const bool vecOk = l.h % 8 == 0 && Aligned16(l.x) && Aligned16(l.out) && vecs <= static_cast<int64_t>(kVecMax) * kThreads &&
        (l.quantMode == TILEXR_EP_QUANT_NONE || (reinterpret_cast<uintptr_t>(l.out) & 7u) == 0);
    if (vecOk) {
        if (vecs <= static_cast<int64_t>(kVecMax / 2) * kWave) {
            DispatchScatterVec<kWave>(l, a);        // narrow rows: one wave per token, four tokens per workgroup
        } else {
            DispatchScatterVec<kThreads>(l, a);
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

hipError_t LaunchInvert(const InvertLaunch &l)
{
    InvertArgs a {};
    a.assist = l.assist;
    a.counts = l.counts;
    a.numCounts = static_cast<int>(l.numCounts);
    a.countsArePrefix = l.countsArePrefix ? 1 : 0;
    a.maxRows = static_cast<int>(l.maxRows);
    a.maxCountPerEntry = static_cast<int>(l.maxCountPerEntry);
    a.rank = l.rank;
    a.bs = static_cast<int>(l.bs);
    a.topK = static_cast<int>(l.topK);
    a.epoch = l.epoch;
    a.inverse = l.inverse;
    const int grid = static_cast<int>((l.maxRows + kThreads - 1) / kThreads);
    hipLaunchKernelGGL(ep_invert_kernel, dim3(grid > 0 ? grid : 1), dim3(kThreads), 0, l.stream, a);
    return hipGetLastError();
}

namespace {

template <int G, int KIND, int INQ, bool BF16, int COMMQ>
void LaunchReduceVec(const ReduceArgs &a, int gridLimit, hipStream_t stream)
{
    constexpr int kTokens = kThreads / G;
    int grid = (a.bs + kTokens - 1) / kTokens;
    if (gridLimit > 0 && grid > gridLimit) {
        grid = gridLimit;
    }
    hipLaunchKernelGGL((ep_reduce_vec_kernel<G, KIND, INQ, BF16, COMMQ>), dim3(grid), dim3(kThreads), 0, stream, a);
}

template <int G, bool BF16>
void DispatchReduceVec(const ReduceLaunch &l, const ReduceArgs &a, int gridLimit)
{
    if (l.reduceKind == kReducePerAdd) {
        LaunchReduceVec<G, kReducePerAdd, 0, BF16, 0>(a, gridLimit, l.stream);
    } else if (l.inQuant == TILEXR_EP_QUANT_TOKEN_INT8) {
        LaunchReduceVec<G, kReduceFp32, TILEXR_EP_QUANT_TOKEN_INT8, BF16, 0>(a, gridLimit, l.stream);
    } else if (l.inQuant == TILEXR_EP_QUANT_FP8_BLOCK128) {
        LaunchReduceVec<G, kReduceFp32, TILEXR_EP_QUANT_FP8_BLOCK128, BF16, 0>(a, gridLimit, l.stream);
    } else if (l.commQuant == TILEXR_EP_QUANT_COMM_MXFP8_E5M2) {
        LaunchReduceVec<G, kReduceFp32, 0, BF16, TILEXR_EP_QUANT_COMM_MXFP8_E5M2>(a, gridLimit, l.stream);
    } else if (l.commQuant == TILEXR_EP_QUANT_MXFP8) {
        LaunchReduceVec<G, kReduceFp32, 0, BF16, TILEXR_EP_QUANT_MXFP8>(a, gridLimit, l.stream);
    } else {
        LaunchReduceVec<G, kReduceFp32, 0, BF16, 0>(a, gridLimit, l.stream);
    }
}

} // namespace

hipError_t LaunchReduce(const ReduceLaunch &l)
{
    ReduceArgs a {};
    a.expertOut = l.expertOut;
    a.rowBytes = l.rowBytes;
    a.inverseTagged = l.inverseTagged;
    a.epoch = l.epoch;
    a.rowIndexMap = l.rowIndexMap;
    a.expertScales = l.expertScales;
    a.tokenMask = l.tokenMask;
    a.sharedExpertX = l.sharedExpertX;
    a.inScales = l.inScales;
    a.bs = static_cast<int>(l.bs);
    a.h = static_cast<int>(l.h);
    a.topK = static_cast<int>(l.topK);
    a.y = l.y;
    a.tileFlags = l.tileFlags;
    a.tileRows = static_cast<int>(l.tileRows);
    a.totalRowsPtr = l.totalRowsPtr;
    a.flagEpoch = l.flagEpoch;
    a.waitTimeoutTicks = l.waitTimeoutTicks;
    a.deviceStatus = l.deviceStatus;
    // A kernel that waits on flags must never crowd out the producer it waits for: keep it to two workgroups per
    // compute unit (8 of 32 wave slots) and let it walk the tokens.
    const int gridLimit = l.tileFlags != nullptr ? 2 * (l.numComputeUnits > 0 ? l.numComputeUnits : 256) : 0;
    const int64_t vecs = l.h / 8;
    const bool mixed = (l.inQuant != 0 && l.commQuant != 0);
    const bool vecOk = !mixed && l.h % 8 == 0 && Aligned16(l.y) && vecs <= static_cast<int64_t>(kVecMax) * kThreads &&
        (l.inQuant == 0 ? (Aligned16(l.expertOut) && l.rowBytes % 16 == 0) :
                          ((reinterpret_cast<uintptr_t>(l.expertOut) & 7u) == 0 && l.rowBytes % 8 == 0)) &&
        (l.sharedExpertX == nullptr || Aligned16(l.sharedExpertX)) &&
        (l.commQuant == 0 || l.h % 32 == 0);
    if (vecOk) {
        if (vecs <= static_cast<int64_t>(kVecMax / 2) * kWave) {
            if (l.bf16) {
                DispatchReduceVec<kWave, true>(l, a, gridLimit);
            } else {
                DispatchReduceVec<kWave, false>(l, a, gridLimit);
            }
        } else {
            if (l.bf16) {
                DispatchReduceVec<kThreads, true>(l, a, gridLimit);
            } else {
                DispatchReduceVec<kThreads, false>(l, a, gridLimit);
            }
        }
    } else {
        int grid = static_cast<int>(l.bs);
        if (gridLimit > 0 && grid > gridLimit) {
            grid = gridLimit;
        }
        if (l.bf16) {
            hipLaunchKernelGGL((ep_reduce_generic_kernel<true>), dim3(grid), dim3(kThreads), 0, l.stream, a,
                l.reduceKind, l.inQuant, l.commQuant);
        } else {
            hipLaunchKernelGGL((ep_reduce_generic_kernel<false>), dim3(grid), dim3(kThreads), 0, l.stream, a,
                l.reduceKind, l.inQuant, l.commQuant);
        }
    }
    return hipGetLastError();
}

} // namespace TileXREp
