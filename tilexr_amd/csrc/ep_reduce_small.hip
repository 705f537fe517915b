// reduce of a small batch straight from the assist table (gfx950, wave64): one launch per combine.
//
// The reference's combine entry points carry no row map: combine finds the row of every (token, k) in the assist
// tuples (memory route: tilexr_ep_combine_memory_kernel.h:256-266, 329-342; MVP route: tilexr_ep_combine_kernel.cpp:28-52,
// 94-97).  For larger calls a first launch inverts the table (ep_invert_kernel); at decode size that launch costs as
// much as half the reduce, and the table is so small (2048 tuples at most, 32 KiB) that a token's workgroup can read all
// of it in the time the inverse's look-up would have taken: one trip to memory for the tuples, the gate weights and the
// number of rows together, then all of the token's rows at once, then the store.
//
// One workgroup per token (workgroup b runs on XCD b % 8, where the single-launch dispatch ran the token's routes: rows
// that still sit in that XCD's L2 are read there); wave w sums vectors [128 w, 128 w + 128) of the row, eight rows in
// flight per lane; waves beyond the row's end only help with the table.  The sums are those of ep_reduce_vec_kernel:
//   KIND fp32     sum = 0; for k = 0..K-1: sum = sum + (w_k * row_k) in fp32, then the shared-expert row, one rounding
//                 (saturating for fp16); an inactive token (mask) gives zeros
//                 (reference: src/ep/kernels/tilexr_ep_combine_memory_kernel.h:505-553, 555-571, 573-601, 632-662)
//   KIND per-add  rows in ascending row index; y = T(float(y) + float(row)) after every add
//                 (reference: src/ep/kernels/tilexr_ep_combine_kernel.cpp:15-26, 54-101)
// Two tuples that name the same (token, k) -- only a corrupted table has them -- leave the higher row, as the
// reference's sequential walk does and as ep_invert_kernel does.
#include <hip/hip_runtime.h>

#include "ep_reduce_common.hip.h"

namespace TileXREp {
namespace {

constexpr int kSmallReduceThreads = 1024;
constexpr int kSmallReduceVecs = 2;         // 16-byte vectors per lane
constexpr int kSmallReduceRows = 8;         // rows in flight per lane
constexpr int kScanBatch = 4;               // tuples a lane has in flight
constexpr int kScanWaves = 4;               // a workgroup has at least this many waves for the table
// Every token's workgroup reads the whole table, so the launch reads tokens x tuples of it in all: up to a million the
// reading costs less than the launch that would invert the table (512 tokens x 2048 tuples: 0.8 us over the reduce that is
// handed a row map, against 2.6 us for that launch), beyond that more (1024 x 2048: 3.4 us, 2048 x 2048: 8.6 us).
constexpr int64_t kSmallScanTuples = int64_t{1} << 20;

struct SmallReduceArgs {
    const void *expertOut;
    const int32_t *assist;          // [n, 4]
    const int32_t *counts;
    int lastCount;                  // index of the word that says how many rows the table holds
    int countsArePrefix;            // memory route: that word is the total; MVP route: one count, out of range reads as 0
    int32_t rank;
    const float *expertScales;      // optional [bs, topK]
    const uint8_t *tokenMask;       // optional [bs]
    const void *sharedExpertX;      // optional [bs, h]
    void *y;
    int h;
    int topK;
    int n;                          // bs * topK
};

template <int KIND, bool BF16>
__global__ __launch_bounds__(kSmallReduceThreads) void ep_reduce_small_kernel(SmallReduceArgs a)
{
    constexpr int V = kSmallReduceVecs;
    constexpr int KB = kSmallReduceRows;
    __shared__ int s_row[kMaxTopK];

    const int token = blockIdx.x;
    const int tid = threadIdx.x;
    const int lane = tid % kWave;
    const int wave = tid / kWave;
    const int vecs = a.h / 8;

    // asked for together: the gate weight of slot `lane`, the number of rows the table holds, the lane's tuples
    float myWeight = 1.0f;
    if (KIND == kReduceFp32 && a.expertScales != nullptr && lane < a.topK) {
        myWeight = a.expertScales[static_cast<int64_t>(token) * a.topK + lane];
    }
    const int held = a.counts[a.lastCount];
    const bool active = a.tokenMask == nullptr || a.tokenMask[token] != 0;
    if (tid < kMaxTopK) {
        s_row[tid] = -1;
    }
    __syncthreads();
    // a tuple beyond the table's end reads as zeros and is beyond `rows` as well
    const __amdgpu_buffer_rsrc_t table = RowResource(a.assist, a.n * 16);
    const int stride = static_cast<int>(blockDim.x);
    for (int first = 0; first < a.n; first += stride * kScanBatch) {
        u32x4 t[kScanBatch];
#pragma unroll
        for (int u = 0; u < kScanBatch; ++u) {
            t[u] = __builtin_amdgcn_raw_buffer_load_b128(table, (first + u * stride + tid) * 16, 0, 0);
        }
        int rows = held;
        if (!a.countsArePrefix && (held < 0 || held > a.n)) {
            rows = 0;
        }
        rows = rows < 0 ? 0 : (rows > a.n ? a.n : rows);
#pragma unroll
        for (int u = 0; u < kScanBatch; ++u) {
            const int row = first + u * stride + tid;
            const bool mine = row < rows && (!a.countsArePrefix || static_cast<int32_t>(t[u][0]) == a.rank) &&
                static_cast<int32_t>(t[u][1]) == token && t[u][2] < static_cast<uint32_t>(a.topK);
            if (mine) {
                atomicMax(&s_row[t[u][2]], row);
            }
        }
    }
    __syncthreads();
    if (KIND == kReducePerAdd) {
        if (tid == 0) {
            SortRows(s_row, a.topK, nullptr);
        }
        __syncthreads();
    }
    const int colBase = wave * (kWave * V);
    if (colBase >= vecs) {
        return;
    }
    // lane k keeps slot k's row and weight
    const int myRow = (lane < a.topK && active) ? s_row[lane] : -1;

    float acc[V][8];
#pragma unroll
    for (int j = 0; j < V; ++j) {
#pragma unroll
        for (int e = 0; e < 8; ++e) {
            acc[j][e] = 0.0f;
        }
    }
    for (int firstSlot = 0; firstSlot < a.topK; firstSlot += KB) {
        u32x4 v16[KB][V];
        int rowOfK[KB];
        float weightOfK[KB];
#pragma unroll
        for (int u = 0; u < KB; ++u) {
            const bool any = firstSlot + u < a.topK;
            const int k = any ? firstSlot + u : 0;
            const int row = any ? __builtin_amdgcn_readlane(myRow, k) : -1;
            rowOfK[u] = row;
            weightOfK[u] = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(myWeight), k));
            const char *base = static_cast<const char *>(a.expertOut) + static_cast<int64_t>(row < 0 ? 0 : row) * a.h * 2;
            // a slot without a row gets a resource of no bytes, and a lane beyond the row's end is beyond the resource's:
            // both read as zeros without a test per load (at this size the kernel is paid in instructions)
            const __amdgpu_buffer_rsrc_t rsrc = RowResource(base, row < 0 ? 0 : vecs * 16);
#pragma unroll
            for (int j = 0; j < V; ++j) {
                v16[u][j] = __builtin_amdgcn_raw_buffer_load_b128(rsrc, (colBase + j * kWave + lane) * 16, 0, kAuxNonTemporal);
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
#pragma unroll
                for (int q = 0; q < 4; ++q) {
                    const float lo = Decode16<BF16>(v16[u][j][q] & 0xffffu);
                    const float hi = Decode16<BF16>(v16[u][j][q] >> 16);
                    if (KIND == kReducePerAdd) {
                        acc[j][2 * q] = RoundTo16<BF16>(__fadd_rn(acc[j][2 * q], lo));
                        acc[j][2 * q + 1] = RoundTo16<BF16>(__fadd_rn(acc[j][2 * q + 1], hi));
                    } else {
                        acc[j][2 * q] = __fadd_rn(acc[j][2 * q], __fmul_rn(lo, w));
                        acc[j][2 * q + 1] = __fadd_rn(acc[j][2 * q + 1], __fmul_rn(hi, w));
                    }
                }
            }
        }
    }
    if (a.sharedExpertX != nullptr && active) {
        const u32x4 *sx = reinterpret_cast<const u32x4 *>(static_cast<const char *>(a.sharedExpertX) +
            static_cast<int64_t>(token) * a.h * 2);
#pragma unroll
        for (int j = 0; j < V; ++j) {
            const int idx = colBase + j * kWave + lane;
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
    u32x4 *dst = reinterpret_cast<u32x4 *>(static_cast<char *>(a.y) + static_cast<int64_t>(token) * a.h * 2);
#pragma unroll
    for (int j = 0; j < V; ++j) {
        const int idx = colBase + j * kWave + lane;
        if (idx < vecs) {
            u32x4 o;
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                o[q] = active ? EncodePair16Sat<BF16>(acc[j][2 * q], acc[j][2 * q + 1]) : 0u;
            }
            __builtin_nontemporal_store(o, dst + idx);
        }
    }
}

template <int KIND>
void LaunchByType(bool bf16, int grid, int threads, hipStream_t stream, const SmallReduceArgs &a)
{
    if (bf16) {
        hipLaunchKernelGGL((ep_reduce_small_kernel<KIND, true>), dim3(grid), dim3(threads), 0, stream, a);
    } else {
        hipLaunchKernelGGL((ep_reduce_small_kernel<KIND, false>), dim3(grid), dim3(threads), 0, stream, a);
    }
}

} // namespace

bool SmallReduceFits(const ReduceLaunch &l)
{
    const int64_t n = l.bs * l.topK;
    const int64_t vecs = l.h / 8;
    return l.assistTable != nullptr && l.rowIndexMap == nullptr && l.inverseTagged == nullptr && l.orderKeys == nullptr &&
        l.bs > 0 && n <= kSmallRoutes && l.bs * n <= kSmallScanTuples && l.topK <= kMaxTopK && l.sharedSlots == 0 && l.tileFlags == nullptr &&
        l.inQuant == 0 && l.commQuant == 0 && l.h % 8 == 0 && l.rowBytes == l.h * 2 &&
        vecs <= static_cast<int64_t>(kSmallReduceThreads / kWave) * kWave * kSmallReduceVecs &&
        l.assistTable->maxRows == n && l.assistTable->maxCountPerEntry == n && l.assistTable->bs == l.bs &&
        l.assistTable->topK == l.topK && (l.assistTable->countsArePrefix || l.assistTable->numCounts == 1) &&
        Aligned16(l.y) && Aligned16(l.expertOut) && Aligned16(l.assistTable->assist) &&
        (l.sharedExpertX == nullptr || Aligned16(l.sharedExpertX));
}

hipError_t LaunchSmallReduce(const ReduceLaunch &l)
{
    if (!SmallReduceFits(l)) {
        return hipErrorInvalidValue;
    }
    SmallReduceArgs a {};
    a.expertOut = l.expertOut;
    a.assist = l.assistTable->assist;
    a.counts = l.assistTable->counts;
    a.lastCount = static_cast<int>(l.assistTable->numCounts - 1);
    a.countsArePrefix = l.assistTable->countsArePrefix ? 1 : 0;
    a.rank = l.assistTable->rank;
    a.expertScales = l.expertScales;
    a.tokenMask = l.tokenMask;
    a.sharedExpertX = l.sharedExpertX;
    a.y = l.y;
    a.h = static_cast<int>(l.h);
    a.topK = static_cast<int>(l.topK);
    a.n = static_cast<int>(l.bs * l.topK);
    const int64_t vecs = l.h / 8;
    const int rowWaves = static_cast<int>((vecs + kWave * kSmallReduceVecs - 1) / (kWave * kSmallReduceVecs));
    const int threads = (rowWaves > kScanWaves ? rowWaves : kScanWaves) * kWave;
    if (l.kernelNameOut != nullptr) {
        *l.kernelNameOut = "ep_reduce_small_kernel";
    }
    if (l.reduceKind == kReducePerAdd) {
        LaunchByType<kReducePerAdd>(l.bf16, static_cast<int>(l.bs), threads, l.stream, a);
    } else {
        LaunchByType<kReduceFp32>(l.bf16, static_cast<int>(l.bs), threads, l.stream, a);
    }
    return hipGetLastError();
}

} // namespace TileXREp
