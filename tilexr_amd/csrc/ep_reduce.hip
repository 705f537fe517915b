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
// This file: the element-granular kernel for any width and alignment, and the choice of kernel and geometry.  The
// register-resident kernels are in ep_reduce_vec.hip.h and ep_reduce_quant.hip.h.
#include "ep_reduce_common.hip.h"

namespace TileXREp {
namespace {

// Element-granular reduce for any h / alignment.  One workgroup per token; a thread owns whole 32-column blocks so
// that the MXFP8 round trip needs no cross-lane traffic.
template <bool BF16>
__global__ __launch_bounds__(kThreads) void ep_reduce_generic_kernel(ReduceArgs a, int kind, int inq, int commq)
{
    __shared__ int s_row[kMaxTopK];
    __shared__ float s_w[kMaxTopK];
    const int tid = threadIdx.x;
    const int b128 = (a.h + 127) / 128;
    for (int token = blockIdx.x; token < a.bs; token += gridDim.x) {
        __syncthreads();
        LoadRoutes<true>(a, token, true, tid, kThreads, s_row, s_w, kRouteCheck);
        __syncthreads();
        if (a.tileFlags != nullptr) {
            // pairs with the producer's release.  Every wave reads rows with ordinary loads below, so every wave
            // invalidates for itself, after the barrier behind which all the token's waits have succeeded and before
            // its first row load: an invalidate issued by one wave says nothing about when a sibling's load may issue
            AcquireRowsFromAgent();
        }
        if (kind == kReducePerAdd) {
            if (tid == 0) {
                SortRows(s_row, a.slots, a.orderKeys);
            }
            __syncthreads();
        }
        const bool active = (a.tokenMask == nullptr || a.tokenMask[token] != 0) &&
            !(a.tileFlags != nullptr && AnyExpired(s_row, a.slots));
        uint16_t *dst = static_cast<uint16_t *>(a.y) + static_cast<int64_t>(token) * a.h;
        const int blocks = (a.h + 31) / 32;
        for (int b = tid; b < blocks; b += kThreads) {
            const int begin = b * 32;
            const int end = min(begin + 32, a.h);
            float acc[32];
            for (int i = 0; i < 32; ++i) {
                acc[i] = 0.0f;
            }
            if (active) {
                for (int k = 0; k < a.slots; ++k) {
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


void LaunchVecKernels(int g, int v, const ReduceLaunch &l, const ReduceArgs &a, int gridLimit)
{
    // one workgroup per token is a geometry of the units with flags only
    const bool flags = a.tileFlags != nullptr || g == kThreads;
    if (l.bf16) {
        (flags ? LaunchReduceVecBf16Flags : LaunchReduceVecBf16)(g, v, l, a, gridLimit);
    } else {
        (flags ? LaunchReduceVecFp16Flags : LaunchReduceVecFp16)(g, v, l, a, gridLimit);
    }
}

void LaunchQuantKernels(int g, int v, const ReduceLaunch &l, const ReduceArgs &a, int gridLimit)
{
    // flags that were all published before this launch began take the kernels without the waiting code
    const bool flags = a.tileFlags != nullptr;
    const bool settled = flags && a.flagsSettled != 0;
    if (l.bf16) {
        (settled ? LaunchReduceQuantBf16Settled : flags ? LaunchReduceQuantBf16Flags : LaunchReduceQuantBf16)(g, v, l, a, gridLimit);
    } else {
        (settled ? LaunchReduceQuantFp16Settled : flags ? LaunchReduceQuantFp16Flags : LaunchReduceQuantFp16)(g, v, l, a, gridLimit);
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
    a.orderKeys = l.orderKeys;
    a.expertScales = l.expertScales;
    a.tokenMask = l.tokenMask;
    a.sharedExpertX = l.sharedExpertX;
    a.inScales = l.inScales;
    a.bs = static_cast<int>(l.bs);
    a.h = static_cast<int>(l.h);
    a.topK = static_cast<int>(l.topK);
    a.slots = static_cast<int>(l.topK + l.sharedSlots);
    a.maxRows = l.maxRows > 0 ? static_cast<int>(l.maxRows) : 0x7fffffff;
    a.y = l.y;
    a.tileFlags = l.tileFlags;
    a.tileRows = static_cast<int>(l.tileRows);
    a.tileShift = -1;
    if (l.tileRows > 0 && (l.tileRows & (l.tileRows - 1)) == 0) {
        a.tileShift = __builtin_ctzll(static_cast<unsigned long long>(l.tileRows));
    }
    a.flagEpoch = l.flagEpoch;
    a.waitTimeoutTicks = l.waitTimeoutTicks;
    a.deviceStatus = l.deviceStatus;
    a.flagsSettled = (l.tileFlags != nullptr && l.producerOrdered) ? 1 : 0;
    a.claim = l.claimWord;
    a.colSlices = 1;
    // A kernel that waits on flags must never crowd out the producer it waits for: its waiting waves keep their
    // registers, and with three or more of these workgroups per compute unit a producer workgroup no longer fits
    // beside them (measured: flag waits expire at six).  Two workgroups per compute unit walk the tokens.
    // A launch whose flags were published earlier on its own stream never waits and gets the ordinary geometry.
    const bool mayWait = l.tileFlags != nullptr && !l.producerOrdered;
    const int gridLimit = mayWait ? 2 * (l.numComputeUnits > 0 ? l.numComputeUnits : 256) : 0;
    const int64_t vecs = l.h / 8;
    const bool plain = l.inQuant == 0 && l.h % 8 == 0 && Aligned16(l.y) && vecs <= 8 * kThreads &&
        Aligned16(l.expertOut) && l.rowBytes % 16 == 0 &&
        (l.sharedExpertX == nullptr || Aligned16(l.sharedExpertX)) && (l.commQuant == 0 || l.h % 32 == 0);
    const int64_t qvecs = l.h / 16;
    const bool quant = l.inQuant != 0 && l.commQuant == 0 && l.reduceKind == kReduceFp32 && l.h % 16 == 0 &&
        qvecs <= 4 * kThreads && Aligned16(l.y) && Aligned16(l.expertOut) && l.rowBytes % 16 == 0 &&
        (l.sharedExpertX == nullptr || Aligned16(l.sharedExpertX));
    if (l.kernelNameOut != nullptr) {
        *l.kernelNameOut = quant ? "ep_reduce_quant_kernel" : (plain ? "ep_reduce_vec_kernel" : "ep_reduce_generic_kernel");
    }
    if (quant) {
        if (qvecs <= kWave) {
            LaunchQuantKernels(kWave, 1, l, a, gridLimit);
        } else if (qvecs <= 2 * kWave) {
            LaunchQuantKernels(2 * kWave, 1, l, a, gridLimit);
        } else if (qvecs <= kThreads) {
            LaunchQuantKernels(kThreads, 1, l, a, gridLimit);
        } else if (qvecs <= 2 * kThreads) {
            LaunchQuantKernels(kThreads, 2, l, a, gridLimit);
        } else {
            LaunchQuantKernels(kThreads, 4, l, a, gridLimit);
        }
    } else if (plain) {
        // a wave per token for narrow rows; wide rows are cut into slices of 128 vectors, one wave each (many small
        // independent waves with four rows in flight each reach the highest gather bandwidth here)
        a.colSlices = 1;
        if (vecs <= 2 * kWave) {
            LaunchVecKernels(kWave, 2, l, a, gridLimit);
        } else if (vecs <= 4 * kWave) {
            LaunchVecKernels(kWave, 4, l, a, gridLimit);
        } else if (mayWait) {
            // readiness flags that may still be pending: one workgroup per token, so that one wave polls the token's
            // tiles instead of one per slice, and few enough workgroups that the producer fits beside them
            if (vecs <= 2 * kThreads) {
                LaunchVecKernels(kThreads, 2, l, a, gridLimit);
            } else if (vecs <= 4 * kThreads) {
                LaunchVecKernels(kThreads, 4, l, a, gridLimit);
            } else {
                LaunchVecKernels(kThreads, 8, l, a, gridLimit);
            }
        } else {
            a.colSlices = static_cast<int>((vecs + 2 * kWave - 1) / (2 * kWave));
            LaunchVecKernels(kWave, 2, l, a, gridLimit);
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

