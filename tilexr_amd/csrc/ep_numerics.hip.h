// Device-side element conversions shared by the scatter and reduce kernels (gfx950, wave64).
//
// Every routine is written so that its result is a pure function of the input bits: separate multiplies and adds
// (the build uses -ffp-contract=off and the explicit *_rn intrinsics) and saturation made explicit.  That is what
// lets the parity tests demand bit equality.  Hardware converts are used only where an exhaustive comparison on
// gfx950 showed them equal to the software codec: v_cvt_pk_bf16_f32 (all 2^32 inputs, NaNs included),
// v_cvt_pk_f32_fp8 (all codes except the sign of NaN code 0x7f) and v_cvt_pk_fp8_f32 (all finite |x| < 464; beyond
// that the hardware returns NaN where this codec saturates, so inputs are clamped first and NaNs patched).
//   int8 rounding      reference: src/ep/kernels/tilexr_ep_dispatch_kernel.cpp:183-193
//   MXFP8 / fp8 codec  reference: tests/ep/demo/mxfp8_golden.h:45-152
//   output casts       reference: src/ep/kernels/tilexr_ep_combine_memory_kernel.h:595 (CAST_RINT, saturating)
#ifndef TILEXR_AMD_EP_NUMERICS_HIP_H
#define TILEXR_AMD_EP_NUMERICS_HIP_H

#include <hip/hip_fp16.h>
#include <hip/hip_runtime.h>

namespace TileXREp {

// exponent fields of the divisors for which DivideByShared is used (see there)
constexpr uint32_t kSharedDivisionMinExponent = 16;
constexpr uint32_t kSharedDivisionMaxExponent = 254;

typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));
typedef unsigned int u32x2 __attribute__((ext_vector_type(2)));

template <bool BF16>
__device__ __forceinline__ float Decode16(uint32_t bits16)
{
    if (BF16) {
        return __uint_as_float(bits16 << 16);
    }
    return __half2float(__ushort_as_half(static_cast<unsigned short>(bits16)));
}

typedef float f32x2 __attribute__((ext_vector_type(2)));
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));

// Two fp32 -> two bf16 (round to nearest even, NaN -> (bits >> 16) | 0x40), packed lo | hi << 16.
__device__ __forceinline__ uint32_t FloatPairToBf16Rne(float lo, float hi)
{
    const f32x2 f = {lo, hi};
    return __builtin_bit_cast(uint32_t, __builtin_convertvector(f, bf16x2));
}

__device__ __forceinline__ uint32_t FloatToBf16Rne(float v)
{
    return FloatPairToBf16Rne(v, 0.0f) & 0xffffu;
}

// An fp32 value rounded to bf16 (same rounding), returned as fp32: the pair convert with 0.0 in the low half leaves the
// rounded value's own fp32 bit pattern, so one instruction does the rounding and no unpacking follows.
__device__ __forceinline__ float FloatRoundedToBf16(float v)
{
    return __uint_as_float(FloatPairToBf16Rne(0.0f, v));
}

// IEEE round-to-nearest-even; overflow becomes infinity.
__device__ __forceinline__ uint32_t FloatToHalfRne(float v)
{
    return __half_as_ushort(__float2half_rn(v));
}

// Same rounding, but magnitudes that would round past 65504 stay at +-65504.
__device__ __forceinline__ uint32_t FloatToHalfRneSat(float v)
{
    const uint32_t u = __float_as_uint(v);
    const uint32_t a = u & 0x7fffffffu;
    if (a >= 0x477ff000u && a <= 0x7f800000u) {
        return ((u >> 16) & 0x8000u) | 0x7bffu;
    }
    return FloatToHalfRne(v);
}

template <bool BF16>
__device__ __forceinline__ uint32_t Encode16Sat(float v)
{
    return BF16 ? FloatToBf16Rne(v) : FloatToHalfRneSat(v);
}

// Two values -> packed 16-bit elements (lo | hi << 16), fp16 saturating as above.
template <bool BF16>
__device__ __forceinline__ uint32_t EncodePair16Sat(float lo, float hi)
{
    return BF16 ? FloatPairToBf16Rne(lo, hi) : (FloatToHalfRneSat(lo) | (FloatToHalfRneSat(hi) << 16));
}

// Round an fp32 value to the 16-bit element type and return it as fp32 again (IEEE, non-saturating).
template <bool BF16>
__device__ __forceinline__ float RoundTo16(float v)
{
    return BF16 ? __uint_as_float(FloatToBf16Rne(v) << 16) : __half2float(__float2half_rn(v));
}

// add +-0.5, truncate toward zero, clamp to [-128, 127]
__device__ __forceinline__ int ClampInt8(float v)
{
    float r = v >= 0.0f ? __fadd_rn(v, 0.5f) : __fadd_rn(v, -0.5f);
    r = fminf(fmaxf(r, -129.0f), 128.0f);
    int i = static_cast<int>(r);
    i = i > 127 ? 127 : i;
    i = i < -128 ? -128 : i;
    return i;
}

// Saturating round-to-nearest-even fp32 -> fp8 code (OCP e4m3fn / e5m2), by bit manipulation.
template <bool E5M2>
__device__ __forceinline__ uint32_t Fp8Encode(float v)
{
    constexpr int kMantBits = E5M2 ? 2 : 3;
    constexpr int kBias = E5M2 ? 15 : 7;
    constexpr int kMinNormalExp = 1 - kBias;
    constexpr uint32_t kMaxCode = E5M2 ? 0x7bu : 0x7eu;
    const uint32_t u = __float_as_uint(v);
    const uint32_t sign = (u >> 24) & 0x80u;
    const uint32_t a = u & 0x7fffffffu;
    if (a > 0x7f800000u) {
        return sign | 0x7fu;
    }
    const int e = static_cast<int>(a >> 23) - 127;
    const uint32_t mant = a & 0x7fffffu;
    uint32_t code;
    if (e < kMinNormalExp) {
        const int shift = 23 - e + kMinNormalExp - kMantBits;   // value / subnormal step = full >> shift
        if (shift > 24) {
            code = 0;
        } else {
            const uint32_t full = mant | 0x800000u;
            const uint32_t kept = full >> shift;
            const uint32_t rem = full & ((1u << shift) - 1u);
            const uint32_t half = 1u << (shift - 1);
            code = kept + ((rem > half || (rem == half && (kept & 1u))) ? 1u : 0u);
        }
    } else if (e > 20) {
        code = kMaxCode;
    } else {
        const uint32_t kept = mant >> (23 - kMantBits);
        const uint32_t rem = mant & ((1u << (23 - kMantBits)) - 1u);
        const uint32_t half = 1u << (22 - kMantBits);
        code = (static_cast<uint32_t>(e + kBias) << kMantBits) + kept +
            ((rem > half || (rem == half && (kept & 1u))) ? 1u : 0u);
        code = code > kMaxCode ? kMaxCode : code;
    }
    return sign | code;
}

template <bool E5M2>
__device__ __forceinline__ float Fp8Decode(uint32_t code)
{
    constexpr int kMantBits = E5M2 ? 2 : 3;
    constexpr int kBias = E5M2 ? 15 : 7;
    constexpr uint32_t kExpMask = E5M2 ? 31u : 15u;
    constexpr uint32_t kMantMask = (1u << kMantBits) - 1u;
    const uint32_t sign = (code & 0x80u) << 24;
    const uint32_t exp = (code >> kMantBits) & kExpMask;
    const uint32_t man = code & kMantMask;
    if (exp == 0) {
        const float mag = static_cast<float>(man) * __uint_as_float(static_cast<uint32_t>(127 + 1 - kBias - kMantBits) << 23);
        return __uint_as_float(__float_as_uint(mag) | sign);
    }
    if (E5M2 && exp == kExpMask) {
        return __uint_as_float(sign | 0x7f800000u | (man << 21));
    }
    if (!E5M2 && exp == kExpMask && man == kMantMask) {
        return __uint_as_float(sign | 0x7fc00000u);
    }
    return __uint_as_float(sign | ((exp + 127u - kBias) << 23) | (man << (23 - kMantBits)));
}

// e4m3 code of x with round-to-nearest-even and saturation to +-448; NaN -> sign | 0x7f.  Same function as
// Fp8Encode<false>, through the hardware convert.
__device__ __forceinline__ uint32_t Fp8E4m3EncodePairSat(float lo, float hi)
{
    const float clo = __builtin_amdgcn_fmed3f(lo, -448.0f, 448.0f);
    const float chi = __builtin_amdgcn_fmed3f(hi, -448.0f, 448.0f);
    uint32_t code = static_cast<uint32_t>(__builtin_amdgcn_cvt_pk_fp8_f32(clo, chi, 0, false)) & 0xffffu;
    if (lo != lo) {
        code = (code & 0xff00u) | ((__float_as_uint(lo) >> 24) & 0x80u) | 0x7fu;
    }
    if (hi != hi) {
        code = (code & 0x00ffu) | ((((__float_as_uint(hi) >> 24) & 0x80u) | 0x7fu) << 8);
    }
    return code;
}

// Four values that are not NaNs -> four e4m3 codes in one word (a | b << 8 | c << 16 | d << 24), same codes as
// Fp8E4m3EncodePairSat: the second convert writes the upper half of the word the first one started.
__device__ __forceinline__ uint32_t Fp8E4m3EncodeFourSat(float a, float b, float c, float d)
{
    const int lower = __builtin_amdgcn_cvt_pk_fp8_f32(__builtin_amdgcn_fmed3f(a, -448.0f, 448.0f),
        __builtin_amdgcn_fmed3f(b, -448.0f, 448.0f), 0, false);
    return static_cast<uint32_t>(__builtin_amdgcn_cvt_pk_fp8_f32(__builtin_amdgcn_fmed3f(c, -448.0f, 448.0f),
        __builtin_amdgcn_fmed3f(d, -448.0f, 448.0f), lower, true));
}

// x / b for many x and one b > 0, for a caller that encodes the quotient as e4m3: the code is the one the correctly
// rounded quotient __fdiv_rn(x, b) gives, on every pair a block quantiser can meet.
// The correctly rounded quotient costs about eleven instructions per element when the compiler expands the division
// (range scaling, reciprocal, two refinements of the reciprocal, quotient, two remainders, fix-up).  Everything that
// depends on b alone is done once here (SharedReciprocal): the reciprocal refined to within a rounding of 1 / b.  An
// element then takes a product, an exact remainder and one correction, plus the sign (b > 0, so the quotient has the
// sign of x; a zero remainder would otherwise turn -0 into +0).  The long form corrects the quotient twice and scales
// the operands' ranges; without that the quotient can be off in its last place (about one pair in five hundred) or,
// for very small divisors, by more.  An exhaustive run over all pairs of 16-bit element patterns and block maxima, bf16
// and fp16 (tests/cxx/shared_division_check.hip), found no pair whose e4m3 code differs for divisors with the exponent
// fields that SharedReciprocalHolds accepts; other divisors (block maxima below 2^-102, or infinite) take the long form.
__device__ __forceinline__ bool SharedReciprocalHolds(float b)
{
    const uint32_t exponent = (__float_as_uint(b) >> 23) & 0xffu;
    return exponent >= kSharedDivisionMinExponent && exponent <= kSharedDivisionMaxExponent;
}

__device__ __forceinline__ float SharedReciprocal(float b)
{
    const float y0 = __builtin_amdgcn_rcpf(b);
    const float e = __builtin_fmaf(-b, y0, 1.0f);
    return __builtin_fmaf(e, y0, y0);
}

__device__ __forceinline__ float DivideByShared(float x, float b, float y)
{
    const float q0 = __fmul_rn(x, y);
    const float r = __builtin_fmaf(-b, q0, x);
    return __builtin_copysignf(__builtin_fmaf(r, y, q0), x);
}

// True when one of the four e4m3 codes in `word` is a NaN code (0x7f / 0xff).
__device__ __forceinline__ bool Fp8E4m3WordHasNan(uint32_t word)
{
    return (((word & 0x7f7f7f7fu) + 0x01010101u) & 0x80808080u) != 0u;
}

// Four e4m3 codes -> four fp32 through the hardware convert alone: the values of Fp8Decode<false> for every code but
// the NaN code 0x7f, whose NaN comes back with the other sign.  For callers that notice a NaN in their result and then
// redo the work with Fp8E4m3DecodeWord.
__device__ __forceinline__ void Fp8E4m3DecodeWordFast(uint32_t word, float *out)
{
    const f32x2 lo = __builtin_amdgcn_cvt_pk_f32_fp8(static_cast<int>(word), false);
    const f32x2 hi = __builtin_amdgcn_cvt_pk_f32_fp8(static_cast<int>(word), true);
    out[0] = lo[0];
    out[1] = lo[1];
    out[2] = hi[0];
    out[3] = hi[1];
}

// Four e4m3 codes -> four fp32, same values as Fp8Decode<false> (NaN codes take the software path).
__device__ __forceinline__ void Fp8E4m3DecodeWord(uint32_t word, float *out)
{
    if (Fp8E4m3WordHasNan(word)) {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            out[i] = Fp8Decode<false>((word >> (8 * i)) & 0xffu);
        }
        return;
    }
    const f32x2 lo = __builtin_amdgcn_cvt_pk_f32_fp8(static_cast<int>(word), false);
    const f32x2 hi = __builtin_amdgcn_cvt_pk_f32_fp8(static_cast<int>(word), true);
    out[0] = lo[0];
    out[1] = lo[1];
    out[2] = hi[0];
    out[3] = hi[1];
}

// Shared exponent of an MXFP8 block: clamp(floor(log2 amax) - emax, -127, 127); all-zero block -> -127.
template <bool E5M2>
__device__ __forceinline__ int MxSharedExponent(float amax)
{
    constexpr int kEmax = E5M2 ? 15 : 8;
    const uint32_t a = __float_as_uint(amax) & 0x7fffffffu;
    if (a == 0) {
        return -127;
    }
    int se = static_cast<int>(a >> 23) - 127 - kEmax;    // denormal amax gives < -127 and is clamped below
    se = se < -127 ? -127 : se;
    se = se > 127 ? 127 : se;
    return se;
}

// 2^e for e in [-127, 127] (2^-127 is a denormal fp32 and is produced exactly)
__device__ __forceinline__ float Exp2Int(int e)
{
    return e >= -126 ? __uint_as_float(static_cast<uint32_t>(e + 127) << 23) : __uint_as_float(0x00400000u);
}

} // namespace TileXREp

#endif // TILEXR_AMD_EP_NUMERICS_HIP_H
