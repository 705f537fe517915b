/*
 * CPU oracle (test infrastructure only; see tilexr_ep_oracle.h).
 * Build: gcc -O2 -ffp-contract=off -fPIC -shared (see Makefile).  -ffp-contract=off matters: the
 * reference rounds after every multiply and every add.
 */
#include "tilexr_ep_oracle.h"

#include <math.h>
#include <stdlib.h>
#include <string.h>

/* ------------------------------------------------------------------------------------------------
 * Scalar numerics
 * ---------------------------------------------------------------------------------------------- */

static inline uint32_t f2u(float v) { uint32_t u; memcpy(&u, &v, 4); return u; }
static inline float u2f(uint32_t u) { float v; memcpy(&v, &u, 4); return v; }

/* fp16 bits -> float.  src/ep/kernels/tilexr_ep_dispatch_kernel.cpp:152-181 builds the value from
 * sign, exponent and mantissa by repeated *2 / *0.5; every step is exact, so the result equals the
 * IEEE value for zeros, subnormals and normals.  Exponent 31 (inf/nan) is not special-cased there
 * (it yields 1.m * 2^16); inputs with exponent 31 are outside the contract and follow IEEE here. */
float orc_half_to_float(uint16_t bits)
{
    const uint32_t sign = (uint32_t)(bits & 0x8000u) << 16;
    const uint32_t exponent = (bits >> 10) & 0x1fu;
    const uint32_t mantissa = bits & 0x3ffu;
    if (exponent == 0) {
        if (mantissa == 0) {
            return u2f(sign);
        }
        const float mag = ldexpf((float)mantissa, -24);
        return sign ? -mag : mag;
    }
    if (exponent == 31) {
        return u2f(sign | 0x7f800000u | (mantissa << 13));
    }
    return u2f(sign | ((exponent + 112u) << 23) | (mantissa << 13));
}

/* tests/ep/demo/tilexr_ep_dispatch_demo.cpp:490-499: bf16 is the top half of an fp32. */
float orc_bf16_to_float(uint16_t bits)
{
    return u2f((uint32_t)bits << 16);
}

static inline float decode_elem(uint16_t bits, int32_t dtype)
{
    return dtype == ORC_DT_BF16 ? orc_bf16_to_float(bits) : orc_half_to_float(bits);
}

/* fp32 -> bf16, round to nearest even (CAST_RINT, tilexr_ep_combine_memory_kernel.h:595). */
uint16_t orc_float_to_bf16_rne(float v)
{
    uint32_t u = f2u(v);
    if ((u & 0x7fffffffu) > 0x7f800000u) {
        return (uint16_t)((u >> 16) | 0x0040u);
    }
    const uint32_t lsb = (u >> 16) & 1u;
    u += 0x7fffu + lsb;
    return (uint16_t)(u >> 16);
}

static uint16_t float_to_half_impl(float v, int saturate)
{
    const uint32_t u = f2u(v);
    const uint16_t sign = (uint16_t)((u >> 16) & 0x8000u);
    const uint32_t a = u & 0x7fffffffu;
    if (a > 0x7f800000u) {
        return (uint16_t)(sign | 0x7e00u);
    }
    if (a >= 0x477ff000u) { /* >= 65520: rounds past the largest finite half */
        if (a == 0x7f800000u && !saturate) {
            return (uint16_t)(sign | 0x7c00u);
        }
        return (uint16_t)(sign | (saturate ? 0x7bffu : 0x7c00u));
    }
    if (a < 0x33000001u) { /* <= 2^-25: rounds to zero (tie at 2^-25 goes to even = 0) */
        return sign;
    }
    const int32_t e = (int32_t)(a >> 23) - 127;
    uint32_t mant = (a & 0x7fffffu) | 0x800000u;
    uint32_t shift;
    uint32_t base;
    if (e < -14) {
        shift = (uint32_t)(13 + (-14 - e));
        base = 0;
    } else {
        shift = 13;
        base = (uint32_t)(e + 15) << 10;
        mant &= 0x7fffffu;
    }
    const uint32_t kept = mant >> shift;
    const uint32_t rem = mant & ((1u << shift) - 1u);
    const uint32_t half = 1u << (shift - 1u);
    uint32_t out = base + kept;
    if (rem > half || (rem == half && (kept & 1u))) {
        ++out;
    }
    return (uint16_t)(sign | out);
}

/* The memory-route kernels clear the float-overflow control register
 * (tilexr_ep_combine_memory_kernel.h:179-181), i.e. saturating casts; the demo clamps its fp16
 * expectation to +-65504 (tests/ep/demo/tilexr_ep_dispatch_demo.cpp:1035-1038). */
uint16_t orc_float_to_half_rne_sat(float v) { return float_to_half_impl(v, 1); }
uint16_t orc_float_to_half_rne(float v) { return float_to_half_impl(v, 0); }

/* src/ep/kernels/tilexr_ep_dispatch_kernel.cpp:183-193: add +-0.5, truncate, clamp to [-128,127]. */
int8_t orc_clamp_int8(float v)
{
    const float rounded = v >= 0.0f ? v + 0.5f : v - 0.5f;
    int32_t as_int;
    if (rounded >= 2147483520.0f) {
        as_int = 2147483647;
    } else if (rounded <= -2147483648.0f) {
        as_int = (-2147483647 - 1);
    } else {
        as_int = (int32_t)rounded;
    }
    if (as_int > 127) {
        as_int = 127;
    } else if (as_int < -128) {
        as_int = -128;
    }
    return (int8_t)as_int;
}

static float round_nearest_even(float v)
{
    /* tests/ep/demo/mxfp8_golden.h:32-43 */
    const float lower = floorf(v);
    const float frac = v - lower;
    if (frac < 0.5f) {
        return lower;
    }
    if (frac > 0.5f) {
        return lower + 1.0f;
    }
    return fmodf(lower, 2.0f) == 0.0f ? lower : lower + 1.0f;
}

static void fp8_params(int32_t fp8_dtype, int *ebits, int *mbits, int *bias, float *max_finite)
{
    if (fp8_dtype == ORC_DT_FP8E5M2) {
        *ebits = 5; *mbits = 2; *bias = 15; *max_finite = 57344.0f;
    } else {
        *ebits = 4; *mbits = 3; *bias = 7; *max_finite = 448.0f;
    }
}

/* Saturating round-to-nearest-even fp32 -> fp8 (OCP e4m3fn / e5m2).
 * tests/ep/demo/mxfp8_golden.h:45-86 (EncodeFp8) after the pre-rounding of :141-150. */
uint8_t orc_fp8_encode(float value, int32_t fp8_dtype)
{
    int ebits, mbits, bias;
    float max_finite;
    fp8_params(fp8_dtype, &ebits, &mbits, &bias, &max_finite);
    const uint8_t sign = signbit(value) ? 0x80u : 0u;
    float mag = fabsf(value);
    if (!(mag == mag)) {
        return (uint8_t)(sign | 0x7fu);
    }
    if (mag == 0.0f) {
        return sign;
    }
    const int min_normal_exp = 1 - bias;
    int enc_exp = 0;
    int enc_man = 0;
    if (mag < ldexpf(1.0f, min_normal_exp)) {
        const float step = ldexpf(1.0f, min_normal_exp - mbits);
        enc_man = (int)round_nearest_even(mag / step);
        if (enc_man >= (1 << mbits)) {
            enc_exp = 1;
            enc_man = 0;
        }
    } else {
        int exponent;
        if (mag >= max_finite) {
            mag = max_finite;
        }
        exponent = ilogbf(mag);
        const float normalized = ldexpf(mag, -exponent);
        enc_man = (int)round_nearest_even((normalized - 1.0f) * (float)(1 << mbits));
        if (enc_man == (1 << mbits)) {
            ++exponent;
            enc_man = 0;
        }
        enc_exp = exponent + bias;
        /* saturate anything that rounded past the largest finite code */
        const int max_code = fp8_dtype == ORC_DT_FP8E5M2 ? 0x7b : 0x7e;
        const int code = (enc_exp << mbits) | enc_man;
        if (code > max_code) {
            return (uint8_t)(sign | max_code);
        }
    }
    return (uint8_t)(sign | (uint8_t)(enc_exp << mbits) | (uint8_t)enc_man);
}

/* tests/ep/demo/mxfp8_golden.h:88-114 */
float orc_fp8_decode(uint8_t value, int32_t fp8_dtype)
{
    int ebits, mbits, bias;
    float max_finite;
    fp8_params(fp8_dtype, &ebits, &mbits, &bias, &max_finite);
    const int emask = (1 << ebits) - 1;
    const int mmask = (1 << mbits) - 1;
    const int exponent = (value >> mbits) & emask;
    const int mantissa = value & mmask;
    const float sign = (value & 0x80u) ? -1.0f : 1.0f;
    if (exponent == 0) {
        if (mantissa == 0) {
            return copysignf(0.0f, sign);
        }
        return sign * ldexpf((float)mantissa, 1 - bias - mbits);
    }
    if (fp8_dtype == ORC_DT_FP8E5M2 && exponent == emask) {
        return mantissa == 0 ? sign * INFINITY : NAN;
    }
    if (fp8_dtype != ORC_DT_FP8E5M2 && exponent == emask && mantissa == mmask) {
        return NAN;
    }
    return sign * ldexpf(1.0f + (float)mantissa / (float)(1 << mbits), exponent - bias);
}

/* tests/ep/demo/mxfp8_golden.h:26-30; src/ep/host/ep_memory_layout.cpp:126-129 */
int64_t orc_mxfp8_scale_count(int64_t h)
{
    const int64_t blocks = (h + 31) / 32;
    return blocks + (blocks & 1);
}

/* ------------------------------------------------------------------------------------------------
 * Row quantisers
 * ---------------------------------------------------------------------------------------------- */

/* src/ep/kernels/tilexr_ep_dispatch_helpers.h:153-191: absmax -> dequantScale = max/127 (1.0 when the row
 * is all zero), quantScale = 1/dequantScale, q = clamp(trunc(v*quantScale +- 0.5)).
 * The reference decodes the input as fp16; decode_dtype == ORC_DT_BF16 is the ext variant. */
float orc_quant_row_token_int8(const uint16_t *src, int64_t h, int32_t decode_dtype, int8_t *dst)
{
    float max_abs = 0.0f;
    for (int64_t i = 0; i < h; ++i) {
        const float a = fabsf(decode_elem(src[i], decode_dtype));
        if (a > max_abs) {
            max_abs = a;
        }
    }
    const float dequant = max_abs > 0.0f ? max_abs / 127.0f : 1.0f;
    const float quant = dequant > 0.0f ? 1.0f / dequant : 1.0f;
    for (int64_t i = 0; i < h; ++i) {
        dst[i] = orc_clamp_int8(decode_elem(src[i], decode_dtype) * quant);
    }
    return dequant;
}

/* src/ep/kernels/tilexr_ep_dispatch_helpers.h:114-136 (input decoded as fp16, scale = scales[0]). */
void orc_quant_row_static_int8(const uint16_t *src, int64_t h, float scale, int8_t *dst)
{
    for (int64_t i = 0; i < h; ++i) {
        dst[i] = orc_clamp_int8(orc_half_to_float(src[i]) * scale);
    }
}

/* tests/ep/demo/mxfp8_golden.h:116-152 (QuantizeMxfp8Row): 32-element blocks, E8M0 shared exponent
 * = clamp(floor(log2 amax) - emax, -127, 127) + 127 (0 for an all-zero block), elements
 * RNE-saturated after dividing by 2^shared.  Scale bytes beyond the last block are zero. */
void orc_quant_row_mxfp8(const uint16_t *src, int64_t h, int32_t dtype, int32_t fp8_dtype,
    uint8_t *dst, uint8_t *scales)
{
    const int64_t scale_count = orc_mxfp8_scale_count(h);
    const int emax = fp8_dtype == ORC_DT_FP8E5M2 ? 15 : 8;
    memset(scales, 0, (size_t)scale_count);
    const int64_t blocks = (h + 31) / 32;
    for (int64_t b = 0; b < blocks; ++b) {
        const int64_t begin = b * 32;
        const int64_t end = begin + 32 < h ? begin + 32 : h;
        float max_abs = 0.0f;
        for (int64_t i = begin; i < end; ++i) {
            const float a = fabsf(decode_elem(src[i], dtype));
            if (a > max_abs) {
                max_abs = a;
            }
        }
        int shared = max_abs == 0.0f ? -127 : ilogbf(max_abs) - emax;
        if (shared < -127) {
            shared = -127;
        }
        if (shared > 127) {
            shared = 127;
        }
        scales[b] = (uint8_t)(shared + 127);
        for (int64_t i = begin; i < end; ++i) {
            dst[i] = orc_fp8_encode(ldexpf(decode_elem(src[i], dtype), -shared), fp8_dtype);
        }
    }
}

/* ext (no reference counterpart): e4m3 with one fp32 scale per 128 columns,
 * scale = amax/448 (1.0 for an all-zero block), q = rne_sat(v / scale). */
void orc_quant_row_fp8_block128(const uint16_t *src, int64_t h, int32_t dtype, uint8_t *dst, float *scales)
{
    const int64_t blocks = (h + 127) / 128;
    for (int64_t b = 0; b < blocks; ++b) {
        const int64_t begin = b * 128;
        const int64_t end = begin + 128 < h ? begin + 128 : h;
        float max_abs = 0.0f;
        for (int64_t i = begin; i < end; ++i) {
            const float a = fabsf(decode_elem(src[i], dtype));
            if (a > max_abs) {
                max_abs = a;
            }
        }
        const float scale = max_abs > 0.0f ? max_abs / 448.0f : 1.0f;
        scales[b] = scale;
        for (int64_t i = begin; i < end; ++i) {
            dst[i] = orc_fp8_encode(decode_elem(src[i], dtype) / scale, ORC_DT_FP8E4M3);
        }
    }
}

/* ------------------------------------------------------------------------------------------------
 * Dispatch
 * ---------------------------------------------------------------------------------------------- */

static int64_t tp_size(const orc_case *c)
{
    return c->tp_world_size > 1 ? c->tp_world_size : 1;
}

/* src/ep/host/ep_layout.cpp:156,171; tests/ep/demo/tilexr_ep_dispatch_demo.cpp:622-630 */
static int64_t local_expert_num(const orc_case *c)
{
    return c->moe_expert_num / (c->rank_size / tp_size(c) - c->shared_expert_rank_num);
}

/* tests/ep/demo/tilexr_ep_dispatch_demo.cpp:632-635: a shared rank presents one local expert */
static int64_t out_local_expert_num(const orc_case *c, int32_t rank)
{
    return rank < c->shared_expert_rank_num ? 1 : local_expert_num(c);
}

/* Destination rank of a shared route (demo :654-657; src/ep/kernels/tilexr_ep_dispatch_memory_kernel.h:635-643;
 * MVP route, where SR == S: tilexr_ep_dispatch_helpers.h:85-87). */
static int64_t shared_dst_rank(const orc_case *c, int32_t src, int64_t s)
{
    const int64_t per = c->shared_expert_rank_num / c->shared_expert_num;
    return src % per + s * per;
}

static int64_t out_row_bytes(const orc_case *c)
{
    return c->quant_mode == ORC_QUANT_NONE ? c->h * 2 : c->h;
}

/* MVP ("UDMA") route.
 *   routing walk   src/ep/kernels/tilexr_ep_dispatch_kernel.cpp:501-571 (token-major, k-minor; token mask
 *                  tested per token; ids outside [0, E) skipped)
 *   drain          src/ep/kernels/tilexr_ep_combine_helpers.h:81-145 (source ranks in order; recvCounts[src];
 *                  expertTokenNums incremented per drained row; optional prefix-sum finalize :67-80)
 *   checker model  tools/checker/src/oracle.cpp:447-484 (same order, unmasked)
 * Quantised payloads always decode the input as fp16 (tilexr_ep_dispatch_helpers.h:121,167). */
/* Appends the rows source rank `src` sends to expert rank `er` (token-major, shared routes then routed ones) and
 * returns how many there were. */
static int32_t mvp_rows_from_source(const orc_case *c, int32_t src, int64_t er, const uint16_t *x, const int32_t *ids,
    const uint8_t *mask, const float *static_scale, uint8_t *expand_x, float *dyn_scales, int32_t *assist,
    int64_t *expert_token_nums, int64_t *out_io)
{
    const int64_t local_e = local_expert_num(c);
    const int64_t row_bytes = out_row_bytes(c);
    const uint16_t *xs = x + (int64_t)src * c->bs * c->h;
    const int32_t *is = ids + (int64_t)src * c->bs * c->top_k;
    const uint8_t *ms = mask ? mask + (int64_t)src * c->bs : NULL;
    /* with tensor-parallel groups the placement rules run over expert ranks and the source is known by its
     * expert rank there (tilexr_ep_dispatch_kernel.cpp:724, 774-776) */
    const int32_t src_expert_rank = src / (int32_t)tp_size(c);
    int64_t out = *out_io;
    int32_t count = 0;
    for (int64_t t = 0; t < c->bs; ++t) {
        if (ms && ms[t] == 0) {
            continue;
        }
        /* one pass over the token's S shared routes, then its top_k routed ones
         * (src/ep/kernels/tilexr_ep_dispatch_kernel.cpp:536-568) */
        for (int64_t r = 0; r < c->shared_expert_num + c->top_k; ++r) {
            const int shared = r < c->shared_expert_num;
            const int64_t k = shared ? c->top_k + r : r - c->shared_expert_num;
            int32_t e;
            int64_t local;
            if (shared) {
                if (shared_dst_rank(c, src_expert_rank, r) != er) {
                    continue;
                }
                e = (int32_t)r;
                /* tilexr_ep_dispatch_helpers.h:99-101: a shared row counts at index expertId */
                local = r;
            } else {
                const int32_t id = is[t * c->top_k + k];
                if (id < 0 || (int64_t)id >= c->moe_expert_num) {
                    continue;
                }
                if (c->shared_expert_rank_num + (int64_t)id / local_e != er) {
                    continue;
                }
                e = (int32_t)(c->shared_expert_num + id);
                local = (int64_t)id % local_e;
            }
            uint8_t *dst = expand_x + out * row_bytes;
            const uint16_t *row = xs + t * c->h;
            if (c->quant_mode == ORC_QUANT_STATIC_INT8) {
                orc_quant_row_static_int8(row, c->h, static_scale[0], (int8_t *)dst);
            } else if (c->quant_mode == ORC_QUANT_TOKEN_INT8) {
                dyn_scales[out] = orc_quant_row_token_int8(row, c->h, ORC_DT_FP16, (int8_t *)dst);
            } else {
                memcpy(dst, row, (size_t)row_bytes);
            }
            assist[out * 4 + 0] = src;
            assist[out * 4 + 1] = (int32_t)t;
            assist[out * 4 + 2] = (int32_t)k;
            assist[out * 4 + 3] = e;
            if (local < local_e) {          /* tilexr_ep_combine_helpers.h:124-128 */
                ++expert_token_nums[local];
            }
            ++count;
            ++out;
        }
    }
    *out_io = out;
    return count;
}

int64_t orc_mvp_dispatch_rank(const orc_case *c, int32_t dst_rank, const uint16_t *x, const int32_t *ids,
    const uint8_t *mask, const float *static_scale, uint8_t *expand_x, float *dyn_scales, int32_t *assist,
    int32_t *recv_counts, int32_t *tp_recv_counts, int64_t *expert_token_nums)
{
    const int64_t local_e = local_expert_num(c);
    const int64_t tp = tp_size(c);
    const int64_t expert_ranks = c->rank_size / tp;
    const int64_t er = dst_rank / tp;
    const int64_t lane = dst_rank % tp;
    int64_t out = 0;
    for (int64_t e = 0; e < local_e; ++e) {
        expert_token_nums[e] = 0;
    }
    /* own lane: the sources of this rank's lane in expert-rank order (tilexr_ep_dispatch_kernel.cpp:809-817);
     * both count arrays are indexed by the source's global rank here (tilexr_ep_combine_helpers.h:92-95) */
    for (int64_t es = 0; es < expert_ranks; ++es) {
        const int32_t src = (int32_t)(es * tp + lane);
        const int32_t count = mvp_rows_from_source(c, src, er, x, ids, mask, static_scale, expand_x, dyn_scales,
            assist, expert_token_nums, &out);
        recv_counts[src] = count;
        if (tp_recv_counts) {
            tp_recv_counts[src] = count;
        }
    }
    /* tensor-parallel publish: the rows the other lanes of the group received follow in lane order, and the
     * first tp entries of tpRecvCounts become rows per lane (:818-827, 662-697) */
    if (tp > 1 && tp_recv_counts) {
        tp_recv_counts[lane] = (int32_t)out;
        for (int64_t l = 0; l < tp; ++l) {
            if (l == lane) {
                continue;
            }
            int32_t lane_rows = 0;
            for (int64_t es = 0; es < expert_ranks; ++es) {
                lane_rows += mvp_rows_from_source(c, (int32_t)(es * tp + l), er, x, ids, mask, static_scale, expand_x,
                    dyn_scales, assist, expert_token_nums, &out);
            }
            tp_recv_counts[l] = lane_rows;
        }
    }
    if (c->token_nums_type == 0) {
        int64_t running = 0;
        for (int64_t e = 0; e < local_e; ++e) {
            running += expert_token_nums[e];
            expert_token_nums[e] = running;
        }
    }
    return out;
}

/* Number of leading flat routes a source rank considers, and whether route i is live.
 *   token mask   src/ep/kernels/tilexr_ep_dispatch_memory_kernel.h:1387-1410,1538-1544: activeCnt = sum(mask),
 *                the FIRST activeCnt*K ids are used (prefix semantics, not a per-token test)
 *   expert mask  :1483-1535: routes whose mask byte is not set become id -1 */
static int64_t mem_route_limit(const orc_case *c, const uint8_t *ms)
{
    if (c->mask_type == ORC_MASK_TOKEN && ms) {
        int64_t active = 0;
        for (int64_t t = 0; t < c->bs; ++t) {
            active += ms[t] != 0;
        }
        return active * c->top_k;
    }
    return c->bs * c->top_k;
}

/* Memory route.
 *   order        local expert -> source rank -> flat route index
 *                (tilexr_ep_dispatch_memory_kernel.h:665-708 slot = rank-within-expert from :791-818;
 *                 :1261-1317 dstPosition = sendCnt[idx-1] + done with idx = localExpert*R + srcRank;
 *                 tests/ep/demo/tilexr_ep_dispatch_demo.cpp:745-763)
 *   sendCounts   inclusive cumsum over idx (:1059-1074; demo :765-792)
 *   tokenNums    :1159-1168 (type 0 = sendCnt[le*R+R-1], type 1 = difference)
 *   assist       {srcRank, token, k, global expert id} (:1240-1258)
 *   ext          capacity: a source rank sends at most `capacity` rows per expert, lowest flat route
 *                indices first; quant_mode TOKEN_INT8 (decode by dtype) and FP8_BLOCK128. */
int64_t orc_mem_dispatch_rank(const orc_case *c, int32_t dst_rank, const uint16_t *x, const int32_t *ids,
    const uint8_t *mask, uint8_t *expand_x, uint8_t *dyn_scales, int32_t *assist, int32_t *send_counts,
    int64_t *expert_token_nums)
{
    const int64_t local_e = local_expert_num(c);
    const int64_t row_bytes = out_row_bytes(c);
    const int64_t routes = c->bs * c->top_k;
    const int64_t mask_stride = c->mask_type == ORC_MASK_EXPERT ? routes : c->bs;
    const int64_t mx_scales = orc_mxfp8_scale_count(c->h);
    const int64_t b128 = (c->h + 127) / 128;
    const int64_t out_local = out_local_expert_num(c, dst_rank);
    const int is_shared_rank = dst_rank < c->shared_expert_rank_num;
    int64_t out = 0;
    for (int64_t le = 0; le < out_local; ++le) {
        /* id (as the caller numbers routed experts) whose rows this segment collects; on a shared rank the
         * segment collects the shared routes aimed at it instead (tilexr_ep_dispatch_memory_kernel.h:622-663) */
        const int64_t expert = ((int64_t)dst_rank - c->shared_expert_rank_num) * local_e + le;
        for (int32_t src = 0; src < c->rank_size; ++src) {
            const uint16_t *xs = x + (int64_t)src * c->bs * c->h;
            const int32_t *is = ids + (int64_t)src * routes;
            const uint8_t *ms = (mask && c->mask_type != ORC_MASK_NONE) ? mask + (int64_t)src * mask_stride : NULL;
            const int64_t limit = mem_route_limit(c, ms);
            int64_t kept = 0;
            /* shared rank: walk (shared expert, token) pairs; otherwise the flat routes */
            const int64_t walk = is_shared_rank ? c->shared_expert_num * (limit / c->top_k) : limit;
            for (int64_t i = 0; i < walk; ++i) {
                int64_t t;
                int64_t k;
                int32_t tuple_expert;
                if (is_shared_rank) {
                    const int64_t tokens = limit / c->top_k;
                    const int64_t s = i / tokens;
                    if (shared_dst_rank(c, src, s) != dst_rank) {
                        continue;
                    }
                    t = i % tokens;
                    if (c->mask_type == ORC_MASK_EXPERT && ms) {
                        /* the shared routes go out for the tokens that keep at least one routed expert
                         * (tilexr_ep_dispatch_memory_kernel.h:1412-1441, 641-647; demo :613-620) */
                        int any = 0;
                        for (int64_t kk = 0; kk < c->top_k; ++kk) {
                            any |= ms[t * c->top_k + kk] != 0;
                        }
                        if (!any) {
                            continue;
                        }
                    }
                    k = c->top_k + s;
                    tuple_expert = (int32_t)s;      /* :1257 topKId - K on a shared rank */
                } else {
                    if (c->mask_type == ORC_MASK_EXPERT && ms && ms[i] == 0) {
                        continue;
                    }
                    if ((int64_t)is[i] != expert) {
                        continue;
                    }
                    if (c->capacity > 0 && kept >= c->capacity) {
                        continue;
                    }
                    t = i / c->top_k;
                    k = i % c->top_k;
                    tuple_expert = (int32_t)(c->shared_expert_num + expert);    /* :1241-1244 */
                }
                ++kept;
                uint8_t *dst = expand_x + out * row_bytes;
                const uint16_t *row = xs + t * c->h;
                switch (c->quant_mode) {
                    case ORC_QUANT_MXFP8:
                        orc_quant_row_mxfp8(row, c->h, c->dtype, c->out_dtype, dst, dyn_scales + out * mx_scales);
                        break;
                    case ORC_QUANT_TOKEN_INT8:
                        ((float *)dyn_scales)[out] = orc_quant_row_token_int8(row, c->h, c->dtype, (int8_t *)dst);
                        break;
                    case ORC_QUANT_FP8_BLOCK128:
                        orc_quant_row_fp8_block128(row, c->h, c->dtype, dst, (float *)dyn_scales + out * b128);
                        break;
                    default:
                        memcpy(dst, row, (size_t)row_bytes);
                        break;
                }
                assist[out * 4 + 0] = src;
                assist[out * 4 + 1] = (int32_t)t;
                assist[out * 4 + 2] = (int32_t)k;
                assist[out * 4 + 3] = tuple_expert;
                ++out;
            }
            send_counts[le * c->rank_size + src] = (int32_t)out;
        }
    }
    int64_t last = 0;
    for (int64_t le = 0; le < out_local; ++le) {
        const int64_t cum = send_counts[le * c->rank_size + c->rank_size - 1];
        expert_token_nums[le] = c->token_nums_type == 0 ? cum : cum - last;
        last = cum;
    }
    return out;
}

/* ------------------------------------------------------------------------------------------------
 * Combine
 * ---------------------------------------------------------------------------------------------- */

/* MVP route: src/ep/kernels/tilexr_ep_combine_kernel.cpp:28-101.
 *   ScatterCombineRows groups each expert rank's rows by recvCounts[src] (counts outside
 *   [0, maxRoutesPerSrc] read as 0) and overwrites the tuple's srcRank with the slot's rank;
 *   DrainCombineRows zeroes y, then walks expert ranks in order and adds every row whose tuple has
 *   0 <= token < bs and 0 <= k < topK:  y = T(float(y) + float(row))  -- one rounding per add (:15-26).
 *   The kernel only runs for fp16 (:125); bf16 with the same per-add rounding is ext. */
void orc_mvp_combine_rank(const orc_case *c, int32_t rank, int64_t max_rows, const uint16_t *expert_out,
    const int32_t *assist, const int32_t *recv_counts, uint16_t *y)
{
    const int64_t max_routes = c->bs * c->top_k;
    const int is_bf16 = c->dtype == ORC_DT_BF16;
    memset(y, 0, (size_t)(c->bs * c->h) * sizeof(uint16_t));
    for (int32_t er = 0; er < c->rank_size; ++er) {
        const int32_t *cnt = recv_counts + (int64_t)er * c->rank_size;
        int64_t in_record = 0;
        for (int32_t s = 0; s < rank; ++s) {
            int64_t n = cnt[s];
            if (n < 0 || n > max_routes) {
                n = 0;
            }
            in_record += n;
        }
        int64_t n = cnt[rank];
        if (n <= 0 || n > max_routes) {
            continue;
        }
        for (int64_t item = 0; item < n; ++item) {
            const int64_t row = in_record + item;
            const int32_t *tuple = assist + ((int64_t)er * max_rows + row) * 4;
            const int32_t token = tuple[1];
            const int32_t k = tuple[2];
            if (token < 0 || (int64_t)token >= c->bs || k < 0 || (int64_t)k >= c->top_k) {
                continue;
            }
            const uint16_t *src = expert_out + ((int64_t)er * max_rows + row) * c->h;
            uint16_t *dst = y + (int64_t)token * c->h;
            for (int64_t i = 0; i < c->h; ++i) {
                if (is_bf16) {
                    dst[i] = orc_float_to_bf16_rne(orc_bf16_to_float(dst[i]) + orc_bf16_to_float(src[i]));
                } else {
                    dst[i] = orc_float_to_half_rne(orc_half_to_float(dst[i]) + orc_half_to_float(src[i]));
                }
            }
        }
    }
}

static int64_t in_row_bytes(const orc_case *c, int32_t in_quant)
{
    return in_quant == 0 ? c->h * 2 : c->h;
}

/* Memory route: src/ep/kernels/tilexr_ep_combine_memory_kernel.h
 *   send     :329-386  row -> slot[token][k] of the tuple's srcRank; rows with rank/token/k out of
 *                      range skipped; rows considered = sendCounts[last] (:256-266)
 *   reduce   :603-669  inactive token (per-token mask test :455-461) -> zeros; else
 *                      sum = 0; for k in 0..K-1: sum += w_k * row_k  (Muls then Add, fp32, :542-551;
 *                      w = 1 without expertScales); then sharedExpertX (:555-571); cast RINT (:595)
 *   mxfp8    comm quant 3 (e5m2) / 4 (e4m3): row is quantised (:360-372) and
 *            sum += (fp8 * 2^(s-127)) * w  (tilexr_ep_mxfp8_quant.h:286-352)
 * The reference waits for every slot of an active token; a slot nobody fills contributes nothing here. */
void orc_mem_combine_rank(const orc_case *c, int32_t rank, int64_t max_rows, const void *expert_out,
    const int32_t *assist, const int32_t *send_counts, const float *expert_scales, const uint8_t *token_mask,
    const uint16_t *shared_expert_x, int32_t comm_quant, int32_t in_quant, const float *in_scales, uint16_t *y)
{
    const int64_t local_e = local_expert_num(c);
    const int64_t n_counts = local_e * c->rank_size;
    const int64_t per_token = c->top_k + c->shared_expert_num;
    const int64_t slots = c->bs * per_token;
    const int64_t rb = in_row_bytes(c, in_quant);
    const int64_t b128 = (c->h + 127) / 128;
    const int64_t in_scales_per_row = in_quant == ORC_QUANT_FP8_BLOCK128 ? b128 : 1;
    const int is_bf16 = c->dtype == ORC_DT_BF16;
    const int32_t fp8 = comm_quant == ORC_QUANT_COMM_MXFP8_E5M2 ? ORC_DT_FP8E5M2 : ORC_DT_FP8E4M3;
    int64_t *slot_row = (int64_t *)malloc((size_t)slots * sizeof(int64_t));
    float *sum = (float *)malloc((size_t)c->h * sizeof(float));
    uint16_t *tmp = (uint16_t *)malloc((size_t)c->h * sizeof(uint16_t));
    uint8_t *q = (uint8_t *)malloc((size_t)c->h);
    uint8_t *qs = (uint8_t *)malloc((size_t)orc_mxfp8_scale_count(c->h));
    for (int64_t i = 0; i < slots; ++i) {
        slot_row[i] = -1;
    }
    for (int32_t er = 0; er < c->rank_size; ++er) {
        int64_t rows = send_counts[(int64_t)er * n_counts + out_local_expert_num(c, er) * c->rank_size - 1];
        if (rows < 0) {
            rows = 0;
        }
        if (rows > max_rows) {
            rows = max_rows;      /* the kernel trusts the count (:256-266); a count beyond the buffer stops at its end here */
        }
        for (int64_t row = 0; row < rows; ++row) {
            const int32_t *tuple = assist + ((int64_t)er * max_rows + row) * 4;
            if (tuple[0] != rank || tuple[1] < 0 || (int64_t)tuple[1] >= c->bs || tuple[2] < 0 ||
                (int64_t)tuple[2] >= per_token) {
                continue;
            }
            slot_row[(int64_t)tuple[1] * per_token + tuple[2]] = (int64_t)er * max_rows + row;
        }
    }
    for (int64_t t = 0; t < c->bs; ++t) {
        uint16_t *dst = y + t * c->h;
        if (token_mask && token_mask[t] == 0) {
            memset(dst, 0, (size_t)c->h * sizeof(uint16_t));
            continue;
        }
        for (int64_t i = 0; i < c->h; ++i) {
            sum[i] = 0.0f;
        }
        /* the top_k routed slots with their gate weights, then the shared slots with weight 1
         * (tilexr_ep_combine_memory_kernel.h:650-657) */
        for (int64_t k = 0; k < per_token; ++k) {
            const int64_t row = slot_row[t * per_token + k];
            if (row < 0) {
                continue;
            }
            const float w = (expert_scales && k < c->top_k) ? expert_scales[t * c->top_k + k] : 1.0f;
            const uint8_t *raw = (const uint8_t *)expert_out + row * rb;
            const uint16_t *elems = (const uint16_t *)raw;
            if (in_quant != 0) {
                const float *sc = in_scales + row * in_scales_per_row;
                for (int64_t i = 0; i < c->h; ++i) {
                    const float d = in_quant == ORC_QUANT_TOKEN_INT8 ?
                        (float)((const int8_t *)raw)[i] * sc[0] :
                        orc_fp8_decode(raw[i], ORC_DT_FP8E4M3) * sc[i / 128];
                    tmp[i] = is_bf16 ? orc_float_to_bf16_rne(d) : orc_float_to_half_rne_sat(d);
                }
                elems = tmp;
            }
            if (comm_quant == ORC_QUANT_COMM_MXFP8_E5M2 || comm_quant == ORC_QUANT_MXFP8) {
                orc_quant_row_mxfp8(elems, c->h, c->dtype, fp8, q, qs);
                for (int64_t i = 0; i < c->h; ++i) {
                    float v = orc_fp8_decode(q[i], fp8) * ldexpf(1.0f, (int)qs[i / 32] - 127);
                    v = v * w;
                    sum[i] = sum[i] + v;
                }
            } else {
                for (int64_t i = 0; i < c->h; ++i) {
                    const float v = decode_elem(elems[i], c->dtype) * w;
                    sum[i] = sum[i] + v;
                }
            }
        }
        if (shared_expert_x) {
            const uint16_t *sx = shared_expert_x + t * c->h;
            for (int64_t i = 0; i < c->h; ++i) {
                sum[i] = sum[i] + decode_elem(sx[i], c->dtype);
            }
        }
        for (int64_t i = 0; i < c->h; ++i) {
            dst[i] = is_bf16 ? orc_float_to_bf16_rne(sum[i]) : orc_float_to_half_rne_sat(sum[i]);
        }
    }
    free(slot_row);
    free(sum);
    free(tmp);
    free(q);
    free(qs);
}
