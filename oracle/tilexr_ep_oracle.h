/*
 * CPU oracle for the single-device MoE expert-parallel dispatch / combine path.
 *
 * THIS IS TEST INFRASTRUCTURE, NOT PRODUCT CODE.  It restates, in plain scalar C, what the
 * reference's kernels and golden models compute, so that the HIP kernels can be checked
 * bit-for-bit.  Only tests, the smoke check and the benchmark's cpu_baseline leg may load it.
 * Nothing in the shipped library links, loads or falls back to anything in this directory.
 *
 * Every function cites the reference file:line it follows (paths relative to the reference
 * checkout).  "ext" marks behaviour the reference does not have (bf16-decoded int8 quant,
 * per-128-column fp8 with fp32 scales, per-expert capacity, quantised combine input); those
 * are defined by this repository's workload list and are pinned by closed forms and library
 * casts in the tests, not by reference vectors.
 *
 * Pin status:
 *   orc_half_to_float / orc_bf16_to_float / float->half / float->bf16 : numpy / torch casts
 *   orc_clamp_int8, per-token int8 (fp16 decode)  : reference formula + demo values
 *   per-token int8 (bf16 decode, ext)             : closed form, exhaustive bf16 sweep
 *   orc_fp8_encode / orc_mxfp8_quant_row          : reference byte goldens + reference golden header build
 *   fp8 block-128 (ext)                           : torch.float8_e4m3fn cast  (reference: parity unpinned)
 *   MVP dispatch order / counts                   : reference checker known answers + checker build
 *   memory dispatch order / sendCounts            : stable-sort invariant + brute force + demo golden restated
 *   capacity drop (ext)                           : brute force            (reference: parity unpinned)
 *   MVP combine (per-add rounding)                : numpy float16 sequential sum
 *   memory combine (fp32 acc, RINT)               : numpy float32 sequential sum + torch cast
 *   shared experts (both routes)                  : the reference demo's golden route model restated as a
 *                                                   brute-force walk in the tests, closed-form row counts
 *   tensor-parallel groups (MVP route)            : the demo's BuildExpectedTpRoutes restated in the tests
 */
#ifndef TILEXR_EP_ORACLE_H
#define TILEXR_EP_ORACLE_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

enum {
    ORC_DT_INT8 = 0,
    ORC_DT_FP16 = 3,
    ORC_DT_BF16 = 11,
    ORC_DT_FP8E4M3 = 15,
    ORC_DT_FP8E5M2 = 16
};

enum {
    ORC_QUANT_NONE = 0,
    ORC_QUANT_STATIC_INT8 = 1,    /* MVP route only */
    ORC_QUANT_TOKEN_INT8 = 2,     /* MVP route (fp16 decode); memory route = ext (decode by dtype) */
    ORC_QUANT_COMM_MXFP8_E5M2 = 3,/* memory combine only */
    ORC_QUANT_MXFP8 = 4,          /* memory dispatch: out dtype selects e4m3/e5m2; combine: e4m3 */
    ORC_QUANT_FP8_BLOCK128 = 5    /* ext */
};

enum { ORC_MASK_NONE = 0, ORC_MASK_TOKEN = 1, ORC_MASK_EXPERT = 2 };

typedef struct {
    int32_t rank_size;        /* logical ranks sharing the device (R) */
    int64_t bs;               /* tokens per source rank */
    int64_t h;
    int64_t top_k;
    int64_t moe_expert_num;   /* E, divisible by R */
    int32_t dtype;            /* ORC_DT_FP16 / ORC_DT_BF16: input element type */
    int32_t quant_mode;
    int32_t out_dtype;        /* fp8 flavour for ORC_QUANT_MXFP8 */
    int32_t token_nums_type;  /* 0 = inclusive prefix sum, 1 = counts */
    int32_t mask_type;
    int64_t capacity;         /* ext: rows kept per expert per destination (0 = unlimited) */
    int64_t shared_expert_num;      /* S: every active token also goes to each of S shared experts */
    int64_t shared_expert_rank_num; /* ranks [0, SR) host the shared experts (SR % S == 0); E % (R - SR) == 0 */
    int64_t tp_world_size;          /* MVP route: ranks form groups of this many lanes (0 or 1 = none); the
                                       placement rules then run over the R / tp expert ranks */
} orc_case;

/* ---- scalar numerics ---- */
float orc_half_to_float(uint16_t bits);
float orc_bf16_to_float(uint16_t bits);
uint16_t orc_float_to_half_rne_sat(float v);   /* saturates to +-65504 */
uint16_t orc_float_to_half_rne(float v);       /* IEEE (overflow -> inf) */
uint16_t orc_float_to_bf16_rne(float v);
int8_t orc_clamp_int8(float v);
uint8_t orc_fp8_encode(float v, int32_t fp8_dtype);
float orc_fp8_decode(uint8_t v, int32_t fp8_dtype);
int64_t orc_mxfp8_scale_count(int64_t h);

/* ---- row quantisers (src = h elements of `dtype`) ---- */
float orc_quant_row_token_int8(const uint16_t *src, int64_t h, int32_t decode_dtype, int8_t *dst);
void orc_quant_row_static_int8(const uint16_t *src, int64_t h, float scale, int8_t *dst);
void orc_quant_row_mxfp8(const uint16_t *src, int64_t h, int32_t dtype, int32_t fp8_dtype,
    uint8_t *dst, uint8_t *scales);
void orc_quant_row_fp8_block128(const uint16_t *src, int64_t h, int32_t dtype, uint8_t *dst, float *scales);

/* ---- dispatch (outputs of ONE destination rank, inputs of ALL source ranks) ----
 * x     [R][bs*h] u16, ids [R][bs*top_k], mask [R][bs] or [R][bs*top_k] (may be NULL)
 * Returns the number of rows written.
 * With shared experts a token emits its S shared routes (topKId = top_k + s, expertId = s, destination rank
 * src % (SR/S) + s * (SR/S)) before its top_k routed ones (expertId = S + id, destination SR + id / localE),
 * localE = E / (R - SR).  expert_token_nums has localE entries (MVP route) or, on the memory route, 1 entry on
 * a shared rank and localE on the others; send_counts likewise 1*R or localE*R entries. */
/* With tensor-parallel groups (tp lanes per expert rank) a rank receives from the sources of its own lane, then
 * appends what the other lanes of its group received, in lane order.  recv_counts[src] is written for own-lane
 * sources only (other entries are left as they are); tp_recv_counts (may be NULL when tp <= 1) gets the same
 * per-source entries and then rows per lane in its first tp entries. */
int64_t orc_mvp_dispatch_rank(const orc_case *c, int32_t dst_rank, const uint16_t *x, const int32_t *ids,
    const uint8_t *mask, const float *static_scale, uint8_t *expand_x, float *dyn_scales, int32_t *assist,
    int32_t *recv_counts, int32_t *tp_recv_counts, int64_t *expert_token_nums);

int64_t orc_mem_dispatch_rank(const orc_case *c, int32_t dst_rank, const uint16_t *x, const int32_t *ids,
    const uint8_t *mask, uint8_t *expand_x, uint8_t *dyn_scales, int32_t *assist, int32_t *send_counts,
    int64_t *expert_token_nums);

/* ---- combine (output of ONE source rank, inputs of ALL expert ranks) ----
 * expert_out [R][max_rows*row_bytes], assist [R][max_rows*4], counts [R][R] (MVP) or [R][localE*R] (memory;
 * a shared rank uses the first R entries of its block). */
void orc_mvp_combine_rank(const orc_case *c, int32_t rank, int64_t max_rows, const uint16_t *expert_out,
    const int32_t *assist, const int32_t *recv_counts, uint16_t *y);

/* in_quant: 0 -> expert_out is `dtype`; ORC_QUANT_TOKEN_INT8 / ORC_QUANT_FP8_BLOCK128 (ext) -> expert_out
 * holds quantised rows with in_scales [R][max_rows*scales_per_row]; each element is dequantised, rounded
 * to `dtype`, then reduced.  comm_quant 3/4 applies the reference's MXFP8 round trip to every row first. */
void orc_mem_combine_rank(const orc_case *c, int32_t rank, int64_t max_rows, const void *expert_out,
    const int32_t *assist, const int32_t *send_counts, const float *expert_scales, const uint8_t *token_mask,
    const uint16_t *shared_expert_x, int32_t comm_quant, int32_t in_quant, const float *in_scales, uint16_t *y);

#ifdef __cplusplus
}
#endif
#endif
