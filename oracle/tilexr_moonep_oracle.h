/*
 * CPU restatement of the reference's plan-driven (MoonEP) dispatch / combine stage -- test infrastructure only.
 * See tilexr_moonep_oracle.c for what each function follows and how it is pinned.
 *
 * Arrays are flat and world-major: [world][...] for every per-rank tensor.
 */
#ifndef TILEXR_MOONEP_ORACLE_H
#define TILEXR_MOONEP_ORACLE_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define ORC_MOON_FLAG_BUILD_DEDUP 1ull            /* src/include/tilexr_moonep.h:22 */

/* src/moonep/common/moonep_peer_window.h:36-43; the combine kernel stores 0 on success (combine kernel :727-733) */
#define ORC_MOON_DISPATCH_OK 2000
#define ORC_MOON_DISPATCH_INVALID_ROUTE 2001
#define ORC_MOON_DISPATCH_REMOTE_FAILURE_BASE 2100
#define ORC_MOON_COMBINE_OK 0
#define ORC_MOON_COMBINE_INVALID_ROUTE 3001
#define ORC_MOON_COMBINE_REMOTE_FAILURE_BASE 3100

typedef struct {
    int64_t world;   /* ranks */
    int64_t s;       /* tokens per rank */
    int64_t k;       /* routes per token */
    int64_t h;       /* hidden size (bf16 elements) */
    int64_t nvs;     /* rows of every rank's receive tensor, >= s * k */
} orc_moon_shape;

int orc_moon_compute_nvs(int64_t s, int64_t k, int64_t e, int64_t world, int64_t token_padding, int64_t *nvs);
int orc_moon_padded_layout(const int32_t *counts, int64_t groups, int64_t token_padding, int64_t nvs, int32_t *cu_seqlens,
    int32_t *zero_ranges /* [groups][2] */);
int orc_moon_decode_route(int32_t encoded, int64_t nvs, int64_t world, int64_t *rank, int64_t *offset, int32_t *duplicate);
int orc_moon_build_dst_local(const orc_moon_shape *sh, const int32_t *dst /* [world][s*k] */,
    int32_t *dst_local /* [world][nvs] */);

/* dst [world][s*k]; hidden [world][s*h]; weights [world][s*k] or NULL; dup_groups [world][nvs*3], dup_loffs [world][nvs],
 * dup_counts [world][2] are outputs with ORC_MOON_FLAG_BUILD_DEDUP and inputs without; hidden_nvsh [world][nvs*h];
 * weights_nvs [world][nvs] (when weights != NULL); status [world]. */
int orc_moon_dispatch_world(const orc_moon_shape *sh, const int32_t *dst, const uint16_t *hidden, const float *weights,
    uint64_t flags, int32_t *dup_groups, int32_t *dup_loffs, int32_t *dup_counts, uint16_t *hidden_nvsh,
    float *weights_nvs, int32_t *status);

/* dst_local [world][nvs]; hidden_nvsh [world][nvs*h]; weights_nvs [world][nvs] or NULL; hidden_sh [world][s*h];
 * weights_sk [world][s*k] (when weights_nvs != NULL); status [world]. */
int orc_moon_combine_world(const orc_moon_shape *sh, const int32_t *dst_local, const int32_t *dup_groups,
    const int32_t *dup_loffs, const int32_t *dup_counts, const uint16_t *hidden_nvsh, const float *weights_nvs,
    uint16_t *hidden_sh, float *weights_sk, int32_t *status);

#ifdef __cplusplus
}
#endif

#endif /* TILEXR_MOONEP_ORACLE_H */
