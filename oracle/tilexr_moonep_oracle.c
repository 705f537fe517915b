/*
 * CPU restatement of the reference's plan-driven (MoonEP) dispatch / combine stage.  TEST INFRASTRUCTURE ONLY: nothing
 * in the product may link or call this file; it exists so that the HIP path can be compared with an independent
 * statement of the reference's algorithm on the same inputs.
 *
 * Each function follows the reference's DEVICE kernels (the behaviour a caller of the library observes), which differ
 * from the reference's own CPU model (tests/moonep/reference/moonep_stage_reference.cpp) in two ways that matter:
 *   - combine sums a duplicate group into its primary row in fp32 and rounds THAT to bf16 before the per-token sum
 *     (src/moonep/combine/kernels/tilexr_moonep_combine_kernel.cpp:449-541), where the CPU model sums all K rows in
 *     fp32 with one rounding (moonep_stage_reference.cpp:354-369);
 *   - the duplicate plan lists groups in the order their first duplicate row appears on the destination rank
 *     (src/moonep/dispatch/kernels/tilexr_moonep_dispatch_kernel.cpp:330-424), where the CPU model lists them in
 *     (source rank, token) order (moonep_stage_reference.cpp:162-232).
 * Where no route is a duplicate the two agree bit for bit, which is how this file is pinned against a build of the
 * reference's CPU model; the duplicate cases are pinned by closed forms in the tests.
 *
 * Pinned by: the known answers of tests/moonep/unit/test_tilexr_moonep_stage_reference.cpp (decode, NvS, padded
 * layout, duplicate plan, balanced round trip = bf16(k * x)), a build of moonep_stage_reference.cpp where the
 * reference checkout is present, and brute-force invariants.  NaN inputs are outside the pinned domain.
 */
#include "tilexr_moonep_oracle.h"

#include <stdlib.h>
#include <string.h>

static inline float bf16_to_float(uint16_t bits)
{
    const uint32_t u = (uint32_t)bits << 16;
    float v;
    memcpy(&v, &u, 4);
    return v;
}

/* round to nearest even (the kernels cast with CAST_RINT, combine kernel :523, :704); NaN stays a quiet NaN */
static inline uint16_t float_to_bf16(float v)
{
    uint32_t u;
    memcpy(&u, &v, 4);
    if ((u & 0x7fffffffu) > 0x7f800000u) {
        return (uint16_t)((u >> 16) | 0x0040u);
    }
    u += 0x7fffu + ((u >> 16) & 1u);
    return (uint16_t)(u >> 16);
}

/* tests/moonep/reference/moonep_stage_reference.cpp:86-107 */
int orc_moon_compute_nvs(int64_t s, int64_t k, int64_t e, int64_t world, int64_t token_padding, int64_t *nvs)
{
    if (nvs == NULL || s <= 0 || k <= 0 || e <= 0 || world <= 0 || token_padding <= 0 || e % world != 0) {
        return -1;
    }
    *nvs = s * k + (token_padding - 1) * 2 * (e / world);
    return 0;
}

/* tests/moonep/reference/moonep_stage_reference.cpp:109-160: cumulative padded ends and the ranges left to zero */
int orc_moon_padded_layout(const int32_t *counts, int64_t groups, int64_t token_padding, int64_t nvs, int32_t *cu_seqlens,
    int32_t *zero_ranges)
{
    if (counts == NULL || groups <= 0 || token_padding <= 0 || nvs <= 0 || cu_seqlens == NULL || zero_ranges == NULL) {
        return -1;
    }
    int64_t cursor = 0;
    for (int64_t g = 0; g < groups; ++g) {
        if (counts[g] < 0) {
            return -1;
        }
        const int64_t real_end = cursor + counts[g];
        int64_t padded_end = real_end;
        if (counts[g] > 0 && real_end % token_padding != 0) {
            padded_end = real_end + token_padding - real_end % token_padding;
        }
        if (padded_end > nvs || padded_end > INT32_MAX) {
            return -1;
        }
        cu_seqlens[g] = (int32_t)padded_end;
        const int64_t zero_end = g + 1 == groups ? nvs : padded_end;
        if (zero_end > real_end) {
            zero_ranges[2 * g] = (int32_t)real_end;
            zero_ranges[2 * g + 1] = (int32_t)(zero_end - real_end);
        } else {
            zero_ranges[2 * g] = 0;
            zero_ranges[2 * g + 1] = 0;
        }
        cursor = padded_end;
    }
    return 0;
}

/* src/moonep/dispatch/kernels/tilexr_moonep_dispatch_kernel.cpp:268-279 (= moonep_stage_reference.cpp:234-251) */
int orc_moon_decode_route(int32_t encoded, int64_t nvs, int64_t world, int64_t *rank, int64_t *offset, int32_t *duplicate)
{
    if (nvs <= 0 || world <= 0) {
        return -1;
    }
    const int64_t e = (int64_t)encoded;
    const int64_t raw = e >= 0 ? e : -e - 1;
    if (raw >= nvs * world) {
        return -1;
    }
    *rank = raw / nvs;
    *offset = raw % nvs;
    *duplicate = encoded < 0;
    return 0;
}

/* Reverse routes as the planner publishes them (src/moonep/planner/kernels/tilexr_moonep_planner_kernel.cpp:250-265,
 * 1051-1082): entry [rank][slot] = source rank * NvS + route index of the route that lands there, -1 elsewhere.  A
 * duplicate route lands in its own slot like any other. */
int orc_moon_build_dst_local(const orc_moon_shape *sh, const int32_t *dst, int32_t *dst_local)
{
    const int64_t n = sh->s * sh->k;
    for (int64_t i = 0; i < sh->world * sh->nvs; ++i) {
        dst_local[i] = -1;
    }
    for (int64_t src = 0; src < sh->world; ++src) {
        for (int64_t route = 0; route < n; ++route) {
            int64_t peer, off;
            int32_t dup;
            if (orc_moon_decode_route(dst[src * n + route], sh->nvs, sh->world, &peer, &off, &dup) != 0) {
                return -1;
            }
            dst_local[peer * sh->nvs + off] = (int32_t)(src * sh->nvs + route);
        }
    }
    return 0;
}

/* dispatch kernel :281-301: the first earlier non-duplicate route of the same token to the same rank */
static int64_t find_primary(const orc_moon_shape *sh, const int32_t *dst_src, int64_t route, int64_t dest_rank)
{
    const int64_t token_start = route / sh->k * sh->k;
    for (int64_t c = token_start; c < route; ++c) {
        if (dst_src[c] < 0) {
            continue;
        }
        int64_t peer, off;
        int32_t dup;
        if (orc_moon_decode_route(dst_src[c], sh->nvs, sh->world, &peer, &off, &dup) != 0) {
            return -1;
        }
        if (peer == dest_rank) {
            return off;
        }
    }
    return -1;
}

/* dispatch kernel :330-424: two passes over the parent table of one destination rank */
static int build_duplicate_plan(int64_t nvs, const int32_t *parents, int32_t *groups, int32_t *loffs, int32_t *counts)
{
    int32_t *group_map = (int32_t *)calloc((size_t)nvs, sizeof(int32_t));
    int32_t group_count = 0, duplicate_count = 0;
    if (group_map == NULL) {
        return -1;
    }
    counts[0] = 0;
    counts[1] = 0;
    for (int64_t loff = 0; loff < nvs; ++loff) {
        if (parents[loff] == 0) {
            continue;
        }
        const int64_t primary = (int64_t)parents[loff] - 1;
        if (primary < 0 || primary >= nvs) {
            free(group_map);
            return 1;
        }
        int32_t group = group_map[primary] - 1;
        if (group_map[primary] == 0) {
            group = group_count++;
            groups[3 * group] = (int32_t)primary;
            groups[3 * group + 1] = 0;
            groups[3 * group + 2] = 0;
            group_map[primary] = group + 1;
        }
        groups[3 * group + 2] += 1;
        ++duplicate_count;
    }
    int32_t prefix = 0;
    for (int32_t g = 0; g < group_count; ++g) {
        const int32_t count = groups[3 * g + 2];
        groups[3 * g + 1] = prefix;
        groups[3 * g + 2] = 0;
        prefix += count;
    }
    for (int64_t loff = 0; loff < nvs; ++loff) {
        if (parents[loff] == 0) {
            continue;
        }
        const int32_t g = group_map[parents[loff] - 1] - 1;
        loffs[groups[3 * g + 1] + groups[3 * g + 2]] = (int32_t)loff;
        groups[3 * g + 2] += 1;
    }
    counts[0] = group_count;
    counts[1] = duplicate_count;
    free(group_map);
    return 0;
}

/* dispatch kernel :108-147 for every rank of the world at once (single hidden chunk: chunking is an artefact of the
 * reference's window size and does not change any output byte) */
int orc_moon_dispatch_world(const orc_moon_shape *sh, const int32_t *dst, const uint16_t *hidden, const float *weights,
    uint64_t flags, int32_t *dup_groups, int32_t *dup_loffs, int32_t *dup_counts, uint16_t *hidden_nvsh,
    float *weights_nvs, int32_t *status)
{
    const int64_t R = sh->world, n = sh->s * sh->k, nvs = sh->nvs, h = sh->h;
    const int build = (flags & ORC_MOON_FLAG_BUILD_DEDUP) != 0;
    int32_t *parents = (int32_t *)calloc((size_t)(R * nvs), sizeof(int32_t));
    if (parents == NULL) {
        return -1;
    }
    /* ClearLocalWindow :206-230: every row and weight of the output starts from zero */
    memset(hidden_nvsh, 0, (size_t)(R * nvs * h) * sizeof(uint16_t));
    if (weights != NULL) {
        memset(weights_nvs, 0, (size_t)(R * nvs) * sizeof(float));
    }
    for (int64_t r = 0; r < R; ++r) {
        status[r] = ORC_MOON_DISPATCH_OK;
    }
    /* ScatterRoutes :303-338 */
    for (int64_t src = 0; src < R; ++src) {
        const int32_t *d = dst + src * n;
        for (int64_t route = 0; route < n; ++route) {
            int64_t peer, off;
            int32_t dup;
            if (orc_moon_decode_route(d[route], nvs, R, &peer, &off, &dup) != 0) {
                status[src] = ORC_MOON_DISPATCH_INVALID_ROUTE;
                break;
            }
            if (!dup) {
                memcpy(hidden_nvsh + (peer * nvs + off) * h, hidden + (src * sh->s + route / sh->k) * h,
                    (size_t)h * sizeof(uint16_t));
            }
            if (weights != NULL) {
                weights_nvs[peer * nvs + off] = weights[src * n + route];
            }
            if (build && dup) {
                const int64_t primary = find_primary(sh, d, route, peer);
                if (primary < 0) {
                    status[src] = ORC_MOON_DISPATCH_INVALID_ROUTE;
                    break;
                }
                parents[peer * nvs + off] = (int32_t)(primary + 1);
            }
        }
    }
    /* a rank whose peer failed reports that peer (WaitAllPeers :559-574 walks peers from its own rank upwards) */
    for (int64_t r = 0; r < R; ++r) {
        if (status[r] != ORC_MOON_DISPATCH_OK) {
            continue;
        }
        for (int64_t o = 0; o < R; ++o) {
            const int64_t peer = (r + o) % R;
            if (status[peer] == ORC_MOON_DISPATCH_INVALID_ROUTE) {
                status[r] = ORC_MOON_DISPATCH_REMOTE_FAILURE_BASE + (int32_t)peer;
                break;
            }
        }
    }
    int ret = 0;
    for (int64_t q = 0; q < R && ret == 0; ++q) {
        int32_t *groups = dup_groups + q * nvs * 3, *loffs = dup_loffs + q * nvs, *counts = dup_counts + q * 2;
        if (status[q] != ORC_MOON_DISPATCH_OK) {
            continue;
        }
        if (build) {
            const int b = build_duplicate_plan(nvs, parents + q * nvs, groups, loffs, counts);
            if (b != 0) {
                status[q] = ORC_MOON_DISPATCH_INVALID_ROUTE;
                ret = b < 0 ? -1 : 0;
                continue;
            }
        }
        /* ExpandDuplicateRows :426-461 */
        if (counts[0] < 0 || counts[0] > nvs || counts[1] < 0 || counts[1] > nvs) {
            status[q] = ORC_MOON_DISPATCH_INVALID_ROUTE;
            continue;
        }
        for (int32_t g = 0; g < counts[0] && status[q] == ORC_MOON_DISPATCH_OK; ++g) {
            const int32_t primary = groups[3 * g], start = groups[3 * g + 1], count = groups[3 * g + 2];
            if (primary < 0 || primary >= nvs || start < 0 || count <= 0 || (int64_t)start + count > counts[1]) {
                status[q] = ORC_MOON_DISPATCH_INVALID_ROUTE;
                break;
            }
            for (int32_t i = 0; i < count; ++i) {
                const int32_t dup = loffs[start + i];
                if (dup < 0 || dup >= nvs) {
                    status[q] = ORC_MOON_DISPATCH_INVALID_ROUTE;
                    break;
                }
                memmove(hidden_nvsh + (q * nvs + dup) * h, hidden_nvsh + (q * nvs + primary) * h,
                    (size_t)h * sizeof(uint16_t));
            }
        }
    }
    free(parents);
    return ret;
}

/* combine kernel :129-177 for every rank of the world at once */
int orc_moon_combine_world(const orc_moon_shape *sh, const int32_t *dst_local, const int32_t *dup_groups,
    const int32_t *dup_loffs, const int32_t *dup_counts, const uint16_t *hidden_nvsh, const float *weights_nvs,
    uint16_t *hidden_sh, float *weights_sk, int32_t *status)
{
    const int64_t R = sh->world, n = sh->s * sh->k, nvs = sh->nvs, h = sh->h;
    uint8_t *mask = (uint8_t *)calloc((size_t)(R * nvs), 1);
    uint16_t *source = (uint16_t *)malloc((size_t)(R * nvs * h) * sizeof(uint16_t));
    uint16_t *recv = (uint16_t *)calloc((size_t)(R * n * h), sizeof(uint16_t));
    float *acc = (float *)malloc((size_t)h * sizeof(float));
    if (mask == NULL || source == NULL || recv == NULL || acc == NULL) {
        free(mask); free(source); free(recv); free(acc);
        return -1;
    }
    /* PrepareChunk :413-447: the expert outputs are copied; the received slots and weights start from zero */
    memcpy(source, hidden_nvsh, (size_t)(R * nvs * h) * sizeof(uint16_t));
    if (weights_nvs != NULL) {
        memset(weights_sk, 0, (size_t)(R * n) * sizeof(float));
    }
    for (int64_t q = 0; q < R; ++q) {
        const int32_t *groups = dup_groups + q * nvs * 3, *loffs = dup_loffs + q * nvs, *counts = dup_counts + q * 2;
        status[q] = ORC_MOON_COMBINE_OK;
        /* BuildDuplicateMask :300-348 */
        if (counts[0] < 0 || counts[0] > nvs || counts[1] < 0 || counts[1] > nvs) {
            status[q] = ORC_MOON_COMBINE_INVALID_ROUTE;
            continue;
        }
        for (int32_t g = 0; g < counts[0] && status[q] == ORC_MOON_COMBINE_OK; ++g) {
            const int32_t primary = groups[3 * g], start = groups[3 * g + 1], count = groups[3 * g + 2];
            if (primary < 0 || primary >= nvs || start < 0 || count <= 0 || (int64_t)start + count > counts[1]) {
                status[q] = ORC_MOON_COMBINE_INVALID_ROUTE;
                break;
            }
            for (int32_t i = 0; i < count; ++i) {
                const int32_t dup = loffs[start + i];
                if (dup < 0 || dup >= nvs || dup == primary) {
                    status[q] = ORC_MOON_COMBINE_INVALID_ROUTE;
                    break;
                }
                mask[q * nvs + dup] = 1;
            }
        }
        /* ValidateReverseRoutes :350-366, DecodeReverseRoute :285-298 */
        for (int64_t row = 0; row < nvs && status[q] == ORC_MOON_COMBINE_OK; ++row) {
            const int32_t enc = dst_local[q * nvs + row];
            if (enc == -1) {
                continue;
            }
            if (enc < 0 || enc / nvs >= R || enc % nvs >= n) {
                status[q] = ORC_MOON_COMBINE_INVALID_ROUTE;
            }
        }
    }
    int failed = 0;
    for (int64_t q = 0; q < R; ++q) {
        failed |= status[q] != ORC_MOON_COMBINE_OK;
    }
    if (failed) {
        /* CrossRankBarrier :391-411: ranks that are fine themselves report the failed peer they meet first */
        for (int64_t r = 0; r < R; ++r) {
            if (status[r] != ORC_MOON_COMBINE_OK) {
                continue;
            }
            for (int64_t peer = 0; peer < R; ++peer) {
                if (status[peer] == ORC_MOON_COMBINE_INVALID_ROUTE) {
                    status[r] = ORC_MOON_COMBINE_REMOTE_FAILURE_BASE + (int32_t)peer;
                    break;
                }
            }
        }
        free(mask); free(source); free(recv); free(acc);
        return 0;
    }
    for (int64_t q = 0; q < R; ++q) {
        const int32_t *groups = dup_groups + q * nvs * 3, *loffs = dup_loffs + q * nvs, *counts = dup_counts + q * 2;
        /* PreReduceDuplicates :449-541: primary = bf16(fp32(primary) + fp32(dup) + ... in list order) */
        for (int32_t g = 0; g < counts[0]; ++g) {
            uint16_t *primary = source + (q * nvs + groups[3 * g]) * h;
            for (int64_t c = 0; c < h; ++c) {
                acc[c] = bf16_to_float(primary[c]);
            }
            for (int32_t i = 0; i < groups[3 * g + 2]; ++i) {
                const uint16_t *dup = source + (q * nvs + loffs[groups[3 * g + 1] + i]) * h;
                for (int64_t c = 0; c < h; ++c) {
                    acc[c] = acc[c] + bf16_to_float(dup[c]);
                }
            }
            for (int64_t c = 0; c < h; ++c) {
                primary[c] = float_to_bf16(acc[c]);
            }
        }
    }
    /* PushPeerRows :568-606 */
    for (int64_t q = 0; q < R; ++q) {
        for (int64_t row = 0; row < nvs; ++row) {
            const int32_t enc = dst_local[q * nvs + row];
            if (enc == -1) {
                continue;
            }
            const int64_t peer = enc / nvs, target = enc % nvs;
            if (!mask[q * nvs + row]) {
                memcpy(recv + (peer * n + target) * h, source + (q * nvs + row) * h, (size_t)h * sizeof(uint16_t));
            }
            if (weights_nvs != NULL) {
                weights_sk[peer * n + target] = weights_nvs[q * nvs + row];
            }
        }
    }
    /* ReduceHiddenChunk :648-717: zero, then the K received slots in slot order, fp32, one rounding */
    for (int64_t p = 0; p < R; ++p) {
        for (int64_t t = 0; t < sh->s; ++t) {
            for (int64_t c = 0; c < h; ++c) {
                acc[c] = 0.0f;
            }
            for (int64_t kk = 0; kk < sh->k; ++kk) {
                const uint16_t *row = recv + (p * n + t * sh->k + kk) * h;
                for (int64_t c = 0; c < h; ++c) {
                    acc[c] = acc[c] + bf16_to_float(row[c]);
                }
            }
            for (int64_t c = 0; c < h; ++c) {
                hidden_sh[(p * sh->s + t) * h + c] = float_to_bf16(acc[c]);
            }
        }
    }
    free(mask); free(source); free(recv); free(acc);
    return 0;
}
