// C entry points over the reference's CPU model of the MoonEP stages, compiled from where it lies
// (tests/moonep/reference/moonep_stage_reference.cpp).  Test infrastructure: used to pin the CPU oracle.
// Arrays are flat and world-major, as in oracle/tilexr_moonep_oracle.h.
#include <cstdint>
#include <cstring>
#include <vector>

#include "moonep_stage_reference.h"

namespace Ref = TileXRMoonEp::Reference;

namespace {

Ref::Shape MakeShape(int64_t world, int64_t s, int64_t k, int64_t h, int64_t nvs)
{
    Ref::Shape shape;
    shape.world = world;
    shape.s = s;
    shape.k = k;
    shape.h = h;
    shape.nvS = nvs;
    return shape;
}

Ref::Destinations MakeDst(const Ref::Shape &shape, const int32_t *dst)
{
    const size_t n = static_cast<size_t>(shape.s * shape.k);
    Ref::Destinations out(static_cast<size_t>(shape.world));
    for (size_t r = 0; r < out.size(); ++r) {
        out[r].assign(dst + r * n, dst + (r + 1) * n);
    }
    return out;
}

template <typename T>
std::vector<std::vector<T>> Split(const T *flat, int64_t world, int64_t per)
{
    std::vector<std::vector<T>> out(static_cast<size_t>(world));
    for (size_t r = 0; r < out.size(); ++r) {
        out[r].assign(flat + r * static_cast<size_t>(per), flat + (r + 1) * static_cast<size_t>(per));
    }
    return out;
}

template <typename T>
void Join(const std::vector<std::vector<T>> &parts, T *flat)
{
    size_t at = 0;
    for (const auto &p : parts) {
        std::memcpy(flat + at, p.data(), p.size() * sizeof(T));
        at += p.size();
    }
}

} // namespace

extern "C" {

int ref_moon_compute_nvs(int64_t s, int64_t k, int64_t e, int64_t world, int64_t padding, int64_t *nvs)
{
    return Ref::ComputeNvS(s, k, e, world, padding, nvs);
}

int ref_moon_padded_layout(const int32_t *counts, int64_t groups, int64_t padding, int64_t nvs, int32_t *cu, int32_t *ranges)
{
    std::vector<int32_t> c(counts, counts + groups), cuOut;
    Ref::FillRanges r;
    const int ret = Ref::BuildPaddedLayout(c, padding, nvs, &cuOut, &r);
    if (ret == 0) {
        for (int64_t g = 0; g < groups; ++g) {
            cu[g] = cuOut[static_cast<size_t>(g)];
            ranges[2 * g] = r[static_cast<size_t>(g)][0];
            ranges[2 * g + 1] = r[static_cast<size_t>(g)][1];
        }
    }
    return ret;
}

int ref_moon_decode_route(int32_t encoded, int64_t capacity, int64_t world, int64_t *rank, int64_t *offset, int32_t *dup)
{
    Ref::DecodedRoute route {};
    const int ret = Ref::DecodeRoute(encoded, capacity, world, &route);
    if (ret == 0) {
        *rank = route.rank;
        *offset = route.offset;
        *dup = route.duplicate ? 1 : 0;
    }
    return ret;
}

uint16_t ref_moon_float_to_bf16(float v) { return Ref::FloatToBfloat16(v); }

int ref_moon_dispatch_bf16(int64_t world, int64_t s, int64_t k, int64_t h, int64_t nvs, const int32_t *dst,
    const uint16_t *hidden, uint16_t *out)
{
    const Ref::Shape shape = MakeShape(world, s, k, h, nvs);
    Ref::Bfloat16Ranks result;
    const int ret = Ref::DispatchBfloat16(shape, MakeDst(shape, dst), Split(hidden, world, s * h), &result);
    if (ret == 0) {
        Join(result, out);
    }
    return ret;
}

int ref_moon_dispatch_f32(int64_t world, int64_t s, int64_t k, int64_t nvs, const int32_t *dst, const float *weights,
    float *out)
{
    const Ref::Shape shape = MakeShape(world, s, k, 0, nvs);
    Ref::Float32Ranks result;
    const int ret = Ref::DispatchFloat32(shape, MakeDst(shape, dst), Split(weights, world, s * k), &result);
    if (ret == 0) {
        Join(result, out);
    }
    return ret;
}

int ref_moon_combine_bf16(int64_t world, int64_t s, int64_t k, int64_t h, int64_t nvs, const int32_t *dst,
    const uint16_t *hiddenNvsh, uint16_t *out)
{
    const Ref::Shape shape = MakeShape(world, s, k, h, nvs);
    Ref::Bfloat16Ranks result;
    const int64_t rows = nvs > 0 ? nvs : s * k;
    const int ret = Ref::CombineBfloat16(shape, MakeDst(shape, dst), Split(hiddenNvsh, world, rows * h), &result);
    if (ret == 0) {
        Join(result, out);
    }
    return ret;
}

int ref_moon_combine_f32(int64_t world, int64_t s, int64_t k, int64_t nvs, const int32_t *dst, const float *weightsNvs,
    float *out)
{
    const Ref::Shape shape = MakeShape(world, s, k, 0, nvs);
    Ref::Float32Ranks result;
    const int64_t rows = nvs > 0 ? nvs : s * k;
    const int ret = Ref::CombineFloat32(shape, MakeDst(shape, dst), Split(weightsNvs, world, rows), &result);
    if (ret == 0) {
        Join(result, out);
    }
    return ret;
}

// Duplicate plans of every destination rank: groups [world][nvs*3], loffs [world][nvs], counts [world][2].
int ref_moon_duplicate_plans(int64_t world, int64_t s, int64_t k, int64_t nvs, const int32_t *dst, int32_t *groups,
    int32_t *loffs, int32_t *counts)
{
    const Ref::Shape shape = MakeShape(world, s, k, 0, nvs);
    Ref::DuplicatePlans plans;
    const int ret = Ref::BuildDuplicatePlans(shape, MakeDst(shape, dst), &plans);
    if (ret != 0) {
        return ret;
    }
    const int64_t rows = nvs > 0 ? nvs : s * k;
    for (int64_t r = 0; r < world; ++r) {
        const Ref::DuplicatePlan &p = plans[static_cast<size_t>(r)];
        for (size_t g = 0; g < p.groups.size(); ++g) {
            for (int j = 0; j < 3; ++j) {
                groups[(r * rows + static_cast<int64_t>(g)) * 3 + j] = p.groups[g][static_cast<size_t>(j)];
            }
        }
        for (size_t i = 0; i < p.loffs.size(); ++i) {
            loffs[r * rows + static_cast<int64_t>(i)] = p.loffs[i];
        }
        counts[2 * r] = p.counts[0];
        counts[2 * r + 1] = p.counts[1];
    }
    return 0;
}

} // extern "C"
