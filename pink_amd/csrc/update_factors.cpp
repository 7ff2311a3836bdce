// update_factors.cpp -- host-only part of the C ABI: the N x N neighbourhood matrix a
// trainer context is created with.
//
// The reference builds it in TrainerCommon's constructor
// (src/SelfOrganizingMapLib/Trainer.h:62,69-76) from the SOM layout's get_distance
// (CartesianLayout.h:47-60,103-129; HexagonalLayout.h:79-104) and one of the functors of
// src/UtilitiesLib/DistributionFunctor.cpp:19-59.  All arithmetic is float, with the same
// libm calls, so the matrix equals the reference's bit for bit on the same libm.
#include <algorithm>
#include <cmath>
#include <cstdint>
#include <cstdlib>
#include <numeric>
#include <random>
#include <vector>

#include "pink_hip.h"

namespace {

struct Grid {
    uint32_t layout;
    uint32_t dims[3];
    uint32_t ndims;
    std::vector<uint32_t> row_offset;   // hexagonal only
    uint32_t radius = 0;

    uint32_t size() const
    {
        if (layout == PINK_HIP_HEXAGONAL) return dims[0] * dims[0] - radius * (radius + 1);
        uint32_t n = 1;
        for (uint32_t i = 0; i < ndims; ++i) n *= dims[i];
        return n;
    }

    void position(uint32_t i, int64_t p[3]) const
    {
        p[0] = p[1] = p[2] = 0;
        if (layout == PINK_HIP_HEXAGONAL) {
            uint32_t r = 0;
            while (r < dims[0] && i >= row_offset[r + 1]) ++r;
            uint32_t q = i - row_offset[r];
            if (radius > r) q += radius - r;
            p[0] = q;
            p[1] = r;
        } else if (ndims == 1) {
            p[0] = i;
        } else if (ndims == 2) {
            p[0] = i % dims[1];
            p[1] = i / dims[1];
        } else {
            const uint32_t z = i / dims[0] / dims[1];
            p[0] = i % dims[1];
            p[1] = (i - z * dims[0] * dims[1]) / dims[1];
            p[2] = z;
        }
    }

    float distance(uint32_t i1, uint32_t i2) const
    {
        int64_t a[3], b[3];
        position(i1, a);
        position(i2, b);
        if (layout == PINK_HIP_HEXAGONAL) {
            const int32_t dx = static_cast<int32_t>(a[0] - b[0]), dy = static_cast<int32_t>(a[1] - b[1]);
            if ((dx >= 0) == (dy >= 0)) return static_cast<float>(std::abs(dx + dy));
            return static_cast<float>(std::max(std::abs(dx), std::abs(dy)));
        }
        float sum = 0.0f;
        for (uint32_t k = 0; k < ndims; ++k) {
            const float diff = static_cast<float>(a[k]) - static_cast<float>(b[k]);
            sum += static_cast<float>(static_cast<double>(diff) * static_cast<double>(diff));
        }
        return std::sqrt(sum);
    }
};

float neighbourhood(uint32_t kind, float sigma, float damping, float distance)
{
    const float pi = static_cast<float>(M_PI);
    switch (kind) {
    case PINK_HIP_STEP:
        return distance <= sigma ? 1.0f : 0.0f;
    case PINK_HIP_GAUSSIAN:
        return damping / (sigma * std::sqrt(2.0f * pi)) * std::exp(-0.5f * std::pow(distance / sigma, 2.0f));
    case PINK_HIP_UNITY_GAUSSIAN:
        return damping * std::exp(-0.5f * std::pow(distance / sigma, 2.0f));
    default: {
        const float d2 = distance * distance, s2 = sigma * sigma;
        return 2.0f * damping / (std::sqrt(3.0f * sigma) * std::pow(pi, 0.25f)) * (1.0f - d2 / s2)
               * std::exp(-d2 / (2.0f * s2));
    }
    }
}

}  // namespace

extern "C" {

uint32_t pink_hip_som_size(uint32_t layout, const uint32_t *dims, uint32_t ndims)
{
    if (!dims || ndims == 0 || ndims > 3) return 0;
    if (layout == PINK_HIP_HEXAGONAL) {
        if (dims[0] % 2 == 0 || (ndims > 1 && dims[1] != dims[0])) return 0;   // HexagonalLayout.h:40-41
        const uint32_t radius = (dims[0] - 1) / 2;
        return dims[0] * dims[0] - radius * (radius + 1);
    }
    uint32_t n = 1;
    for (uint32_t i = 0; i < ndims; ++i) n *= dims[i];
    return n;
}

static Grid make_grid(uint32_t layout, const uint32_t *dims, uint32_t ndims)
{
    Grid g{};
    g.layout = layout;
    g.ndims = ndims;
    for (uint32_t i = 0; i < 3; ++i) g.dims[i] = i < ndims ? dims[i] : 1;
    if (layout == PINK_HIP_HEXAGONAL) {
        g.radius = (dims[0] - 1) / 2;
        g.row_offset.assign(dims[0] + 1, 0);
        for (uint32_t r = 0; r < dims[0]; ++r) {
            const uint32_t away = r > g.radius ? r - g.radius : g.radius - r;
            g.row_offset[r + 1] = g.row_offset[r] + dims[0] - away;
        }
    }
    return g;
}

int pink_hip_layout_distances(uint32_t layout, const uint32_t *dims, uint32_t ndims, float *distances_out)
{
    const uint32_t N = pink_hip_som_size(layout, dims, ndims);
    if (N == 0 || !distances_out) return PINK_HIP_EINVAL;
    const Grid g = make_grid(layout, dims, ndims);
    for (uint32_t i = 0; i < N; ++i)
        for (uint32_t j = 0; j < N; ++j) distances_out[static_cast<size_t>(i) * N + j] = g.distance(i, j);
    return PINK_HIP_OK;
}

int pink_hip_make_update_factors(uint32_t layout, const uint32_t *dims, uint32_t ndims, uint32_t functor,
                                 float sigma, float damping, float max_update_distance, float *factors_out)
{
    const uint32_t N = pink_hip_som_size(layout, dims, ndims);
    if (N == 0 || !factors_out || functor > PINK_HIP_MEXICAN_HAT) return PINK_HIP_EINVAL;
    if (functor == PINK_HIP_MEXICAN_HAT && sigma <= 0.0f) return PINK_HIP_EINVAL;   // DistributionFunctor.cpp:50
    const Grid g = make_grid(layout, dims, ndims);
    for (uint32_t i = 0; i < N; ++i)
        for (uint32_t j = 0; j < N; ++j) {
            const float d = g.distance(i, j);
            float f = 0.0f;
            if (max_update_distance <= 0 || d < max_update_distance) f = neighbourhood(functor, sigma, damping, d);
            factors_out[static_cast<size_t>(i) * N + j] = f;
        }
    return PINK_HIP_OK;
}

int pink_hip_shuffled_order(uint64_t seed, uint32_t n, uint32_t *order_out)
{
    if (n && !order_out) return PINK_HIP_EINVAL;
    // The order is whatever the C++ library's engines and std::shuffle give for these calls
    // (DataIteratorShuffled.h:62-69): the library decides, as it does for the reference.
    std::iota(order_out, order_out + n, 0u);
    std::default_random_engine engine(seed);
    std::mt19937 generator(engine());
    std::shuffle(order_out, order_out + n, generator);
    return PINK_HIP_OK;
}

int pink_hip_fill_random_uniform(float *values_out, size_t length, uint32_t seed)
{
    if (length && !values_out) return PINK_HIP_EINVAL;
    std::mt19937 generator(seed);
    std::uniform_real_distribution<float> uniform(0.0f);
    for (size_t i = 0; i < length; ++i) values_out[i] = uniform(generator);
    return PINK_HIP_OK;
}

}  // extern "C"
