// ref_shim.cpp -- TEST INFRASTRUCTURE ONLY.
//
// extern "C" entry points over the REAL reference headers, compiled where they
// lie (-I<reference>/src) into oracle/_ref/libpink_ref.so by oracle/Makefile.
// Only headers that build from the reference tree as it is are included:
// ImageProcessingLib/*, SelfOrganizingMapLib/{CartesianLayout,HexagonalLayout,
// Data,generate_rotated_images}.h, UtilitiesLib/{DistributionFunctor,Filler}.h.
// Trainer.h, Mapper.h, SOM.h and generate_euclidean_distance_matrix.h include
// UtilitiesLib/InputData.h, which needs a header the reference's CMake generates
// (Version.h); they are not built here.
//
// Used by tests to check oracle/pink_oracle.c bit-for-bit and to write golden
// fixtures.  Never shipped, never linked into the library.
#include <cmath>
#include <cstdint>
#include <cstring>
#include <vector>

#include "SelfOrganizingMapLib/CartesianLayout.h"
#include "SelfOrganizingMapLib/HexagonalLayout.h"
#include "SelfOrganizingMapLib/Data.h"
#include "SelfOrganizingMapLib/generate_rotated_images.h"
#include "ImageProcessingLib/euclidean_distance.h"
#include "ImageProcessingLib/circular_euclidean_distance.h"
#include "UtilitiesLib/DistributionFunctor.h"
#include "UtilitiesLib/Filler.h"
#include "SelfOrganizingMapLib/DataIteratorShuffled.h"
#include "UtilitiesLib/ProgressBar.h"
#include <sstream>

using namespace pink;

namespace {

template <typename T>
T ssd(const T* a, const T* b, uint32_t channels, uint32_t dim, uint32_t ed, uint32_t shape, uint32_t data_dims)
{
    if (data_dims == 2) {
        CartesianLayout<2> layout{{dim, dim}};
        if (shape == 0) return EuclideanDistanceFunctor<CartesianLayout<2>>()(a, b, layout, ed);
        return CircularEuclideanDistanceFunctor<CartesianLayout<2>>()(a, b, layout, ed);
    }
    CartesianLayout<3> layout{{channels, dim, dim}};
    if (shape == 0) return EuclideanDistanceFunctor<CartesianLayout<3>>()(a, b, layout, ed);
    return CircularEuclideanDistanceFunctor<CartesianLayout<3>>()(a, b, layout, ed);
}

} // namespace

extern "C" {

void ref_rotate_bilinear(const float* src, float* dst, uint32_t sh, uint32_t sw, uint32_t dh, uint32_t dw, float alpha)
{
    rotate_bilinear(src, dst, sh, sw, dh, dw, alpha);
}

void ref_resize(const float* src, float* dst, uint32_t sh, uint32_t sw, uint32_t dh, uint32_t dw)
{
    resize(src, dst, sh, sw, dh, dw);
}

/// data_dims = 2: SpatialTransformer<CartesianLayout<2>>; 3: <CartesianLayout<3>> (channel-first)
int ref_rotated_images(const float* image, uint32_t channels, uint32_t image_dim, uint32_t neuron_dim,
    uint32_t num_rot, int use_flip, uint32_t data_dims, float* out)
{
    try {
        std::vector<float> result;
        if (data_dims == 2) {
            Data<CartesianLayout<2>, float> data({{image_dim, image_dim}},
                std::vector<float>(image, image + size_t(image_dim) * image_dim));
            CartesianLayout<2> neuron_layout{{neuron_dim, neuron_dim}};
            result = SpatialTransformer<CartesianLayout<2>>()(data, num_rot, use_flip != 0,
                Interpolation::BILINEAR, neuron_layout);
        } else {
            Data<CartesianLayout<3>, float> data({{channels, image_dim, image_dim}},
                std::vector<float>(image, image + size_t(channels) * image_dim * image_dim));
            CartesianLayout<3> neuron_layout{{channels, neuron_dim, neuron_dim}};
            result = SpatialTransformer<CartesianLayout<3>>()(data, num_rot, use_flip != 0,
                Interpolation::BILINEAR, neuron_layout);
        }
        std::memcpy(out, result.data(), result.size() * sizeof(float));
        return static_cast<int>(result.size());
    } catch (...) {
        return -1;
    }
}

/// Integer instantiation used by the reference's own test (generate_rotated_images.cpp:15-41)
int ref_rotated_images_int(const int* image, uint32_t channels, uint32_t image_dim, uint32_t neuron_dim,
    uint32_t num_rot, int use_flip, uint32_t data_dims, int* out)
{
    std::vector<int> result;
    if (data_dims == 2) {
        Data<CartesianLayout<2>, int> data({{image_dim, image_dim}},
            std::vector<int>(image, image + size_t(image_dim) * image_dim));
        CartesianLayout<2> neuron_layout{{neuron_dim, neuron_dim}};
        result = SpatialTransformer<CartesianLayout<2>>()(data, num_rot, use_flip != 0,
            Interpolation::BILINEAR, neuron_layout);
    } else {
        Data<CartesianLayout<3>, int> data({{channels, image_dim, image_dim}},
            std::vector<int>(image, image + size_t(channels) * image_dim * image_dim));
        CartesianLayout<3> neuron_layout{{channels, neuron_dim, neuron_dim}};
        result = SpatialTransformer<CartesianLayout<3>>()(data, num_rot, use_flip != 0,
            Interpolation::BILINEAR, neuron_layout);
    }
    std::memcpy(out, result.data(), result.size() * sizeof(int));
    return static_cast<int>(result.size());
}

float ref_ssd_f32(const float* a, const float* b, uint32_t channels, uint32_t dim, uint32_t ed,
    uint32_t shape, uint32_t data_dims)
{
    return ssd<float>(a, b, channels, dim, ed, shape, data_dims);
}

int32_t ref_ssd_i32(const int32_t* a, const int32_t* b, uint32_t channels, uint32_t dim, uint32_t ed,
    uint32_t shape, uint32_t data_dims)
{
    return ssd<int32_t>(a, b, channels, dim, ed, shape, data_dims);
}

int64_t ref_ssd_i64(const int64_t* a, const int64_t* b, uint32_t channels, uint32_t dim, uint32_t ed,
    uint32_t shape, uint32_t data_dims)
{
    return ssd<int64_t>(a, b, channels, dim, ed, shape, data_dims);
}

float ref_cartesian_distance(const uint32_t* dims, uint32_t ndims, uint32_t i1, uint32_t i2)
{
    if (ndims == 1) return CartesianLayout<1>{{dims[0]}}.get_distance(i1, i2);
    if (ndims == 2) return CartesianLayout<2>{{dims[0], dims[1]}}.get_distance(i1, i2);
    return CartesianLayout<3>{{dims[0], dims[1], dims[2]}}.get_distance(i1, i2);
}

uint32_t ref_hex_size(uint32_t dim)
{
    HexagonalLayout::DimensionType d{{dim, dim}};
    return HexagonalLayout(d).size();
}

float ref_hex_distance(uint32_t dim, uint32_t i1, uint32_t i2)
{
    HexagonalLayout::DimensionType d{{dim, dim}};
    return HexagonalLayout(d).get_distance(i1, i2);
}

/// kind: 0 Step, 1 Gaussian, 2 UnityGaussian, 3 MexicanHat
float ref_functor(uint32_t kind, float sigma, float damping, float distance)
{
    switch (kind) {
        case 0: return StepFunctor(sigma)(distance);
        case 1: return GaussianFunctor(sigma, damping)(distance);
        case 2: return UnityGaussianFunctor(sigma, damping)(distance);
        default: return MexicanHatFunctor(sigma, damping)(distance);
    }
}

void ref_fill_random_uniform(float* a, size_t n, uint32_t seed) { fill_random_uniform(a, n, seed); }

/// The visiting order of the reference's DataIteratorShuffled over an in-memory data file of
/// n one-pixel images whose pixel is the entry's index.
void ref_shuffled_order(uint64_t seed, uint32_t n, int shuffle, uint32_t* order)
{
    std::stringstream ss;
    const int head[8] = {2, 0, 0, static_cast<int>(n), 0, 2, 1, 1};
    ss.write(reinterpret_cast<const char*>(head), sizeof(head));
    for (uint32_t i = 0; i < n; ++i) {
        const float v = static_cast<float>(i);
        ss.write(reinterpret_cast<const char*>(&v), sizeof(v));
    }
    DataIteratorShuffled<CartesianLayout<2>, float> it(ss, seed, shuffle != 0);
    const DataIteratorShuffled<CartesianLayout<2>, float> end(ss, true);
    for (uint32_t i = 0; it != end && i < n; ++it, ++i) order[i] = static_cast<uint32_t>((*it)[0]);
}

/// The ticks at which the training loop of Pink/main_generic.h:78-90 finds ProgressBar::valid() true
/// (checked after each image, before the increment); returns their number.
int ref_progress_ticks(int total, int max_prints, int* ticks_out)
{
    std::stringstream sink;
    ProgressBar bar(total, 70, max_prints, sink);
    int k = 0;
    for (int t = 0; t < total; ++t, ++bar)
        if (bar.valid()) ticks_out[k++] = t;
    return k;
}

} // extern "C"
