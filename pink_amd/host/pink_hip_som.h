// pink_hip_som.h -- the GPU specialisations pink::Trainer<..., true> and
// pink::Mapper<..., true> on top of the C ABI (include/pink_hip.h), for a plain C++17
// host compiler.
//
// They take the place of the nvcc-only specialisations of the reference
// (src/SelfOrganizingMapLib/Trainer.h:198-337, Mapper.h:126-232): same constructor
// arguments, same operator(), update_som(), get_update_info(), same exceptions for bad
// arguments.  Inside the reference tree include this header after Trainer.h / Mapper.h
// (built without nvcc, so their own `true` specialisations are not compiled) and link
// libpink_hip.so.  Outside it, define PINK_HIP_STANDALONE to get the small set of
// containers, enums and functors of pink_hip_standalone.h that carry the same member
// names.
//
// The templates only use what the reference's SOM, Data and layout classes offer:
//   som.get_som_layout().size() / .get_distance(i, j), som.get_neuron_layout().m_dimension,
//   som.get_data_pointer(), som.get_number_of_neurons(), som.get_neuron_size(),
//   data.get_layout().m_dimension, data.get_data_pointer().
#pragma once

#include <cstdint>
#include <functional>
#include <string>
#include <tuple>
#include <type_traits>
#include <vector>

#include "pink_hip.h"

#ifdef PINK_HIP_STANDALONE
#include "pink_hip_standalone.h"
#endif

namespace pink {

template <typename SOMLayout, typename DataLayout, typename T, bool UseGPU>
class Trainer;
template <typename SOMLayout, typename DataLayout, typename T, bool UseGPU>
class Mapper;

namespace hip_detail {

/// channels and edge length of a CartesianLayout<2> (edge, edge) or <3> (channels, edge, edge)
template <typename Layout>
inline void image_geometry(Layout const& layout, uint32_t& channels, uint32_t& edge)
{
    static_assert(Layout::dimensionality == 2 || Layout::dimensionality == 3,
        "only 2-dimensional and channel-first 3-dimensional data exist on the device");
    auto const dim = layout.m_dimension;
    if (Layout::dimensionality == 2) {
        if (dim[0] != dim[1]) throw pink::exception("Images must be quadratic.");
        channels = 1;
        edge = dim[0];
    } else {
        if (dim[1] != dim[Layout::dimensionality - 1]) throw pink::exception("Images must be quadratic.");
        channels = dim[0];
        edge = dim[1];
    }
}

inline void check(pink_hip_ctx* ctx, int status)
{
    if (status != PINK_HIP_OK) throw pink::exception(pink_hip_last_error(ctx));
}

/// Owns one pink_hip_ctx.
class Context
{
public:
    Context() = default;
    Context(Context const&) = delete;
    Context& operator = (Context const&) = delete;
    ~Context() { pink_hip_destroy(m_ctx); }

    template <typename SOMType>
    void create(SOMType const& som, std::vector<float> const* update_factors, uint32_t number_of_rotations,
        bool use_flip, Interpolation interpolation, uint32_t euclidean_distance_dim,
        EuclideanDistanceShape euclidean_distance_shape, DataType euclidean_distance_type)
    {
        pink_hip_config cfg{};
        cfg.som_size = som.get_number_of_neurons();
        image_geometry(som.get_neuron_layout(), cfg.channels, cfg.neuron_dim);
        cfg.image_dim = cfg.neuron_dim;     // set for real by the first image
        cfg.num_rot = number_of_rotations;
        cfg.use_flip = use_flip ? 1 : 0;
        cfg.interpolation = interpolation == Interpolation::BILINEAR ? PINK_HIP_BILINEAR : PINK_HIP_NEAREST_NEIGHBOR;
        cfg.ed_dim = euclidean_distance_dim;
        cfg.ed_shape = euclidean_distance_shape == EuclideanDistanceShape::CIRCULAR ? PINK_HIP_CIRCULAR : PINK_HIP_QUADRATIC;
        cfg.ed_type = euclidean_distance_type == DataType::UINT8 ? PINK_HIP_UINT8
                    : euclidean_distance_type == DataType::UINT16 ? PINK_HIP_UINT16 : PINK_HIP_FLOAT;
        cfg.update_factors = update_factors ? update_factors->data() : nullptr;
        m_cfg = cfg;
        if (update_factors) m_factors = *update_factors;
        m_som_copy.assign(som.get_data_pointer(), som.get_data_pointer() + som.size());
        // Validate the arguments now (the reference throws from the constructor); the device
        // context itself is built when the first image tells the image size.
        if (number_of_rotations == 0 or (number_of_rotations != 1 and number_of_rotations % 4 != 0))
            throw pink::exception("Number of rotations must be 1 or larger then 1 and divisible by 4");
        if (euclidean_distance_dim > cfg.neuron_dim)
            throw pink::exception("Euclidean distance dimension larger than neuron dimension");
    }

    /// (Re)build the device context for images of the given geometry.
    pink_hip_ctx* for_image(uint32_t channels, uint32_t image_dim)
    {
        if (channels != m_cfg.channels) throw pink::exception("image and neuron channel counts differ");
        if (m_ctx and image_dim == m_cfg.image_dim) return m_ctx;
        if (m_ctx) {            // image size changed: keep the trained weights and the update counts
            check(m_ctx, pink_hip_get_som(m_ctx, m_som_copy.data()));
            if (!m_factors.empty()) m_counts_base = update_counts();
            pink_hip_destroy(m_ctx);
            m_ctx = nullptr;
        }
        m_cfg.image_dim = image_dim;
        m_cfg.update_factors = m_factors.empty() ? nullptr : m_factors.data();
        pink_hip_ctx* ctx = nullptr;
        if (pink_hip_create(&ctx, &m_cfg) != PINK_HIP_OK) throw pink::exception(pink_hip_last_error(nullptr));
        m_ctx = ctx;
        check(m_ctx, pink_hip_set_som(m_ctx, m_som_copy.data()));
        return m_ctx;
    }

    pink_hip_ctx* get() const { return m_ctx; }

    /// How often each neuron was the best match, over every context this object has had.
    std::vector<uint32_t> update_counts() const
    {
        std::vector<uint32_t> counts(m_cfg.som_size, 0u);
        if (m_ctx) check(m_ctx, pink_hip_update_counts(m_ctx, counts.data()));
        for (size_t i = 0; i < m_counts_base.size(); ++i) counts[i] += m_counts_base[i];
        return counts;
    }
    std::vector<float> const& initial_som() const { return m_som_copy; }

private:
    pink_hip_ctx* m_ctx = nullptr;
    pink_hip_config m_cfg{};
    std::vector<float> m_factors;
    std::vector<float> m_som_copy;
    std::vector<uint32_t> m_counts_base;
};

} // namespace hip_detail

/// GPU version of training (reference: Trainer.h:201-335)
template <typename SOMLayout, typename DataLayout, typename T>
class Trainer<SOMLayout, DataLayout, T, true> : public TrainerBase
{
    static_assert(std::is_same<T, float>::value, "the device path trains float SOMs");
    typedef SOM<SOMLayout, DataLayout, T> SOMType;
    typedef Data<SOMLayout, uint32_t> UpdateInfoType;

public:

    Trainer(Trainer const&) = delete;

    Trainer(SOMType& som, std::function<float(float)> const& distribution_function, int verbosity,
        uint32_t number_of_rotations, bool use_flip, float max_update_distance,
        Interpolation interpolation, uint32_t euclidean_distance_dim,
        EuclideanDistanceShape const& euclidean_distance_shape = EuclideanDistanceShape::QUADRATIC,
        [[maybe_unused]] uint32_t block_size = 256, DataType euclidean_distance_type = DataType::FLOAT)
     : m_som(som),
       m_verbosity(verbosity)
    {
        if (number_of_rotations == 0 or (number_of_rotations != 1 and number_of_rotations % 4 != 0))
            throw pink::exception("Number of rotations must be 1 or larger then 1 and divisible by 4");

        // The N x N neighbourhood matrix of TrainerCommon (Trainer.h:69-76)
        auto const som_layout = som.get_som_layout();
        uint32_t const som_size = static_cast<uint32_t>(som_layout.size());
        std::vector<float> factors(static_cast<size_t>(som_size) * som_size, 0.0f);
        for (uint32_t i = 0; i < som_size; ++i) {
            for (uint32_t j = 0; j < som_size; ++j) {
                float distance = som_layout.get_distance(i, j);
                if (max_update_distance <= 0 or distance < max_update_distance)
                    factors[static_cast<size_t>(i) * som_size + j] = distribution_function(distance);
            }
        }
        m_device.create(som, &factors, number_of_rotations, use_flip, interpolation, euclidean_distance_dim,
            euclidean_distance_shape, euclidean_distance_type);
    }

    /// Training the SOM by a single data point
    void operator () (Data<DataLayout, T> const& data)
    {
        uint32_t channels = 0, image_dim = 0;
        hip_detail::image_geometry(data.get_layout(), channels, image_dim);
        auto* ctx = m_device.for_image(channels, image_dim);
        // nothing is handed back: the library copies the image and returns; images are trained in order, a
        // launch group at a time (when the group is full, or when update_som / get_update_info follows)
        hip_detail::check(ctx, pink_hip_train(ctx, data.get_data_pointer(), 1, nullptr));
    }

    /// Training by several data points stored back to back, in order
    void operator () (T const* images, uint32_t number_of_images, uint32_t channels, uint32_t image_dim)
    {
        auto* ctx = m_device.for_image(channels, image_dim);
        hip_detail::check(ctx, pink_hip_train(ctx, images, number_of_images, nullptr));
    }

    void update_som()
    {
        if (auto* ctx = m_device.get()) hip_detail::check(ctx, pink_hip_get_som(ctx, m_som.get_data_pointer()));
    }

    /// m_update_info of the reference (Trainer.h:79,94-95): counted on the device, read back here
    auto get_update_info() const
    {
        UpdateInfoType info(m_som.get_som_layout(), 0u);
        auto const counts = m_device.update_counts();
        for (size_t i = 0; i < counts.size(); ++i) info[static_cast<uint32_t>(i)] = counts[i];
        return info;
    }

private:

    /// A reference to the SOM will be trained
    SOMType& m_som;
    int m_verbosity;
    hip_detail::Context m_device;
};

/// GPU version of mapping (reference: Mapper.h:129-230)
template <typename SOMLayout, typename DataLayout, typename T>
class Mapper<SOMLayout, DataLayout, T, true> : public MapperBase
{
    static_assert(std::is_same<T, float>::value, "the device path maps float SOMs");

public:

    Mapper(SOM<SOMLayout, DataLayout, T> const& som, int verbosity, uint32_t number_of_rotations, bool use_flip,
        Interpolation interpolation, uint32_t euclidean_distance_dim,
        EuclideanDistanceShape const& euclidean_distance_shape = EuclideanDistanceShape::QUADRATIC,
        [[maybe_unused]] uint32_t block_size = 256, DataType euclidean_distance_type = DataType::FLOAT)
     : m_som_size(som.get_number_of_neurons()),
       m_verbosity(verbosity)
    {
        m_device.create(som, nullptr, number_of_rotations, use_flip, interpolation, euclidean_distance_dim,
            euclidean_distance_shape, euclidean_distance_type);
    }

    /// Mapping of a single data point: (sqrt of the minimal distance, best rotation) per neuron
    auto operator () (Data<DataLayout, T> const& data)
    {
        uint32_t channels = 0, image_dim = 0;
        hip_detail::image_geometry(data.get_layout(), channels, image_dim);
        auto* ctx = m_device.for_image(channels, image_dim);
        std::vector<float> euclidean_distance_matrix(m_som_size);
        std::vector<uint32_t> best_rotation_matrix(m_som_size);
        hip_detail::check(ctx, pink_hip_map(ctx, data.get_data_pointer(), 1, euclidean_distance_matrix.data(),
            best_rotation_matrix.data()));
        return std::make_tuple(euclidean_distance_matrix, best_rotation_matrix);
    }

    /// Mapping of several data points stored back to back
    auto operator () (T const* images, uint32_t number_of_images, uint32_t channels, uint32_t image_dim)
    {
        auto* ctx = m_device.for_image(channels, image_dim);
        std::vector<float> euclidean_distance_matrix(static_cast<size_t>(number_of_images) * m_som_size);
        std::vector<uint32_t> best_rotation_matrix(static_cast<size_t>(number_of_images) * m_som_size);
        hip_detail::check(ctx, pink_hip_map(ctx, images, number_of_images, euclidean_distance_matrix.data(),
            best_rotation_matrix.data()));
        return std::make_tuple(euclidean_distance_matrix, best_rotation_matrix);
    }

private:

    uint32_t m_som_size;
    int m_verbosity;
    hip_detail::Context m_device;
};

} // namespace pink
