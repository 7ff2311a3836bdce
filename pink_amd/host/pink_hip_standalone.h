// pink_hip_standalone.h -- the few host types pink_hip_som.h needs when it is built outside
// the reference tree: layouts, Data, SOM, enums, exception and neighbourhood functors with
// the member names of the reference (src/SelfOrganizingMapLib/{CartesianLayout,
// HexagonalLayout,Data,SOM}.h, src/UtilitiesLib/{DataType,Interpolation,
// EuclideanDistanceShape,DistributionFunctor,pink_exception}.h).  Grid distances and
// functor values come from the library's own helpers so there is one implementation.
#pragma once

#include <array>
#include <cmath>
#include <cstdint>
#include <numeric>
#include <stdexcept>
#include <string>
#include <vector>

#include "pink_hip.h"

namespace pink {

struct exception : public std::runtime_error
{
    explicit exception(std::string const& msg) : std::runtime_error(msg) {}
};

enum class DataType { FLOAT, UINT16, UINT8 };
enum class Interpolation { NEAREST_NEIGHBOR, BILINEAR };
enum class EuclideanDistanceShape { QUADRATIC, CIRCULAR };

struct TrainerBase
{
    virtual ~TrainerBase() {}
    virtual void update_som() = 0;
};

struct MapperBase
{
    virtual ~MapperBase() {}
};

template <uint8_t dim>
struct CartesianLayout
{
    static const uint8_t dimensionality = dim;
    typedef uint32_t IndexType;
    typedef std::array<uint32_t, dim> DimensionType;

    bool operator == (CartesianLayout const& other) const { return m_dimension == other.m_dimension; }

    size_t size() const
    {
        size_t n = 1;
        for (auto d : m_dimension) n *= d;
        return n;
    }

    uint32_t get_dimension(IndexType i) const { return m_dimension[i]; }
    DimensionType get_dimension() const { return m_dimension; }
    uint32_t get_last_dimension() const { return m_dimension[dim - 1]; }

    /// Euclidean distance of two cells given as array indices
    float get_distance(IndexType i1, IndexType i2) const
    {
        float one = 0.0f;
        // row i1 of the step-function matrix with width d is 1 exactly where distance <= d;
        // the distance itself is simpler to form here, in the reference's float arithmetic.
        uint32_t p1[3] = {0, 0, 0}, p2[3] = {0, 0, 0};
        position(i1, p1);
        position(i2, p2);
        for (uint8_t k = 0; k < dim; ++k) {
            float diff = static_cast<float>(p1[k]) - static_cast<float>(p2[k]);
            one += static_cast<float>(static_cast<double>(diff) * static_cast<double>(diff));
        }
        return std::sqrt(one);
    }

    DimensionType m_dimension;

private:
    void position(IndexType i, uint32_t p[3]) const
    {
        if (dim == 1) { p[0] = i; }
        else if (dim == 2) { p[1] = i / m_dimension[1]; p[0] = i % m_dimension[1]; }
        else {
            uint32_t z = i / m_dimension[0] / m_dimension[1];
            p[2] = z;
            p[1] = (i - z * m_dimension[0] * m_dimension[1]) / m_dimension[1];
            p[0] = i % m_dimension[1];
        }
    }
};

struct HexagonalLayout
{
    static const uint8_t dimensionality = 2;
    typedef uint32_t IndexType;
    typedef std::array<uint32_t, 2> DimensionType;

    HexagonalLayout() : m_dimension({0, 0}) {}

    HexagonalLayout(DimensionType const& dimension) : m_dimension(dimension)
    {
        if (dimension[0] % 2 == 0) throw pink::exception("Only odd dimensions are allowed for hexagonal layout");
        if (dimension[0] != dimension[1]) throw pink::exception("dimension[0] must be identical to dimension[1]");
        uint32_t const radius = (dimension[0] - 1) / 2;
        m_row_offset.assign(dimension[0] + 1, 0);
        for (uint32_t r = 0; r < dimension[0]; ++r)
            m_row_offset[r + 1] = m_row_offset[r] + dimension[0] - (r > radius ? r - radius : radius - r);
    }

    bool operator == (HexagonalLayout const& other) const { return m_dimension == other.m_dimension; }

    size_t size() const { return m_row_offset.empty() ? 0 : m_row_offset.back(); }
    DimensionType get_dimension() const { return m_dimension; }

    /// Cube-metric distance of two cells given as array indices
    float get_distance(IndexType i1, IndexType i2) const
    {
        int32_t q1, r1, q2, r2;
        position(i1, q1, r1);
        position(i2, q2, r2);
        int32_t const dx = q1 - q2, dy = r1 - r2;
        if ((dx >= 0) == (dy >= 0)) return static_cast<float>(std::abs(dx + dy));
        return static_cast<float>(std::max(std::abs(dx), std::abs(dy)));
    }

    DimensionType m_dimension;

private:
    void position(IndexType i, int32_t& q, int32_t& r) const
    {
        uint32_t const radius = (m_dimension[0] - 1) / 2;
        uint32_t row = 0;
        while (row < m_dimension[0] and i >= m_row_offset[row + 1]) ++row;
        uint32_t col = i - m_row_offset[row];
        if (radius > row) col += radius - row;
        q = static_cast<int32_t>(col);
        r = static_cast<int32_t>(row);
    }

    std::vector<uint32_t> m_row_offset;
};

template <typename Layout, typename T>
class Data
{
public:
    typedef Layout LayoutType;

    Data() : m_layout() {}
    explicit Data(Layout const& layout) : m_layout(layout), m_data(layout.size()) {}
    Data(Layout const& layout, T value) : m_layout(layout), m_data(layout.size(), value) {}
    Data(Layout const& layout, std::vector<T> const& data) : m_layout(layout), m_data(data) {}

    bool operator == (Data const& other) const { return m_layout == other.m_layout and m_data == other.m_data; }
    size_t size() const { return m_data.size(); }
    T& operator [] (uint32_t i) { return m_data[i]; }
    T const& operator [] (uint32_t i) const { return m_data[i]; }
    T* get_data_pointer() { return m_data.data(); }
    T const* get_data_pointer() const { return m_data.data(); }
    std::vector<T> get_data() const { return m_data; }
    Layout get_layout() const { return m_layout; }
    typename Layout::DimensionType get_dimension() const { return m_layout.m_dimension; }

private:
    Layout m_layout;
    std::vector<T> m_data;
};

template <typename SOMLayout, typename NeuronLayout, typename T>
class SOM
{
public:
    typedef SOMLayout SOMLayoutType;
    typedef NeuronLayout NeuronLayoutType;

    SOM(SOMLayout const& som_layout, NeuronLayout const& neuron_layout, T value)
     : m_som_layout(som_layout), m_neuron_layout(neuron_layout), m_data(som_layout.size() * neuron_layout.size(), value) {}
    SOM(SOMLayout const& som_layout, NeuronLayout const& neuron_layout, std::vector<T> const& data)
     : m_som_layout(som_layout), m_neuron_layout(neuron_layout), m_data(data) {}

    size_t size() const { return m_data.size(); }
    T* get_data_pointer() { return m_data.data(); }
    T const* get_data_pointer() const { return m_data.data(); }
    uint32_t get_number_of_neurons() const { return static_cast<uint32_t>(m_som_layout.size()); }
    uint32_t get_neuron_size() const { return static_cast<uint32_t>(m_neuron_layout.size()); }
    SOMLayout get_som_layout() const { return m_som_layout; }
    NeuronLayout get_neuron_layout() const { return m_neuron_layout; }

private:
    SOMLayout m_som_layout;
    NeuronLayout m_neuron_layout;
    std::vector<T> m_data;
};

/// Neighbourhood functors (values: src/UtilitiesLib/DistributionFunctor.cpp:19-59)
struct StepFunctor
{
    explicit StepFunctor(float value) : m_value(value) {}
    float operator () (float distance) const { return distance <= m_value ? 1.0f : 0.0f; }
    float m_value;
};

struct GaussianFunctor
{
    GaussianFunctor(float sigma, float damping) : m_sigma(sigma), m_damping(damping) {}
    float operator () (float distance) const
    {
        return m_damping / (m_sigma * std::sqrt(2.0f * static_cast<float>(M_PI)))
             * std::exp(-0.5f * std::pow(distance / m_sigma, 2.0f));
    }
    float m_sigma, m_damping;
};

struct UnityGaussianFunctor
{
    UnityGaussianFunctor(float sigma, float damping) : m_sigma(sigma), m_damping(damping) {}
    float operator () (float distance) const { return m_damping * std::exp(-0.5f * std::pow(distance / m_sigma, 2.0f)); }
    float m_sigma, m_damping;
};

struct MexicanHatFunctor
{
    MexicanHatFunctor(float sigma, float damping) : m_sigma(sigma), m_damping(damping)
    {
        if (sigma <= 0.0f) throw std::runtime_error("MexicanHatFunctor: sigma <= 0 not defined.");
    }
    float operator () (float distance) const
    {
        float const d2 = distance * distance, s2 = m_sigma * m_sigma;
        return 2.0f * m_damping / (std::sqrt(3.0f * m_sigma) * std::pow(static_cast<float>(M_PI), 0.25f))
             * (1.0f - d2 / s2) * std::exp(-d2 / (2.0f * s2));
    }
    float m_sigma, m_damping;
};

} // namespace pink
