// Dimensions / TensorShape / Strides / Coordinates: x-fastest index containers of up to 6 dimensions.
// Mirrors arm_compute/core/{Dimensions,TensorShape,Strides,Coordinates}.h of the reference (same member names, same
// "trailing ones are not counted" rule for num_dimensions()).
#ifndef ACL_MI355_CORE_DIMENSIONS_H
#define ACL_MI355_CORE_DIMENSIONS_H

#include "arm_compute/core/Error.h"

#include <algorithm>
#include <array>
#include <cstddef>
#include <cstdint>
#include <functional>
#include <numeric>

namespace arm_compute
{
constexpr size_t MAX_DIMS = 6;

template <typename T>
class Dimensions
{
public:
    static constexpr size_t num_max_dimensions = MAX_DIMS;

    template <typename... Ts>
    explicit Dimensions(Ts... dims) : _id{{static_cast<T>(dims)...}}, _num_dimensions{sizeof...(dims)}
    {
    }
    Dimensions(const Dimensions &)            = default;
    Dimensions &operator=(const Dimensions &) = default;

    void set(size_t dimension, T value, bool increase_dim_unit = true)
    {
        ARM_COMPUTE_ERROR_ON(dimension >= num_max_dimensions);
        _id[dimension] = value;
        if (increase_dim_unit || value != 1)
            _num_dimensions = std::max(_num_dimensions, dimension + 1);
    }
    T x() const { return _id[0]; }
    T y() const { return _id[1]; }
    T z() const { return _id[2]; }
    const T &operator[](size_t dimension) const
    {
        ARM_COMPUTE_ERROR_ON(dimension >= num_max_dimensions);
        return _id[dimension];
    }
    T &operator[](size_t dimension)
    {
        ARM_COMPUTE_ERROR_ON(dimension >= num_max_dimensions);
        return _id[dimension];
    }
    unsigned int num_dimensions() const { return static_cast<unsigned int>(_num_dimensions); }
    void         set_num_dimensions(size_t num_dimensions) { _num_dimensions = num_dimensions; }
    typename std::array<T, num_max_dimensions>::const_iterator begin() const { return _id.begin(); }
    typename std::array<T, num_max_dimensions>::const_iterator end() const { return _id.end(); }

protected:
    ~Dimensions() = default;
    std::array<T, num_max_dimensions> _id;
    size_t                            _num_dimensions{0};
};

template <typename T>
inline bool operator==(const Dimensions<T> &lhs, const Dimensions<T> &rhs)
{
    return (lhs.num_dimensions() == rhs.num_dimensions()) && std::equal(lhs.begin(), lhs.end(), rhs.begin());
}
template <typename T>
inline bool operator!=(const Dimensions<T> &lhs, const Dimensions<T> &rhs)
{
    return !(lhs == rhs);
}

class Strides : public Dimensions<uint32_t>
{
public:
    template <typename... Ts>
    constexpr Strides(Ts... strides) : Dimensions{strides...}
    {
    }
};

class Coordinates : public Dimensions<int>
{
public:
    template <typename... Ts>
    constexpr Coordinates(Ts... coords) : Dimensions{coords...}
    {
    }
};

class TensorShape : public Dimensions<size_t>
{
public:
    template <typename... Ts>
    TensorShape(Ts... dims) : Dimensions{dims...}
    {
        // unset dimensions are 1, and trailing ones do not count
        if (_num_dimensions > 0)
            std::fill(_id.begin() + _num_dimensions, _id.end(), 1);
        apply_dimension_correction();
    }
    TensorShape &set(size_t dimension, size_t value, bool apply_dim_correction = true, bool increase_dim_unit = true)
    {
        // a 0-d shape is first filled with ones so that total_size() stays meaningful
        if (_num_dimensions == 0)
            std::fill(_id.begin(), _id.end(), 1);
        Dimensions::set(dimension, value, increase_dim_unit);
        if (apply_dim_correction)
            apply_dimension_correction();
        return *this;
    }
    size_t total_size() const
    {
        return std::accumulate(_id.begin(), _id.end(), size_t(1), std::multiplies<size_t>());
    }
    size_t total_size_upper(size_t dimension) const
    {
        ARM_COMPUTE_ERROR_ON(dimension >= TensorShape::num_max_dimensions);
        return std::accumulate(_id.begin() + dimension, _id.end(), size_t(1), std::multiplies<size_t>());
    }
    size_t total_size_lower(size_t dimension) const
    {
        ARM_COMPUTE_ERROR_ON(dimension > TensorShape::num_max_dimensions);
        return std::accumulate(_id.begin(), _id.begin() + dimension, size_t(1), std::multiplies<size_t>());
    }

private:
    void apply_dimension_correction()
    {
        for (int i = static_cast<int>(_num_dimensions) - 1; i > 0; --i)
        {
            if (_id[i] == 1)
                --_num_dimensions;
            else
                break;
        }
    }
};
} // namespace arm_compute
#endif
