// Enumerations and small value types of the arm_compute surface that the quantized-GEMM path touches.
// Mirrors the corresponding declarations of arm_compute/core/Types.h, core/CoreTypes.h, core/Size2D.h and
// function_info/ActivationLayerInfo.h of the reference (same names, same default values).
#ifndef ACL_MI355_CORE_TYPES_H
#define ACL_MI355_CORE_TYPES_H

#include "arm_compute/core/Coordinates.h"
#include "arm_compute/core/Error.h"
#include "arm_compute/core/QuantizationInfo.h"
#include "arm_compute/core/Strides.h"
#include "arm_compute/core/TensorShape.h"

#include <cstddef>
#include <cstdint>
#include <utility>

namespace arm_compute
{
enum class DataType
{
    UNKNOWN,
    U8,
    S8,
    QSYMM8,
    QASYMM8,
    QASYMM8_SIGNED,
    QSYMM8_PER_CHANNEL,
    U16,
    S16,
    QSYMM16,
    QASYMM16,
    U32,
    S32,
    U64,
    S64,
    BFLOAT16,
    F16,
    F32,
    F64,
    SIZET
};

enum class DataLayout
{
    UNKNOWN,
    NCHW,
    NHWC,
    NCDHW,
    NDHWC
};

enum class DataLayoutDimension
{
    CHANNEL,
    HEIGHT,
    WIDTH,
    DEPTH,
    BATCHES
};

enum class DimensionRoundingType
{
    FLOOR,
    CEIL
};

inline size_t data_size_from_type(DataType dt)
{
    switch (dt)
    {
        case DataType::U8:
        case DataType::S8:
        case DataType::QSYMM8:
        case DataType::QASYMM8:
        case DataType::QASYMM8_SIGNED:
        case DataType::QSYMM8_PER_CHANNEL:
            return 1;
        case DataType::U16:
        case DataType::S16:
        case DataType::QSYMM16:
        case DataType::QASYMM16:
        case DataType::BFLOAT16:
        case DataType::F16:
            return 2;
        case DataType::U32:
        case DataType::S32:
        case DataType::F32:
            return 4;
        case DataType::U64:
        case DataType::S64:
        case DataType::F64:
        case DataType::SIZET:
            return 8;
        default:
            return 0;
    }
}
inline bool is_data_type_quantized(DataType dt)
{
    switch (dt)
    {
        case DataType::QSYMM8:
        case DataType::QASYMM8:
        case DataType::QASYMM8_SIGNED:
        case DataType::QSYMM8_PER_CHANNEL:
        case DataType::QSYMM16:
        case DataType::QASYMM16:
            return true;
        default:
            return false;
    }
}
inline bool is_data_type_quantized_asymmetric(DataType dt)
{
    return dt == DataType::QASYMM8 || dt == DataType::QASYMM8_SIGNED || dt == DataType::QASYMM16;
}
inline bool is_data_type_quantized_asymmetric_signed(DataType dt)
{
    return dt == DataType::QASYMM8_SIGNED;
}
inline bool is_data_type_quantized_per_channel(DataType dt)
{
    return dt == DataType::QSYMM8_PER_CHANNEL;
}
// lowest / highest representable value of the 8-bit quantized types and S32 (get_min_max of the reference, as int32)
inline std::pair<int32_t, int32_t> get_min_max(DataType dt)
{
    switch (dt)
    {
        case DataType::U8:
        case DataType::QASYMM8:
            return {0, 255};
        case DataType::S8:
        case DataType::QSYMM8:
        case DataType::QASYMM8_SIGNED:
        case DataType::QSYMM8_PER_CHANNEL:
            return {-128, 127};
        case DataType::S16:
        case DataType::QSYMM16:
            return {-32768, 32767};
        default:
            return {std::numeric_limits<int32_t>::lowest(), std::numeric_limits<int32_t>::max()};
    }
}

// index of a logical dimension inside a tensor shape for a given layout (x-fastest shapes: NCHW = [W,H,C,N], NHWC = [C,W,H,N])
inline size_t get_data_layout_dimension_index(DataLayout layout, DataLayoutDimension dim)
{
    if (layout == DataLayout::NHWC)
    {
        switch (dim)
        {
            case DataLayoutDimension::CHANNEL:
                return 0;
            case DataLayoutDimension::WIDTH:
                return 1;
            case DataLayoutDimension::HEIGHT:
                return 2;
            default:
                return 3;
        }
    }
    switch (dim)
    {
        case DataLayoutDimension::WIDTH:
            return 0;
        case DataLayoutDimension::HEIGHT:
            return 1;
        case DataLayoutDimension::CHANNEL:
            return 2;
        default:
            return 3;
    }
}

struct BorderSize
{
    constexpr BorderSize() noexcept : top{0}, right{0}, bottom{0}, left{0} {}
    explicit constexpr BorderSize(unsigned int size) noexcept : top{size}, right{size}, bottom{size}, left{size} {}
    constexpr BorderSize(unsigned int top_bottom, unsigned int left_right)
        : top{top_bottom}, right{left_right}, bottom{top_bottom}, left{left_right}
    {
    }
    constexpr BorderSize(unsigned int top, unsigned int right, unsigned int bottom, unsigned int left)
        : top{top}, right{right}, bottom{bottom}, left{left}
    {
    }
    constexpr bool empty() const { return top == 0 && right == 0 && bottom == 0 && left == 0; }
    unsigned int   top, right, bottom, left;
};
using PaddingSize = BorderSize;

class Size2D
{
public:
    Size2D() = default;
    Size2D(size_t w, size_t h) noexcept : width(w), height(h) {}
    size_t area() const { return width * height; }
    size_t x() const { return width; }
    size_t y() const { return height; }
    bool   operator==(const Size2D &o) const { return width == o.width && height == o.height; }
    bool   operator!=(const Size2D &o) const { return !(*this == o); }
    size_t width{0};
    size_t height{0};
};

class PadStrideInfo
{
public:
    PadStrideInfo(unsigned int stride_x = 1, unsigned int stride_y = 1, unsigned int pad_x = 0, unsigned int pad_y = 0,
                  DimensionRoundingType round = DimensionRoundingType::FLOOR)
        : _stride(std::make_pair(stride_x, stride_y)), _pad_left(pad_x), _pad_top(pad_y), _pad_right(pad_x),
          _pad_bottom(pad_y), _round_type(round)
    {
    }
    PadStrideInfo(unsigned int stride_x, unsigned int stride_y, unsigned int pad_left, unsigned int pad_right,
                  unsigned int pad_top, unsigned int pad_bottom, DimensionRoundingType round)
        : _stride(std::make_pair(stride_x, stride_y)), _pad_left(pad_left), _pad_top(pad_top), _pad_right(pad_right),
          _pad_bottom(pad_bottom), _round_type(round)
    {
    }
    std::pair<unsigned int, unsigned int> stride() const { return _stride; }
    bool padding_is_symmetric() const { return (_pad_left == _pad_right) && (_pad_top == _pad_bottom); }
    std::pair<unsigned int, unsigned int> pad() const { return std::make_pair(_pad_left, _pad_top); }
    unsigned int          pad_left() const { return _pad_left; }
    unsigned int          pad_right() const { return _pad_right; }
    unsigned int          pad_top() const { return _pad_top; }
    unsigned int          pad_bottom() const { return _pad_bottom; }
    DimensionRoundingType round() const { return _round_type; }
    bool has_padding() const { return (_pad_left != 0 || _pad_top != 0 || _pad_right != 0 || _pad_bottom != 0); }

private:
    std::pair<unsigned int, unsigned int> _stride;
    unsigned int                          _pad_left, _pad_top, _pad_right, _pad_bottom;
    DimensionRoundingType                 _round_type;
};

// output width / height of a convolution (src/core/Utils.cpp:288-332 of the reference)
std::pair<unsigned int, unsigned int> scaled_dimensions(int width, int height, int kernel_width, int kernel_height,
                                                        const PadStrideInfo &pad_stride_info,
                                                        const Size2D        &dilation = Size2D(1U, 1U));

class ActivationLayerInfo
{
public:
    enum class ActivationFunction
    {
        LOGISTIC,
        TANH,
        RELU,
        BOUNDED_RELU,
        LU_BOUNDED_RELU,
        LEAKY_RELU,
        SOFT_RELU,
        ELU,
        ABS,
        SQUARE,
        SQRT,
        LINEAR,
        IDENTITY,
        HARD_SWISH,
        SWISH,
        GELU
    };
    ActivationLayerInfo() = default;
    ActivationLayerInfo(ActivationFunction f, float a = 0.0f, float b = 0.0f) : _act(f), _a(a), _b(b), _enabled(true) {}
    ActivationFunction activation() const { return _act; }
    float a() const { return _a; }
    float b() const { return _b; }
    bool  enabled() const { return _enabled; }

private:
    ActivationFunction _act     = {ActivationFunction::IDENTITY};
    float              _a       = {};
    float              _b       = {};
    bool               _enabled = {false};
};

// (min, max) clamp that a fused RELU / BOUNDED_RELU / LU_BOUNDED_RELU turns into, in the output's quantized domain
// (src/core/Utils.cpp:442-462 of the reference)
std::pair<int32_t, int32_t> get_quantized_activation_min_max(const ActivationLayerInfo &act_info, DataType data_type,
                                                             UniformQuantizationInfo oq_info);

enum class WeightFormat
{
    UNSPECIFIED = 0x1,
    ANY         = 0x2
};

class WeightsInfo
{
public:
    WeightsInfo() = default;
    WeightsInfo(bool are_reshaped, unsigned int kernel_width, unsigned int kernel_height, unsigned int num_kernels,
                bool retain_internal_weights = false, WeightFormat weight_format = WeightFormat::UNSPECIFIED)
        : _are_reshaped(are_reshaped), _kernel_width(kernel_width), _kernel_height(kernel_height),
          _num_kernels(num_kernels), _retain_internal_weights(retain_internal_weights), _weight_format(weight_format)
    {
    }
    bool are_reshaped() const { return _are_reshaped; }
    unsigned int num_kernels() const { return _num_kernels; }
    std::pair<unsigned int, unsigned int> kernel_size() const { return std::make_pair(_kernel_width, _kernel_height); }
    bool         retain_internal_weights() const { return _retain_internal_weights; }
    WeightFormat weight_format() const { return _weight_format; }

private:
    bool         _are_reshaped{false};
    unsigned int _kernel_width{0}, _kernel_height{0}, _num_kernels{0};
    bool         _retain_internal_weights{false};
    WeightFormat _weight_format{WeightFormat::UNSPECIFIED};
};
} // namespace arm_compute
#endif
