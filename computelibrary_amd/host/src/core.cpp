// Core types of the arm_compute surface kept by this build: TensorInfo layout, allocator, conv output size,
// activation -> clamp bounds, float scale -> fixed-point multiplier.
#include "arm_compute/core/TensorInfo.h"
#include "arm_compute/core/utils/quantization/AsymmHelpers.h"
#include "arm_compute/runtime/TensorAllocator.h"

#include <cmath>
#include <cstdlib>
#include <cstring>

namespace arm_compute
{
// ---------------------------------------------------------------------------------------------------------------------
// TensorInfo: strides in bytes, x fastest; padding (left/right on x, top/bottom on y) enlarges strides and moves the
// first element, like arm_compute/core/TensorInfo.cpp:230-330 of the reference
// ---------------------------------------------------------------------------------------------------------------------
TensorInfo::TensorInfo()
    : _total_size(0), _offset_first_element_in_bytes(0), _strides_in_bytes(), _num_channels(0), _tensor_shape(),
      _data_type(DataType::UNKNOWN), _is_resizable(true), _padding(0), _quantization_info(),
      _data_layout(DataLayout::NCHW), _are_values_constant(true)
{
}

TensorInfo::TensorInfo(const ITensorInfo &info) : TensorInfo()
{
    _total_size                    = info.total_size();
    _offset_first_element_in_bytes = info.offset_first_element_in_bytes();
    _strides_in_bytes              = info.strides_in_bytes();
    _num_channels                  = info.num_channels();
    _tensor_shape                  = info.tensor_shape();
    _data_type                     = info.data_type();
    _is_resizable                  = info.is_resizable();
    _padding                       = info.padding();
    _quantization_info             = info.quantization_info();
    _data_layout                   = info.data_layout();
    _are_values_constant           = info.are_values_constant();
}

TensorInfo::TensorInfo(const TensorShape &tensor_shape, size_t num_channels, DataType data_type) : TensorInfo()
{
    init(tensor_shape, num_channels, data_type);
}
TensorInfo::TensorInfo(const TensorShape &tensor_shape, size_t num_channels, DataType data_type, DataLayout data_layout)
    : TensorInfo()
{
    init(tensor_shape, num_channels, data_type);
    _data_layout = data_layout;
}
TensorInfo::TensorInfo(const TensorShape &tensor_shape, size_t num_channels, DataType data_type,
                       QuantizationInfo quantization_info)
    : TensorInfo()
{
    init(tensor_shape, num_channels, data_type);
    _quantization_info = std::move(quantization_info);
}

void TensorInfo::init(const TensorShape &tensor_shape, size_t num_channels, DataType data_type)
{
    _data_type    = data_type;
    _num_channels = num_channels;
    _tensor_shape = tensor_shape;
    _padding      = PaddingSize(0);
    recompute_layout();
}

void TensorInfo::init(const TensorShape &tensor_shape, size_t num_channels, DataType data_type,
                      const Strides &strides_in_bytes, size_t offset_first_element_in_bytes, size_t total_size_in_bytes)
{
    _data_type                     = data_type;
    _num_channels                  = num_channels;
    _tensor_shape                  = tensor_shape;
    _strides_in_bytes              = strides_in_bytes;
    _offset_first_element_in_bytes = offset_first_element_in_bytes;
    _total_size                    = total_size_in_bytes;
}

void TensorInfo::recompute_layout()
{
    const size_t esz     = element_size();
    const size_t stride_x = esz;
    const size_t stride_y = (_tensor_shape[0] + _padding.left + _padding.right) * stride_x;
    Strides      strides(static_cast<uint32_t>(stride_x), static_cast<uint32_t>(stride_y));
    size_t       total = _tensor_shape.num_dimensions() == 0 ? 0 : stride_y;
    if (_tensor_shape.num_dimensions() >= 2)
        total = (_tensor_shape[1] + _padding.top + _padding.bottom) * stride_y;
    for (size_t i = 2; i < MAX_DIMS; ++i)
    {
        strides.set(i, static_cast<uint32_t>(total));
        if (i < _tensor_shape.num_dimensions())
            total *= _tensor_shape[i];
    }
    strides.set_num_dimensions(std::max<size_t>(_tensor_shape.num_dimensions(), 2));
    _strides_in_bytes              = strides;
    _offset_first_element_in_bytes = _padding.left * stride_x + _padding.top * stride_y;
    _total_size                    = total;
}

std::unique_ptr<ITensorInfo> TensorInfo::clone() const
{
    return std::make_unique<TensorInfo>(*this);
}
ITensorInfo &TensorInfo::set_data_type(DataType data_type)
{
    _data_type = data_type;
    recompute_layout();
    return *this;
}
ITensorInfo &TensorInfo::set_num_channels(int num_channels)
{
    _num_channels = num_channels;
    recompute_layout();
    return *this;
}
ITensorInfo &TensorInfo::set_tensor_shape(const TensorShape &shape)
{
    _tensor_shape = shape;
    recompute_layout();
    return *this;
}
ITensorInfo &TensorInfo::set_quantization_info(const QuantizationInfo &quantization_info)
{
    _quantization_info = quantization_info;
    return *this;
}
ITensorInfo &TensorInfo::set_data_layout(const DataLayout &data_layout)
{
    _data_layout = data_layout;
    return *this;
}
ITensorInfo &TensorInfo::set_are_values_constant(bool are_values_constant)
{
    _are_values_constant = are_values_constant;
    return *this;
}
ITensorInfo &TensorInfo::set_is_resizable(bool is_resizable)
{
    _is_resizable = is_resizable;
    return *this;
}
ITensorInfo &TensorInfo::reset_padding()
{
    _padding = PaddingSize(0);
    recompute_layout();
    return *this;
}
bool TensorInfo::auto_padding()
{
    return extend_padding(PaddingSize(4));
}
bool TensorInfo::extend_padding(const PaddingSize &padding)
{
    ARM_COMPUTE_ERROR_ON_MSG(!_is_resizable, "padding of a tensor that already owns memory cannot change");
    bool updated = false;
    if (padding.top > _padding.top)
        _padding.top = padding.top, updated = true;
    if (padding.right > _padding.right)
        _padding.right = padding.right, updated = true;
    if (padding.bottom > _padding.bottom)
        _padding.bottom = padding.bottom, updated = true;
    if (padding.left > _padding.left)
        _padding.left = padding.left, updated = true;
    recompute_layout();
    return updated;
}
int32_t TensorInfo::offset_element_in_bytes(const Coordinates &pos) const
{
    int32_t offset = static_cast<int32_t>(_offset_first_element_in_bytes);
    for (size_t i = 0; i < _tensor_shape.num_dimensions(); ++i)
        offset += pos[i] * static_cast<int32_t>(_strides_in_bytes[i]);
    return offset;
}

// ---------------------------------------------------------------------------------------------------------------------
// TensorAllocator
// ---------------------------------------------------------------------------------------------------------------------
TensorAllocator::TensorAllocator(TensorAllocator &&o) noexcept
    : _info(o._info), _ptr(o._ptr), _owned(o._owned), _alignment(o._alignment)
{
    o._ptr   = nullptr;
    o._owned = false;
}
TensorAllocator &TensorAllocator::operator=(TensorAllocator &&o) noexcept
{
    if (this != &o)
    {
        free();
        _info = o._info, _ptr = o._ptr, _owned = o._owned, _alignment = o._alignment;
        o._ptr = nullptr, o._owned = false;
    }
    return *this;
}
TensorAllocator::~TensorAllocator()
{
    if (_owned && _ptr)
        std::free(_ptr);
}
void TensorAllocator::init(const TensorInfo &input, size_t alignment)
{
    _info      = input;
    _alignment = alignment;
}
void TensorAllocator::allocate()
{
    ARM_COMPUTE_ERROR_ON_MSG(_ptr != nullptr, "tensor already has memory");
    const size_t align = std::max<size_t>(_alignment, 64);
    const size_t bytes = (std::max<size_t>(_info.total_size(), 1) + align - 1) / align * align;
    _ptr               = static_cast<uint8_t *>(std::aligned_alloc(align, bytes));
    ARM_COMPUTE_ERROR_ON_MSG(_ptr == nullptr, "out of host memory");
    std::memset(_ptr, 0, bytes);
    _owned = true;
    _info.set_is_resizable(false);
}
void TensorAllocator::free()
{
    if (_owned && _ptr)
        std::free(_ptr);
    _ptr   = nullptr;
    _owned = false;
    _info.set_is_resizable(true);
}
Status TensorAllocator::import_memory(void *memory)
{
    ARM_COMPUTE_RETURN_ERROR_ON(memory == nullptr);
    ARM_COMPUTE_RETURN_ERROR_ON_MSG(_ptr != nullptr && _owned, "tensor already owns memory");
    ARM_COMPUTE_RETURN_ERROR_ON(_alignment != 0 && (reinterpret_cast<uintptr_t>(memory) % _alignment) != 0);
    _ptr   = static_cast<uint8_t *>(memory);
    _owned = false;
    _info.set_is_resizable(false);
    return Status{};
}

// ---------------------------------------------------------------------------------------------------------------------
// Utils
// ---------------------------------------------------------------------------------------------------------------------
std::pair<unsigned int, unsigned int> scaled_dimensions(int width, int height, int kernel_width, int kernel_height,
                                                        const PadStrideInfo &info, const Size2D &dilation)
{
    const int   dx = static_cast<int>(dilation.x()), dy = static_cast<int>(dilation.y());
    const int   sx = static_cast<int>(info.stride().first), sy = static_cast<int>(info.stride().second);
    const float fw = static_cast<float>(width + static_cast<int>(info.pad_left() + info.pad_right()) -
                                        (dx * (kernel_width - 1) + 1)) / sx + 1;
    const float fh = static_cast<float>(height + static_cast<int>(info.pad_top() + info.pad_bottom()) -
                                        (dy * (kernel_height - 1) + 1)) / sy + 1;
    int w = 0, h = 0;
    if (info.round() == DimensionRoundingType::FLOOR)
        w = static_cast<int>(std::floor(fw)), h = static_cast<int>(std::floor(fh));
    else
        w = static_cast<int>(std::ceil(fw)), h = static_cast<int>(std::ceil(fh));
    return std::make_pair(static_cast<unsigned int>(std::max(1, w)), static_cast<unsigned int>(std::max(1, h)));
}

std::pair<int32_t, int32_t> get_quantized_activation_min_max(const ActivationLayerInfo &act_info, DataType data_type,
                                                             UniformQuantizationInfo oq_info)
{
    const bool is_signed = is_data_type_quantized_asymmetric_signed(data_type);
    const int  a_int = is_signed ? quantize_qasymm8_signed(act_info.a(), oq_info) : quantize_qasymm8(act_info.a(), oq_info);
    const int  b_int = is_signed ? quantize_qasymm8_signed(act_info.b(), oq_info) : quantize_qasymm8(act_info.b(), oq_info);
    const int32_t type_max = get_min_max(data_type).second;
    const int32_t lo = act_info.activation() != ActivationLayerInfo::ActivationFunction::LU_BOUNDED_RELU
                           ? std::min(oq_info.offset, type_max)
                           : b_int;
    const int32_t hi = act_info.activation() == ActivationLayerInfo::ActivationFunction::RELU ? type_max : a_int;
    return std::make_pair(lo, hi);
}

// ---------------------------------------------------------------------------------------------------------------------
// quantization helpers
// ---------------------------------------------------------------------------------------------------------------------
namespace quantization
{
namespace
{
// A real multiplier as mantissa * 2^(exponent - 31) with |mantissa| in [2^30, 2^31) (or 0): the form the fixed-point
// output stage multiplies by. frexp gives the fraction in [0.5, 1); a fraction so close to 1 that it rounds up to 2^31
// is renormalised to 2^30 with the exponent one higher.
struct Q31
{
    int64_t mantissa;
    int     exponent;
};

Q31 to_q31(float real)
{
    int          exponent = 0;
    const double fraction = std::frexp(static_cast<double>(real), &exponent);
    int64_t      mantissa = std::llround(std::ldexp(fraction, 31)); // halves away from zero, like std::round
    if (mantissa == (int64_t{1} << 31))
    {
        mantissa >>= 1;
        ++exponent;
    }
    return {mantissa, exponent};
}
} // namespace

// Semantics of src/core/utils/quantization/AsymmHelpers.cpp:43-115: (multiplier, shift) with shift > 0 a rounding right
// shift after the multiply and shift < 0 a left shift before it; real multipliers of 1 and above take the left-shift form.
Status calculate_quantized_multiplier(float multiplier, int32_t *quant_multiplier, int32_t *shift, bool ignore_epsilon)
{
    if (multiplier < 1.f)
        return calculate_quantized_multiplier_less_than_one(multiplier, quant_multiplier, shift, ignore_epsilon);
    int32_t      left   = 0;
    const Status status = calculate_quantized_multiplier_greater_than_one(multiplier, quant_multiplier, &left);
    if (shift != nullptr)
        *shift = -left;
    return status;
}

Status calculate_quantized_multiplier_less_than_one(float multiplier, int32_t *quant_multiplier, int32_t *right_shift,
                                                    bool ignore_epsilon)
{
    ARM_COMPUTE_RETURN_ERROR_ON(quant_multiplier == nullptr);
    ARM_COMPUTE_RETURN_ERROR_ON(right_shift == nullptr);
    // the reference tolerates values a hair outside [0, 1] unless told not to
    const float slack = ignore_epsilon ? 0.f : 0.00001f;
    ARM_COMPUTE_RETURN_ERROR_ON(multiplier < -slack);
    ARM_COMPUTE_RETURN_ERROR_ON(multiplier > 1.f + slack);
    Q31 q     = to_q31(multiplier);
    int right = -q.exponent;
    if (ignore_epsilon && right > 31)
        q.mantissa = 0, right = 0; // too small to leave a trace in 32 bits
    ARM_COMPUTE_RETURN_ERROR_ON(right < 0);
    *quant_multiplier = static_cast<int32_t>(q.mantissa);
    *right_shift      = right;
    return Status{};
}

Status calculate_quantized_multiplier_greater_than_one(float multiplier, int32_t *quantized_multiplier,
                                                       int32_t *left_shift)
{
    ARM_COMPUTE_RETURN_ERROR_ON(quantized_multiplier == nullptr);
    ARM_COMPUTE_RETURN_ERROR_ON(left_shift == nullptr);
    ARM_COMPUTE_RETURN_ERROR_ON(multiplier < 1.f);
    const Q31 q = to_q31(multiplier);
    ARM_COMPUTE_RETURN_ERROR_ON(q.exponent < 0);
    *quantized_multiplier = static_cast<int32_t>(q.mantissa);
    *left_shift           = q.exponent;
    return Status{};
}

// One (multiplier, shift) per weight scale from input_scale * weight_scale / output_scale
// (src/core/utils/quantization/AsymmHelpers.cpp:117-152). Per-channel vectors get 32 spare zero entries at the end:
// callers written against the reference size their buffers that way.
Status calculate_quantized_multipliers(const QuantizationInfo &iq_info, const QuantizationInfo &wq_info,
                                       const QuantizationInfo &oq_info, GEMMLowpOutputStageInfo &stage_info)
{
    ARM_COMPUTE_RETURN_ERROR_ON(iq_info.scale().empty());
    ARM_COMPUTE_RETURN_ERROR_ON(wq_info.scale().empty());
    ARM_COMPUTE_RETURN_ERROR_ON(oq_info.scale().empty());
    const std::vector<float> &w_scales = wq_info.scale();
    const size_t              channels = w_scales.size();
    const float               in_scale = iq_info.scale().front(), out_scale = oq_info.scale().front();
    std::vector<int32_t> &mults = stage_info.gemmlowp_multipliers, &shifts = stage_info.gemmlowp_shifts;
    mults.assign(channels == 1 ? 1 : channels + 32, 0);
    shifts.assign(mults.size(), 0);
    for (size_t ch = 0; ch < channels; ++ch)
        ARM_COMPUTE_RETURN_ON_ERROR(calculate_quantized_multiplier(in_scale * w_scales[ch] / out_scale, &mults[ch], &shifts[ch]));
    stage_info.gemmlowp_multiplier = mults.front();
    stage_info.gemmlowp_shift      = shifts.front();
    return Status{};
}

std::pair<int, int> get_min_max_values_from_quantized_data_type(DataType data_type)
{
    const auto mm = get_min_max(data_type);
    return std::make_pair(static_cast<int>(mm.first), static_cast<int>(mm.second));
}
} // namespace quantization
} // namespace arm_compute
