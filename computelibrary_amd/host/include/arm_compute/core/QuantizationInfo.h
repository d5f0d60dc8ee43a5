// QuantizationInfo: per-tensor (scale, offset) or per-channel scales, plus the scalar quantize helpers the path uses.
// Mirrors arm_compute/core/QuantizationInfo.h:46-188,256-330 of the reference.
#ifndef ACL_MI355_CORE_QUANTIZATIONINFO_H
#define ACL_MI355_CORE_QUANTIZATIONINFO_H

#include <algorithm>
#include <cmath>
#include <cstdint>
#include <limits>
#include <vector>

namespace arm_compute
{
using qasymm8_signed_t = int8_t;
using qasymm8_t        = uint8_t;

struct UniformQuantizationInfo
{
    UniformQuantizationInfo() : scale(0.f), offset(0) {}
    UniformQuantizationInfo(float scale, int32_t offset) : scale(scale), offset(offset) {}
    bool empty() const { return scale == 0; }
    float   scale;
    int32_t offset;
};

class QuantizationInfo
{
public:
    QuantizationInfo() noexcept : _scale(), _offset() {}
    QuantizationInfo(float scale) : _scale(1, scale), _offset() {}
    QuantizationInfo(float scale, int offset, bool is_dynamic = false)
        : _scale(1, scale), _offset(1, offset), _is_dynamic(is_dynamic)
    {
    }
    QuantizationInfo(std::vector<float> scale) : _scale(std::move(scale)), _offset() {}
    QuantizationInfo(std::vector<float> scale, std::vector<int32_t> offset, bool is_dynamic = false)
        : _scale(std::move(scale)), _offset(std::move(offset)), _is_dynamic(is_dynamic)
    {
    }
    const std::vector<float>   &scale() const { return _scale; }
    const std::vector<int32_t> &offset() const { return _offset; }
    bool is_dynamic() const { return _is_dynamic; }
    bool empty() const { return _scale.empty() && _offset.empty(); }
    UniformQuantizationInfo uniform() const
    {
        UniformQuantizationInfo uqinfo;
        uqinfo.scale  = _scale.empty() ? 0 : _scale[0];
        uqinfo.offset = _offset.empty() ? 0 : _offset[0];
        return uqinfo;
    }

private:
    std::vector<float>   _scale;
    std::vector<int32_t> _offset;
    bool                 _is_dynamic = false;
};

inline bool operator==(const QuantizationInfo &lhs, const QuantizationInfo &rhs)
{
    return (lhs.scale() == rhs.scale()) && (lhs.offset() == rhs.offset());
}
inline bool operator!=(const QuantizationInfo &lhs, const QuantizationInfo &rhs)
{
    return !(lhs == rhs);
}

// lround(value / scale) + offset, clamped to the type (QuantizationInfo.h:268-273 of the reference)
inline uint8_t quantize_qasymm8(float value, const UniformQuantizationInfo &qinfo)
{
    const int quantized = static_cast<int>(std::lround(value / qinfo.scale)) + qinfo.offset;
    return static_cast<uint8_t>(std::max(0, std::min(255, quantized)));
}
inline int8_t quantize_qasymm8_signed(float value, const UniformQuantizationInfo &qinfo)
{
    const int quantized = static_cast<int>(std::lround(value / qinfo.scale)) + qinfo.offset;
    return static_cast<int8_t>(std::max(-128, std::min(127, quantized)));
}
inline float dequantize_qasymm8(uint8_t value, const UniformQuantizationInfo &qinfo)
{
    return (static_cast<int>(value) - qinfo.offset) * qinfo.scale;
}
inline float dequantize_qasymm8_signed(int8_t value, const UniformQuantizationInfo &qinfo)
{
    return (static_cast<int>(value) - qinfo.offset) * qinfo.scale;
}
} // namespace arm_compute
#endif
