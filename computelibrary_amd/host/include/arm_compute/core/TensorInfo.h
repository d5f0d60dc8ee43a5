// Concrete tensor metadata. Mirrors arm_compute/core/TensorInfo.h of the reference: dense strides derived from shape and
// padding, x-fastest, padding added by extend_padding() changes strides and the first-element offset.
#ifndef ACL_MI355_CORE_TENSORINFO_H
#define ACL_MI355_CORE_TENSORINFO_H

#include "arm_compute/core/ITensorInfo.h"

namespace arm_compute
{
class TensorInfo final : public ITensorInfo
{
public:
    TensorInfo();
    TensorInfo(const ITensorInfo &info);
    TensorInfo(const TensorInfo &)            = default;
    TensorInfo &operator=(const TensorInfo &) = default;
    TensorInfo(const TensorShape &tensor_shape, size_t num_channels, DataType data_type);
    TensorInfo(const TensorShape &tensor_shape, size_t num_channels, DataType data_type, DataLayout data_layout);
    TensorInfo(const TensorShape &tensor_shape, size_t num_channels, DataType data_type,
               QuantizationInfo quantization_info);

    void init(const TensorShape &tensor_shape, size_t num_channels, DataType data_type);
    void init(const TensorShape &tensor_shape, size_t num_channels, DataType data_type, const Strides &strides_in_bytes,
              size_t offset_first_element_in_bytes, size_t total_size_in_bytes);

    std::unique_ptr<ITensorInfo> clone() const override;
    ITensorInfo &set_data_type(DataType data_type) override;
    ITensorInfo &set_num_channels(int num_channels) override;
    ITensorInfo &set_tensor_shape(const TensorShape &shape) override;
    ITensorInfo &set_quantization_info(const QuantizationInfo &quantization_info) override;
    ITensorInfo &set_data_layout(const DataLayout &data_layout) override;
    ITensorInfo &set_are_values_constant(bool are_values_constant) override;
    ITensorInfo &set_is_resizable(bool is_resizable) override;
    ITensorInfo &reset_padding() override;
    bool         auto_padding() override;
    bool         extend_padding(const PaddingSize &padding) override;
    size_t       dimension(size_t index) const override { return _tensor_shape[index]; }
    size_t       dimension(DataLayoutDimension dimension) const override
    {
        return _tensor_shape[get_data_layout_dimension_index(_data_layout, dimension)];
    }
    const Strides &strides_in_bytes() const override { return _strides_in_bytes; }
    size_t         offset_first_element_in_bytes() const override { return _offset_first_element_in_bytes; }
    int32_t        offset_element_in_bytes(const Coordinates &pos) const override;
    size_t         element_size() const override { return data_size_from_type(_data_type) * _num_channels; }
    size_t         num_dimensions() const override { return _tensor_shape.num_dimensions(); }
    size_t         num_channels() const override { return _num_channels; }
    const TensorShape &tensor_shape() const override { return _tensor_shape; }
    DataType       data_type() const override { return _data_type; }
    size_t         total_size() const override { return _total_size; }
    PaddingSize    padding() const override { return _padding; }
    bool           has_padding() const override { return !_padding.empty(); }
    bool           is_resizable() const override { return _is_resizable; }
    bool           is_dynamic() const override { return false; }
    bool           are_values_constant() const override { return _are_values_constant; }
    QuantizationInfo quantization_info() const override { return _quantization_info; }
    DataLayout     data_layout() const override { return _data_layout; }

private:
    void recompute_layout();

    size_t           _total_size;
    size_t           _offset_first_element_in_bytes;
    Strides          _strides_in_bytes;
    size_t           _num_channels;
    TensorShape      _tensor_shape;
    DataType         _data_type;
    bool             _is_resizable;
    PaddingSize      _padding;
    QuantizationInfo _quantization_info;
    DataLayout       _data_layout;
    bool             _are_values_constant;
};
} // namespace arm_compute
#endif
