// Tensor metadata interface. Mirrors the members of arm_compute/core/ITensorInfo.h:81-334 of the reference that this
// path reads: shape, strides and first-element offset in bytes, data type, quantization, layout, constness, padding.
#ifndef ACL_MI355_CORE_ITENSORINFO_H
#define ACL_MI355_CORE_ITENSORINFO_H

#include "arm_compute/core/Types.h"

#include <memory>

namespace arm_compute
{
class ITensorInfo
{
public:
    virtual ~ITensorInfo()                                                              = default;
    virtual std::unique_ptr<ITensorInfo> clone() const                                  = 0;
    virtual ITensorInfo &set_data_type(DataType data_type)                              = 0;
    virtual ITensorInfo &set_num_channels(int num_channels)                             = 0;
    virtual ITensorInfo &set_tensor_shape(const TensorShape &shape)                     = 0;
    virtual ITensorInfo &set_quantization_info(const QuantizationInfo &quantization_info) = 0;
    virtual ITensorInfo &set_data_layout(const DataLayout &data_layout)                 = 0;
    virtual ITensorInfo &set_are_values_constant(bool are_values_constant)              = 0;
    virtual ITensorInfo &set_is_resizable(bool is_resizable)                            = 0;
    virtual ITensorInfo &reset_padding()                                                = 0;
    virtual bool         auto_padding()                                                 = 0;
    virtual bool         extend_padding(const PaddingSize &padding)                     = 0;
    virtual size_t       dimension(size_t index) const                                  = 0;
    virtual size_t       dimension(DataLayoutDimension dimension) const                 = 0;
    virtual const Strides &strides_in_bytes() const                                     = 0;
    virtual size_t       offset_first_element_in_bytes() const                          = 0;
    virtual int32_t      offset_element_in_bytes(const Coordinates &pos) const          = 0;
    virtual size_t       element_size() const                                           = 0;
    virtual size_t       num_dimensions() const                                         = 0;
    virtual size_t       num_channels() const                                           = 0;
    virtual const TensorShape &tensor_shape() const                                     = 0;
    virtual DataType     data_type() const                                              = 0;
    virtual size_t       total_size() const                                             = 0;
    virtual PaddingSize  padding() const                                                = 0;
    virtual bool         has_padding() const                                            = 0;
    virtual bool         is_resizable() const                                           = 0;
    virtual bool         is_dynamic() const                                             = 0;
    virtual bool         are_values_constant() const                                    = 0;
    virtual QuantizationInfo quantization_info() const                                  = 0;
    virtual DataLayout   data_layout() const                                            = 0;
};
} // namespace arm_compute
#endif
