// Mirrors arm_compute/runtime/FunctionDescriptors.h:61-89 of the reference (the 2-D convolution descriptor).
#ifndef ACL_MI355_RUNTIME_FUNCTIONDESCRIPTORS_H
#define ACL_MI355_RUNTIME_FUNCTIONDESCRIPTORS_H

#include "arm_compute/core/Types.h"

namespace arm_compute
{
/** Descriptor used by the 2d Convolution function */
struct Conv2dInfo
{
    Conv2dInfo() = default;
    Conv2dInfo(const PadStrideInfo &conv_info, const Size2D &dilation, const ActivationLayerInfo &act_info,
               bool enable_fast_math, unsigned int num_groups, const WeightsInfo &weights_info = WeightsInfo(),
               bool use_fp32_acc = false)
        : conv_info(conv_info), dilation(dilation), act_info(act_info), enable_fast_math(enable_fast_math),
          num_groups(num_groups), weights_info(weights_info), use_fp32_acc(use_fp32_acc)
    {
    }

    PadStrideInfo       conv_info{};
    Size2D              dilation{1U, 1U};
    ActivationLayerInfo act_info{};
    bool                enable_fast_math{false};
    unsigned int        num_groups{1};
    WeightsInfo         weights_info{};
    bool                use_fp32_acc{false}; // relevant only for FP16
};
} // namespace arm_compute
#endif
