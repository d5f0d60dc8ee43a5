// Mirrors arm_compute/function_info/FullyConnectedLayerInfo.h:37-72 of the reference.
#ifndef ACL_MI355_FUNCTION_INFO_FULLYCONNECTEDLAYERINFO_H
#define ACL_MI355_FUNCTION_INFO_FULLYCONNECTEDLAYERINFO_H

#include "arm_compute/core/Types.h"

namespace arm_compute
{
/** Fully connected layer info */
struct FullyConnectedLayerInfo
{
    ActivationLayerInfo activation_info{};                   /**< Fused activation applied after the matrix multiplication */
    DataLayout          weights_trained_layout{DataLayout::NCHW}; /**< Layout the weights were trained with */
    bool                transpose_weights{true};             /**< The weights arrive as [num_outputs rows][num_inputs] */
    bool                are_weights_reshaped{false};         /**< The weights are already transposed */
    bool                retain_internal_weights{false};      /**< Keep the packed weights of an earlier configure() */
    bool                enable_fast_math{false};
    bool                fp_mixed_precision{false};

    FullyConnectedLayerInfo &set_weights_trained_layout(DataLayout layout)
    {
        weights_trained_layout = layout;
        return *this;
    }
    FullyConnectedLayerInfo &set_transpose_weights(bool should_transpose_weights)
    {
        transpose_weights = should_transpose_weights;
        return *this;
    }
};
} // namespace arm_compute
#endif
