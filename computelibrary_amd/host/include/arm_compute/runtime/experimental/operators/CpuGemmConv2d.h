// Mirrors arm_compute/runtime/experimental/operators/CpuGemmConv2d.h:46-153 of the reference.
#ifndef ACL_MI355_RUNTIME_EXPERIMENTAL_OPERATORS_CPUGEMMCONV2D_H
#define ACL_MI355_RUNTIME_EXPERIMENTAL_OPERATORS_CPUGEMMCONV2D_H

#include "arm_compute/core/ITensorInfo.h"
#include "arm_compute/core/ITensorPack.h"
#include "arm_compute/core/Types.h"
#include "arm_compute/function_info/GEMMInfo.h"
#include "arm_compute/runtime/NEON/INEOperator.h"

#include <memory>

namespace arm_compute
{
namespace experimental
{
namespace op
{
/** Stateless quantized convolution: configured on tensor *infos*, run on an ITensorPack
 * (ACL_SRC_0 = src, ACL_SRC_1 = weights, ACL_SRC_2 = biases, ACL_DST = dst). The same validate() rules, arithmetic and
 * kernels as NEGEMMConvolutionLayer. Tensors whose memory was imported from device pointers are used in place. The packed
 * weights and every intermediate live in device memory owned by the operator: workspace() asks the caller for nothing.
 */
class CpuGemmConv2d : public INEOperator
{
public:
    CpuGemmConv2d();
    CpuGemmConv2d(const CpuGemmConv2d &)            = delete;
    CpuGemmConv2d(CpuGemmConv2d &&)                 = delete;
    CpuGemmConv2d &operator=(const CpuGemmConv2d &) = delete;
    CpuGemmConv2d &operator=(CpuGemmConv2d &&)      = delete;
    ~CpuGemmConv2d();

    void configure(const ITensorInfo *src, const ITensorInfo *weights, const ITensorInfo *biases, ITensorInfo *dst,
                   const PadStrideInfo &conv_info, const WeightsInfo &weights_info = WeightsInfo(),
                   const Size2D &dilation = Size2D(1U, 1U), const ActivationLayerInfo &act_info = ActivationLayerInfo(),
                   bool enable_fast_math = false, unsigned int num_groups = 1);
    static Status validate(const ITensorInfo *src, const ITensorInfo *weights, const ITensorInfo *biases,
                           const ITensorInfo *output, const PadStrideInfo &conv_info,
                           const WeightsInfo &weights_info = WeightsInfo(), const Size2D &dilation = Size2D(1U, 1U),
                           const ActivationLayerInfo &act_info = ActivationLayerInfo(), bool enable_fast_math = false,
                           unsigned int num_groups = 1);
    static Status has_opt_impl(arm_compute::WeightFormat &expected_weight_format, const ITensorInfo *src,
                               const ITensorInfo *weights, const ITensorInfo *biases, const ITensorInfo *output,
                               const PadStrideInfo &conv_info, const WeightsInfo &weights_info = WeightsInfo(),
                               const Size2D &dilation = Size2D(1U, 1U),
                               const ActivationLayerInfo &act_info = ActivationLayerInfo(), bool enable_fast_math = false);
    /** Re-derive the output stage from the quantization infos the tensors of the pack carry now
     * (src/cpu/operators/CpuGemmConv2d.cpp:1075-1109 of the reference) without re-packing the weights. */
    void update_quantization_parameters(ITensorPack &tensors);

    void               run(ITensorPack &tensors) override;
    void               prepare(ITensorPack &tensors) override;
    MemoryRequirements workspace() const override;

private:
    struct Impl;
    std::unique_ptr<Impl> _impl;
};
} // namespace op
} // namespace experimental
} // namespace arm_compute
#endif
