// Mirrors arm_compute/runtime/NEON/functions/NEFullyConnectedLayer.h:84-170 of the reference for quantized tensors.
#ifndef ACL_MI355_RUNTIME_NEFULLYCONNECTEDLAYER_H
#define ACL_MI355_RUNTIME_NEFULLYCONNECTEDLAYER_H

#include "arm_compute/core/ITensor.h"
#include "arm_compute/function_info/FullyConnectedLayerInfo.h"
#include "arm_compute/runtime/IFunction.h"
#include "arm_compute/runtime/IMemoryManager.h"

#include <memory>

namespace arm_compute
{
/** Fully connected layer on quantized tensors: dst[batch][num_outputs] = requantize(src_flat[batch][num_inputs] * W + bias).
 *
 * Follows CpuFullyConnected (src/cpu/operators/CpuFullyConnected.cpp:58-115, 160-190, 232-344 of the reference): the
 * zero points of input and weights are negated into the GEMM's added offsets, the output stage is QUANTIZE_DOWN_FIXEDPOINT
 * with multiplier/shift from (input.scale * weights.scale / output.scale) and bounds from the fused activation, an input
 * coming from a convolution is flattened (a no-op on contiguous memory), and weights trained in the other data layout
 * are re-ordered once at prepare(). The weight transpose of the reference is folded into the packing of B.
 *
 * This build covers src / weights / dst of the same type QASYMM8 or QASYMM8_SIGNED and S32 biases.
 */
class NEFullyConnectedLayer : public IFunction
{
public:
    NEFullyConnectedLayer(std::shared_ptr<IMemoryManager> memory_manager = nullptr, IWeightsManager *weights_manager = nullptr);
    NEFullyConnectedLayer(const NEFullyConnectedLayer &)            = delete;
    NEFullyConnectedLayer(NEFullyConnectedLayer &&)                 = default;
    NEFullyConnectedLayer &operator=(const NEFullyConnectedLayer &) = delete;
    NEFullyConnectedLayer &operator=(NEFullyConnectedLayer &&)      = default;
    ~NEFullyConnectedLayer();

    void configure(const ITensor *input, const ITensor *weights, const ITensor *biases, ITensor *output,
                   FullyConnectedLayerInfo fc_info = FullyConnectedLayerInfo(), const WeightsInfo &weights_info = WeightsInfo());
    static Status validate(const ITensorInfo *input, const ITensorInfo *weights, const ITensorInfo *biases,
                           const ITensorInfo *output, FullyConnectedLayerInfo fc_info = FullyConnectedLayerInfo(),
                           const WeightsInfo &weights_info = WeightsInfo());
    static Status has_opt_impl(WeightFormat &expected_weight_format, const ITensorInfo *input, const ITensorInfo *weights,
                               const ITensorInfo *biases, const ITensorInfo *output, const FullyConnectedLayerInfo &fc_info,
                               const WeightsInfo &weights_info);

    void run() override;
    void prepare() override;

    const char *kernel_name() const;

private:
    struct Impl;
    std::unique_ptr<Impl> _impl;
};
} // namespace arm_compute
#endif
