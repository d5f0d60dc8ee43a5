// Mirrors arm_compute/runtime/NEON/functions/NEGEMMConvolutionLayer.h:50-231 of the reference for quantized tensors.
#ifndef ACL_MI355_RUNTIME_NEGEMMCONVOLUTIONLAYER_H
#define ACL_MI355_RUNTIME_NEGEMMCONVOLUTIONLAYER_H

#include "arm_compute/core/ITensor.h"
#include "arm_compute/function_info/GEMMInfo.h"
#include "arm_compute/runtime/IFunction.h"
#include "arm_compute/runtime/IMemoryManager.h"

#include <memory>

namespace arm_compute
{
/** Convolution lowered to a low-precision GEMM (im2col + weight flattening + GEMMLowp + fixed-point output stage).
 *
 * This build covers the quantized NHWC configurations: input / output QASYMM8 or QASYMM8_SIGNED, weights of the same type
 * or QSYMM8_PER_CHANNEL, S32 biases. The im2col matrix is never materialised where the channel count is a multiple of 16
 * and the weights are symmetric (implicit GEMM); otherwise it is built in device workspace first.
 */
class NEGEMMConvolutionLayer : public IFunction
{
public:
    NEGEMMConvolutionLayer(const std::shared_ptr<IMemoryManager> &memory_manager  = nullptr,
                           IWeightsManager                       *weights_manager = nullptr);
    NEGEMMConvolutionLayer(const NEGEMMConvolutionLayer &)            = delete;
    NEGEMMConvolutionLayer(NEGEMMConvolutionLayer &&)                 = default;
    NEGEMMConvolutionLayer &operator=(const NEGEMMConvolutionLayer &) = delete;
    NEGEMMConvolutionLayer &operator=(NEGEMMConvolutionLayer &&)      = default;
    ~NEGEMMConvolutionLayer();

    void configure(const ITensor *input, const ITensor *weights, const ITensor *biases, ITensor *output,
                   const PadStrideInfo &conv_info, const WeightsInfo &weights_info = WeightsInfo(),
                   const Size2D &dilation = Size2D(1U, 1U), const ActivationLayerInfo &act_info = ActivationLayerInfo(),
                   bool enable_fast_math = false, unsigned int num_groups = 1);
    static Status validate(const ITensorInfo *input, const ITensorInfo *weights, const ITensorInfo *biases,
                           const ITensorInfo *output, const PadStrideInfo &conv_info,
                           const WeightsInfo &weights_info = WeightsInfo(), const Size2D &dilation = Size2D(1U, 1U),
                           const ActivationLayerInfo &act_info = ActivationLayerInfo(), bool enable_fast_math = false,
                           unsigned int num_groups = 1);
    static Status has_opt_impl(WeightFormat &expected_weight_format, const ITensorInfo *src, const ITensorInfo *weights,
                               const ITensorInfo *biases, const ITensorInfo *dst, const PadStrideInfo &conv_info,
                               const WeightsInfo &weights_info = WeightsInfo(), const Size2D &dilation = Size2D(1U, 1U),
                               const ActivationLayerInfo &act_info = ActivationLayerInfo(),
                               bool enable_fast_math = false);
    void update_quantization_parameters();

    void run() override;
    void prepare() override;

    const char *kernel_name() const;

private:
    struct Impl;
    std::unique_ptr<Impl> _impl;
};
} // namespace arm_compute
#endif
