// Mirrors arm_compute/runtime/NEON/functions/NEGEMMConv2d.h:45-124 of the reference for quantized tensors.
#ifndef ACL_MI355_RUNTIME_NEGEMMCONV2D_H
#define ACL_MI355_RUNTIME_NEGEMMCONV2D_H

#include "arm_compute/core/ITensor.h"
#include "arm_compute/runtime/FunctionDescriptors.h"
#include "arm_compute/runtime/IFunction.h"
#include "arm_compute/runtime/IMemoryManager.h"
#include "arm_compute/runtime/NEON/functions/NEGEMMConvolutionLayer.h"

#include <memory>

namespace arm_compute
{
/** 2-D convolution handed straight to the GEMM back end ("direct" / indirect-buffer convolution of the reference,
 * src/cpu/operators/CpuGemmDirectConv2d.cpp:84-224): NHWC only, no dilation, the same output stage as
 * NEGEMMConvolutionLayer (calculate_output_stage_metadata, :46-83). On this hardware both functions run the same
 * implicit-GEMM kernel; this class adds the reference's narrower accept / reject rules.
 */
class NEGEMMConv2d : public IFunction
{
public:
    NEGEMMConv2d(const std::shared_ptr<IMemoryManager> &memory_manager = nullptr);
    NEGEMMConv2d(const NEGEMMConv2d &)            = delete;
    NEGEMMConv2d(NEGEMMConv2d &&)                 = default;
    NEGEMMConv2d &operator=(const NEGEMMConv2d &) = delete;
    NEGEMMConv2d &operator=(NEGEMMConv2d &&)      = default;
    ~NEGEMMConv2d();

    void configure(ITensor *input, const ITensor *weights, const ITensor *biases, ITensor *output, const Conv2dInfo &info);
    static Status validate(const ITensorInfo *input, const ITensorInfo *weights, const ITensorInfo *biases,
                           const ITensorInfo *output, const Conv2dInfo &info);

    void run() override;
    void prepare() override;

    const char *kernel_name() const;

private:
    std::unique_ptr<NEGEMMConvolutionLayer> _conv;
};
} // namespace arm_compute
#endif
