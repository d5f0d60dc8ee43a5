// Mirrors arm_compute/runtime/experimental/operators/CpuGEMMLowp.h:40-140 of the reference.
#ifndef ACL_MI355_RUNTIME_EXPERIMENTAL_OPERATORS_CPUGEMMLOWP_H
#define ACL_MI355_RUNTIME_EXPERIMENTAL_OPERATORS_CPUGEMMLOWP_H

#include "arm_compute/core/ITensorInfo.h"
#include "arm_compute/core/ITensorPack.h"
#include "arm_compute/function_info/GEMMInfo.h"
#include "arm_compute/runtime/NEON/INEOperator.h"

#include <memory>

namespace arm_compute
{
namespace experimental
{
namespace op
{
/** Stateless low-precision GEMM: configured on tensor *infos*, run on an ITensorPack
 * (ACL_SRC_0 = a, ACL_SRC_1 = b, ACL_SRC_2 = bias, ACL_DST = output). The same validate() rules, arithmetic and kernels as
 * NEGEMMLowpMatrixMultiplyCore. Tensors whose memory was imported from device pointers are used in place, so a framework
 * that keeps its activations on the GPU pays no copy per run(). The packed weights live in a device workspace owned by the
 * operator: workspace() reports no auxiliary tensors for the caller to provide.
 */
class CpuGEMMLowp : public INEOperator
{
public:
    CpuGEMMLowp();
    CpuGEMMLowp(const CpuGEMMLowp &)            = delete;
    CpuGEMMLowp(CpuGEMMLowp &&)                 = default;
    CpuGEMMLowp &operator=(const CpuGEMMLowp &) = delete;
    CpuGEMMLowp &operator=(CpuGEMMLowp &&)      = default;
    ~CpuGEMMLowp();

    void configure(const ITensorInfo *a, const ITensorInfo *b, const ITensorInfo *c, ITensorInfo *output,
                   const GEMMInfo &gemm_info = GEMMInfo());
    static Status validate(const ITensorInfo *a, const ITensorInfo *b, const ITensorInfo *c, const ITensorInfo *output,
                           const GEMMInfo &gemm_info = GEMMInfo());
    /** New (per-tensor) quantization of a, b and the output without re-packing b
     * (src/runtime/experimental/operators/CpuGEMMLowp.cpp:89-126 of the reference). With negated_offsets the zero points
     * of a and b are negated before use, as convolution and fully connected callers need. */
    void update_quantization_parameters(const QuantizationInfo &a, const QuantizationInfo &b, const QuantizationInfo &c,
                                        const DataType data_type, const bool is_prepared, const bool negated_offsets);

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
