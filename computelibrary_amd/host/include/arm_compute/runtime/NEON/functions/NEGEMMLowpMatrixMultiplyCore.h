// Mirrors arm_compute/runtime/NEON/functions/NEGEMMLowpMatrixMultiplyCore.h:50-133 of the reference: same class name,
// same member signatures, same semantics. The work runs on an MI355X through the C ABI of include/mi355_gemmlowp.h.
#ifndef ACL_MI355_RUNTIME_NEGEMMLOWPMATRIXMULTIPLYCORE_H
#define ACL_MI355_RUNTIME_NEGEMMLOWPMATRIXMULTIPLYCORE_H

#include "arm_compute/core/ITensor.h"
#include "arm_compute/function_info/GEMMInfo.h"
#include "arm_compute/runtime/IFunction.h"
#include "arm_compute/runtime/IMemoryManager.h"

#include <memory>

namespace arm_compute
{
/** Low-precision matrix multiply: dst = sum_k (a + a_offset)(b + b_offset), optionally followed by the fused output
 * stage carried by GEMMInfo::gemmlowp_output_stage() (QUANTIZE_DOWN_FIXEDPOINT -> QASYMM8 / QASYMM8_SIGNED), or
 * dequantised to F32 when the destination is F32.
 *
 * Valid configurations (a, b, c, dst): a QASYMM8 / QASYMM8_SIGNED; b QASYMM8 / QASYMM8_SIGNED / QSYMM8 /
 * QSYMM8_PER_CHANNEL; c S32 bias (with an output stage) or F32 bias (F32 destination) or nullptr;
 * dst S32 / QASYMM8 / QASYMM8_SIGNED / F32.
 *
 * The offsets taken from QuantizationInfo are ADDED to the matrix values, exactly as in the reference
 * (callers holding true zero points negate them first).
 */
class NEGEMMLowpMatrixMultiplyCore : public IFunction
{
public:
    NEGEMMLowpMatrixMultiplyCore(std::shared_ptr<IMemoryManager> memory_manager  = nullptr,
                                 IWeightsManager                *weights_manager = nullptr);
    NEGEMMLowpMatrixMultiplyCore(const NEGEMMLowpMatrixMultiplyCore &)            = delete;
    NEGEMMLowpMatrixMultiplyCore(NEGEMMLowpMatrixMultiplyCore &&)                 = default;
    NEGEMMLowpMatrixMultiplyCore &operator=(const NEGEMMLowpMatrixMultiplyCore &) = delete;
    NEGEMMLowpMatrixMultiplyCore &operator=(NEGEMMLowpMatrixMultiplyCore &&)      = default;
    ~NEGEMMLowpMatrixMultiplyCore();

    void configure(const ITensor *a, const ITensor *b, const ITensor *c, ITensor *output,
                   const GEMMInfo &gemm_info = GEMMInfo());
    static Status validate(const ITensorInfo *a, const ITensorInfo *b, const ITensorInfo *c, const ITensorInfo *output,
                           const GEMMInfo &gemm_info = GEMMInfo());
    /** Re-reads the quantization info of a, b and output and rebuilds the (per-tensor) output stage without re-packing b. */
    void update_quantization_parameters();

    void run() override;
    void prepare() override;

    /** Name of the device kernel the last run() dispatched to (not part of the reference API; for logs and tests). */
    const char *kernel_name() const;

private:
    struct Impl;
    std::unique_ptr<Impl> _impl;
};
} // namespace arm_compute
#endif
