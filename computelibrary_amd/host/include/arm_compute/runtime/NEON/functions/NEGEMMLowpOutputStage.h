// Mirrors arm_compute/runtime/NEON/functions/NEGEMMLowpOutputStage.h:52-107 of the reference.
#ifndef ACL_MI355_RUNTIME_NEGEMMLOWPOUTPUTSTAGE_H
#define ACL_MI355_RUNTIME_NEGEMMLOWPOUTPUTSTAGE_H

#include "arm_compute/core/ITensor.h"
#include "arm_compute/function_info/GEMMInfo.h"
#include "arm_compute/runtime/IFunction.h"

#include <memory>

namespace arm_compute
{
/** Stand-alone output stage: S32 (+ S32 bias) -> QASYMM8 / QASYMM8_SIGNED with QUANTIZE_DOWN_FIXEDPOINT. */
class NEGEMMLowpOutputStage : public IFunction
{
public:
    NEGEMMLowpOutputStage();
    NEGEMMLowpOutputStage(const NEGEMMLowpOutputStage &)            = delete;
    NEGEMMLowpOutputStage(NEGEMMLowpOutputStage &&)                 = default;
    NEGEMMLowpOutputStage &operator=(const NEGEMMLowpOutputStage &) = delete;
    NEGEMMLowpOutputStage &operator=(NEGEMMLowpOutputStage &&)      = default;
    ~NEGEMMLowpOutputStage();

    void configure(const ITensor *input, const ITensor *bias, ITensor *output, const GEMMLowpOutputStageInfo &info);
    static Status validate(const ITensorInfo *input, const ITensorInfo *bias, const ITensorInfo *output,
                           const GEMMLowpOutputStageInfo &info);
    void run() override;

private:
    struct Impl;
    std::unique_ptr<Impl> _impl;
};
} // namespace arm_compute
#endif
