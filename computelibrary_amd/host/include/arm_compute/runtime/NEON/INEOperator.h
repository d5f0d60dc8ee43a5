// Mirrors arm_compute/runtime/NEON/INEOperator.h:48-83 of the reference: the stateless operator interface.
#ifndef ACL_MI355_RUNTIME_INEOPERATOR_H
#define ACL_MI355_RUNTIME_INEOPERATOR_H

#include "arm_compute/core/ITensorPack.h"
#include "arm_compute/core/experimental/Types.h"

namespace arm_compute
{
namespace experimental
{
class INEOperator
{
public:
    virtual ~INEOperator()                              = default;
    virtual void               run(ITensorPack &tensors) = 0;
    virtual void               prepare(ITensorPack &constants) { (void)constants; }
    virtual MemoryRequirements workspace() const { return {}; }
};
} // namespace experimental
} // namespace arm_compute
#endif
