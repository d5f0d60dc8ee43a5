// Tensor interface: metadata + a byte buffer. Mirrors arm_compute/core/ITensor.h:38-103 of the reference.
// In this build buffer() may return host memory (results are copied to and from the GPU inside run()) or device memory
// imported with TensorAllocator::import_memory() (used in place).
#ifndef ACL_MI355_CORE_ITENSOR_H
#define ACL_MI355_CORE_ITENSOR_H

#include "arm_compute/core/ITensorInfo.h"

namespace arm_compute
{
class ITensor
{
public:
    virtual ~ITensor()                       = default;
    virtual ITensorInfo *info() const        = 0;
    virtual ITensorInfo *info()              = 0;
    virtual uint8_t     *buffer() const      = 0;
    uint8_t *ptr_to_element(const Coordinates &id) const
    {
        return buffer() + info()->offset_element_in_bytes(id);
    }
    bool is_used() const { return _is_used; }
    void mark_as_unused() const { _is_used = false; }
    void mark_as_used() const { _is_used = true; }

private:
    mutable bool _is_used = {true};
};
} // namespace arm_compute
#endif
