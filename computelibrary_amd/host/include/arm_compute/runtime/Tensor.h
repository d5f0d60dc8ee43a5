// Mirrors arm_compute/runtime/Tensor.h of the reference.
#ifndef ACL_MI355_RUNTIME_TENSOR_H
#define ACL_MI355_RUNTIME_TENSOR_H

#include "arm_compute/core/ITensor.h"
#include "arm_compute/runtime/TensorAllocator.h"

namespace arm_compute
{
class Tensor : public ITensor
{
public:
    Tensor()                    = default;
    Tensor(Tensor &&) noexcept  = default;
    Tensor &operator=(Tensor &&) noexcept = default;
    ITensorInfo     *info() const override { return const_cast<TensorInfo *>(&_allocator.info()); }
    ITensorInfo     *info() override { return &_allocator.info(); }
    uint8_t         *buffer() const override { return _allocator.data(); }
    TensorAllocator *allocator() { return &_allocator; }

private:
    mutable TensorAllocator _allocator{};
};
} // namespace arm_compute
#endif
