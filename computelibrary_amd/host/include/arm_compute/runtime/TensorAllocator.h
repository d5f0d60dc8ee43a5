// Backing memory of a Tensor. Mirrors arm_compute/runtime/TensorAllocator.h:45-120 of the reference:
// init() -> allocate() / import_memory() -> free(). allocate() gives 64-byte aligned host memory; import_memory()
// adopts caller memory without owning it, and that memory may live on the GPU (hipMalloc / torch device tensors), in which
// case the functions of this build read and write it in place without any host <-> device copy.
#ifndef ACL_MI355_RUNTIME_TENSORALLOCATOR_H
#define ACL_MI355_RUNTIME_TENSORALLOCATOR_H

#include "arm_compute/core/Error.h"
#include "arm_compute/core/TensorInfo.h"

namespace arm_compute
{
class TensorAllocator
{
public:
    TensorAllocator()                                   = default;
    TensorAllocator(const TensorAllocator &)            = delete;
    TensorAllocator &operator=(const TensorAllocator &) = delete;
    TensorAllocator(TensorAllocator &&o) noexcept;
    TensorAllocator &operator=(TensorAllocator &&o) noexcept;
    ~TensorAllocator();

    void init(const TensorInfo &input, size_t alignment = 0);
    TensorInfo       &info() { return _info; }
    const TensorInfo &info() const { return _info; }
    size_t            alignment() const { return _alignment; }
    uint8_t          *data() const { return _ptr; }
    void              allocate();
    void              free();
    bool              is_allocated() const { return _ptr != nullptr; }
    Status            import_memory(void *memory);

private:
    TensorInfo _info{};
    uint8_t   *_ptr{nullptr};
    bool       _owned{false};
    size_t     _alignment{0};
};
} // namespace arm_compute
#endif
