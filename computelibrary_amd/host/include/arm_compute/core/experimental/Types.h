// Mirrors arm_compute/core/experimental/Types.h:41-126 of the reference: tensor slots of an ITensorPack and the
// auxiliary-memory descriptors an operator reports through workspace().
#ifndef ACL_MI355_CORE_EXPERIMENTAL_TYPES_H
#define ACL_MI355_CORE_EXPERIMENTAL_TYPES_H

#include <algorithm>
#include <cstddef>
#include <vector>

namespace arm_compute
{
enum TensorType : int32_t
{
    ACL_UNKNOWN = -1,
    ACL_SRC_DST = 0,
    ACL_SRC     = 0,
    ACL_SRC_0   = 0,
    ACL_SRC_1   = 1,
    ACL_SRC_2   = 2,
    ACL_SRC_3   = 3,
    ACL_SRC_4   = 4,
    ACL_SRC_5   = 5,
    ACL_SRC_6   = 6,
    ACL_SRC_END = 6,
    ACL_DST     = 30,
    ACL_DST_0   = 30,
    ACL_DST_1   = 31,
    ACL_DST_2   = 32,
    ACL_DST_END = 32,
    ACL_INT     = 50,
    ACL_INT_0   = 50,
    ACL_INT_1   = 51,
    ACL_INT_2   = 52,
    ACL_INT_3   = 53,
    ACL_INT_4   = 54,
    ACL_SRC_VEC = 256,
    ACL_DST_VEC = 512,
    ACL_INT_VEC = 1024,
    ACL_BIAS        = ACL_SRC_2,
    ACL_VEC_ROW_SUM = ACL_SRC_3,
    ACL_VEC_COL_SUM = ACL_SRC_4,
    ACL_SHIFTS      = ACL_SRC_5,
    ACL_MULTIPLIERS = ACL_SRC_6
};

namespace experimental
{
enum class MemoryLifetime
{
    Temporary  = 0,
    Persistent = 1,
    Prepare    = 2
};

struct MemoryInfo
{
    MemoryInfo() = default;
    MemoryInfo(int slot, size_t size, size_t alignment = 0) noexcept : slot(slot), size(size), alignment(alignment) {}
    MemoryInfo(int slot, MemoryLifetime lifetime, size_t size, size_t alignment = 0) noexcept
        : slot(slot), lifetime(lifetime), size(size), alignment(alignment)
    {
    }
    bool merge(int s, size_t new_size, size_t new_alignment = 0) noexcept
    {
        if (s != slot)
            return false;
        size      = std::max(size, new_size);
        alignment = std::max(alignment, new_alignment);
        return true;
    }
    int            slot{ACL_UNKNOWN};
    MemoryLifetime lifetime{MemoryLifetime::Temporary};
    size_t         size{0};
    size_t         alignment{64};
};

using MemoryRequirements = std::vector<MemoryInfo>;
} // namespace experimental
} // namespace arm_compute
#endif
