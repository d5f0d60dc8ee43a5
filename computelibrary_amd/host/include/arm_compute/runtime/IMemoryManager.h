// The reference's functions accept an optional host memory manager / weights manager. This build owns its device
// workspace itself; the parameters are kept so call sites compile unchanged and must be null or are ignored.
#ifndef ACL_MI355_RUNTIME_IMEMORYMANAGER_H
#define ACL_MI355_RUNTIME_IMEMORYMANAGER_H
namespace arm_compute
{
class IMemoryManager
{
public:
    virtual ~IMemoryManager() = default;
};
class IWeightsManager
{
public:
    virtual ~IWeightsManager() = default;
};
} // namespace arm_compute
#endif
