// Mirrors arm_compute/runtime/IFunction.h:30-66 of the reference.
#ifndef ACL_MI355_RUNTIME_IFUNCTION_H
#define ACL_MI355_RUNTIME_IFUNCTION_H
namespace arm_compute
{
class IFunction
{
public:
    virtual ~IFunction() = default;
    /** Run the function. Synchronous: results are in the output tensor's buffer on return. */
    virtual void run() = 0;
    /** One-off work on constant inputs (weight re-layout, column sums). Idempotent; run() calls it. */
    virtual void prepare() {}
};
} // namespace arm_compute
#endif
