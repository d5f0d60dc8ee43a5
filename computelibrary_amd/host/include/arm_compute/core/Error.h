// Status / error model of the arm_compute surface kept by this build.
// Mirrors arm_compute/core/Error.h:40-140,310-482 of the reference: validate() returns a Status and never throws;
// configure()/run() raise std::runtime_error through ARM_COMPUTE_ERROR_THROW_ON.
#ifndef ACL_MI355_CORE_ERROR_H
#define ACL_MI355_CORE_ERROR_H

#include <stdexcept>
#include <string>

namespace arm_compute
{
enum class ErrorCode
{
    OK,
    RUNTIME_ERROR,
    UNSUPPORTED_EXTENSION_USE
};

class Status
{
public:
    Status() : _code(ErrorCode::OK), _error_description(" ") {}
    Status(ErrorCode error_status, std::string error_description = " ")
        : _code(error_status), _error_description(std::move(error_description))
    {
    }
    explicit  operator bool() const noexcept { return _code == ErrorCode::OK; }
    ErrorCode error_code() const { return _code; }
    std::string error_description() const { return _error_description; }
    void throw_if_error() const
    {
        if (!bool(*this))
            throw std::runtime_error(_error_description);
    }

private:
    ErrorCode   _code;
    std::string _error_description;
};

inline Status create_error(ErrorCode code, const std::string &msg, const char *function, const char *file, int line)
{
    return Status(code, std::string("in ") + function + " " + file + ":" + std::to_string(line) + ": " + msg);
}
} // namespace arm_compute

#define ARM_COMPUTE_UNUSED(...) ((void)sizeof((__VA_ARGS__, 0)))
#define ARM_COMPUTE_CREATE_ERROR(code, msg) arm_compute::create_error(code, msg, __func__, __FILE__, __LINE__)
#define ARM_COMPUTE_RETURN_ERROR_ON_MSG(cond, msg)                                           \
    do                                                                                       \
    {                                                                                        \
        if (cond)                                                                            \
            return ARM_COMPUTE_CREATE_ERROR(arm_compute::ErrorCode::RUNTIME_ERROR, msg);     \
    } while (false)
#define ARM_COMPUTE_RETURN_ERROR_ON(cond) ARM_COMPUTE_RETURN_ERROR_ON_MSG(cond, #cond)
#define ARM_COMPUTE_RETURN_ERROR_MSG(msg) return ARM_COMPUTE_CREATE_ERROR(arm_compute::ErrorCode::RUNTIME_ERROR, msg)
#define ARM_COMPUTE_RETURN_ON_ERROR(status)   \
    do                                        \
    {                                         \
        const auto s_ = (status);             \
        if (!bool(s_))                        \
            return s_;                        \
    } while (false)
#define ARM_COMPUTE_RETURN_ERROR_ON_NULLPTR(...)                                                   \
    do                                                                                             \
    {                                                                                              \
        const void *ptrs_[] = {__VA_ARGS__};                                                       \
        for (const void *p_ : ptrs_)                                                               \
            if (p_ == nullptr)                                                                     \
                return ARM_COMPUTE_CREATE_ERROR(arm_compute::ErrorCode::RUNTIME_ERROR, "nullptr object: " #__VA_ARGS__); \
    } while (false)
#define ARM_COMPUTE_ERROR_THROW_ON(status) (status).throw_if_error()
#define ARM_COMPUTE_ERROR(msg) \
    throw std::runtime_error(ARM_COMPUTE_CREATE_ERROR(arm_compute::ErrorCode::RUNTIME_ERROR, msg).error_description())
#define ARM_COMPUTE_ERROR_ON_MSG(cond, msg) \
    do                                      \
    {                                       \
        if (cond)                           \
            ARM_COMPUTE_ERROR(msg);         \
    } while (false)
#define ARM_COMPUTE_ERROR_ON(cond) ARM_COMPUTE_ERROR_ON_MSG(cond, #cond)
#define ARM_COMPUTE_ERROR_ON_NULLPTR(...)                       \
    do                                                          \
    {                                                           \
        const void *ptrs_[] = {__VA_ARGS__};                    \
        for (const void *p_ : ptrs_)                            \
            if (p_ == nullptr)                                  \
                ARM_COMPUTE_ERROR("nullptr object: " #__VA_ARGS__); \
    } while (false)

#endif
