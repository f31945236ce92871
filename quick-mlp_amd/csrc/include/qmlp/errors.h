#pragma once

#include "common.h"

#include <cstdarg>
#include <exception>
#include <sstream>
#include <stdexcept>
#include <string>

QUICKMLP_NAMESPACE_BEGIN

/** Raised for problems in the network / encoding / activation specification. */
class configuration_error : public std::exception
{
    std::string message_;

public:
    explicit configuration_error(const std::string& message) : message_(message) {}
    configuration_error(const char* fmt, ...) __attribute__((format(printf, 2, 3)))
    {
        va_list ap;
        va_start(ap, fmt);
        message_ = vformat(fmt, ap);
        va_end(ap);
    }
    const char* what() const noexcept override { return message_.c_str(); }
};

/** Raised when a call through the HIP C ABI fails (device, compiler or launch errors). */
class hip_error : public std::runtime_error
{
public:
    explicit hip_error(const std::string& message) : std::runtime_error(message) {}
};

/** Throws hip_error with the ABI's last error message if 'status' is non-zero. */
void checkHip(int status, const char* file, int line);
#define QMLP_HIP_CALL(expr) ::qmlp::checkHip((expr), __FILE__, __LINE__)

/** what() of an exception including all nested exceptions, one per line. */
std::string describeException(const std::exception& e);

namespace detail {
inline std::string if_empty_then(const std::string& x, const std::string& y) { return x.empty() ? y : x; }
inline std::ostream& _str(std::ostream& ss) { return ss; }
template <typename T>
inline std::ostream& _str(std::ostream& ss, const T& t)
{
    ss << t;
    return ss;
}
template <typename T, typename... Args>
inline std::ostream& _str(std::ostream& ss, const T& t, const Args&... args)
{
    return _str(_str(ss, t), args...);
}
} // namespace detail

template <typename... Args>
inline std::string str(const Args&... args)
{
    std::ostringstream ss;
    detail::_str(ss, args...);
    return ss.str();
}

QUICKMLP_NAMESPACE_END

#define CHECK_ERROR(cond, ...)                                                                     \
    do {                                                                                           \
        if (!(cond)) {                                                                             \
            throw std::runtime_error(QUICKMLP_NAMESPACE::detail::if_empty_then(                    \
                QUICKMLP_NAMESPACE::str(__VA_ARGS__), "Expected " #cond " to be true, but got false.  ")); \
        }                                                                                          \
    } while (false)

#define CHECK_DIM(x, d) CHECK_ERROR((x.ndim() == (d)), #x " must be a tensor with ", d, " dimensions, but has ", x.ndim(), " dimensions")
#define CHECK_SIZE(x, d, s) CHECK_ERROR((static_cast<int64_t>(x.size(d)) == static_cast<int64_t>(s)), #x " must have ", s, " entries at dimension ", d, ", but has ", x.size(d), " entries")
#define CHECK_DTYPE(x, t) CHECK_ERROR(x.precision() == t, #x " must be of type ", QUICKMLP_NAMESPACE::Tensor::NamePerEntry[t], ", but is ", QUICKMLP_NAMESPACE::Tensor::NamePerEntry[x.precision()])
