#include <qmlp/common.h>
#include <qmlp/errors.h>
#include <qmlp/logger.h>
#include <qmlp/tmp_memory.h>

#include "qmlp_hip.h"

#include <cstdarg>
#include <cstdio>
#include <vector>

QUICKMLP_NAMESPACE_BEGIN

std::string vformat(const char* fmt, va_list ap)
{
    va_list ap2;
    va_copy(ap2, ap);
    int n = std::vsnprintf(nullptr, 0, fmt, ap2);
    va_end(ap2);
    if (n < 0) return fmt;
    std::vector<char> buf(static_cast<size_t>(n) + 1);
    std::vsnprintf(buf.data(), buf.size(), fmt, ap);
    return std::string(buf.data(), static_cast<size_t>(n));
}

std::string format(const char* fmt, ...)
{
    va_list ap;
    va_start(ap, fmt);
    std::string s = vformat(fmt, ap);
    va_end(ap);
    return s;
}

void checkHip(int status, const char* file, int line)
{
    if (status == 0) return;
    throw hip_error(format("%s (%s:%d)", qmlp_hip_last_error(), file, line));
}

static void describeImpl(const std::exception& e, std::string& out, int level)
{
    if (level > 0) out += "\n";
    out.append(static_cast<size_t>(2 * level), ' ');
    out += e.what();
    try {
        std::rethrow_if_nested(e);
    } catch (const std::exception& nested) {
        describeImpl(nested, out, level + 1);
    } catch (...) {
    }
}

std::string describeException(const std::exception& e)
{
    std::string out;
    describeImpl(e, out, 0);
    return out;
}

void Logger::log(Level l, const char* fmt, va_list ap)
{
    if (!should_log(l)) return;
    static const char* NAMES[] = {"debug", "info", "warning", "error"};
    std::string msg = vformat(fmt, ap);
    std::lock_guard<std::mutex> lock(mutex_);
    std::fprintf(l >= WARN ? stderr : stdout, "[%s] [%s] %s\n", name_.c_str(), NAMES[l], msg.c_str());
    std::fflush(l >= WARN ? stderr : stdout);
}

#define QMLP_LOG_IMPL(fn, lvl)            \
    void Logger::fn(const char* fmt, ...) \
    {                                     \
        if (!should_log(lvl)) return;     \
        va_list ap;                       \
        va_start(ap, fmt);                \
        log(lvl, fmt, ap);                \
        va_end(ap);                       \
    }
QMLP_LOG_IMPL(debug, DEBUG)
QMLP_LOG_IMPL(info, INFO)
QMLP_LOG_IMPL(warn, WARN)
QMLP_LOG_IMPL(error, ERROR)

TmpMemory::TmpMemory(size_t numBytes) : memory_(nullptr)
{
    if (numBytes > 0) QMLP_HIP_CALL(qmlp_hip_malloc(&memory_, numBytes));
}

TmpMemory::~TmpMemory() { qmlp_hip_free(memory_); }

QUICKMLP_NAMESPACE_END
