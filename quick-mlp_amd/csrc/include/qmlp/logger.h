#pragma once

#include "common.h"

#include <memory>
#include <mutex>
#include <string>

QUICKMLP_NAMESPACE_BEGIN

/** Minimal leveled logger ("qmlp"); messages are printf-formatted. */
class Logger
{
public:
    enum Level { DEBUG = 0, INFO = 1, WARN = 2, ERROR = 3, OFF = 4 };

    explicit Logger(const std::string& name) : name_(name), level_(WARN) {}
    void set_level(Level l) { level_ = l; }
    [[nodiscard]] Level level() const { return level_; }
    [[nodiscard]] bool should_log(Level l) const { return l >= level_ && level_ != OFF; }

    void log(Level l, const char* fmt, va_list ap);
    void debug(const char* fmt, ...) __attribute__((format(printf, 2, 3)));
    void info(const char* fmt, ...) __attribute__((format(printf, 2, 3)));
    void warn(const char* fmt, ...) __attribute__((format(printf, 2, 3)));
    void error(const char* fmt, ...) __attribute__((format(printf, 2, 3)));

private:
    std::string name_;
    Level level_;
    std::mutex mutex_;
};
typedef std::shared_ptr<Logger> logger_t;

QUICKMLP_NAMESPACE_END
