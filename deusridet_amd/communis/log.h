// log.h -- LOG_{DEBUG,INFO,WARN,ERROR}(module, fmt, ...) with the shape of the
// reference's macros (src/communis/log.h:59-62): stderr, timestamp, severity,
// module.  The minimum level starts at WARN unless DEUSRIDET_LOG=debug|info is
// set, so that tests and benchmarks stay quiet.
#pragma once

#include <cstdarg>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <ctime>

namespace deusridet {
namespace log {

enum class Level { DEBUG, INFO, WARN, ERROR };

inline Level initial_level()
{
    const char *e = std::getenv("DEUSRIDET_LOG");
    if (!e) return Level::WARN;
    if (!std::strcmp(e, "debug")) return Level::DEBUG;
    if (!std::strcmp(e, "info")) return Level::INFO;
    if (!std::strcmp(e, "error")) return Level::ERROR;
    return Level::WARN;
}

inline Level &min_level()
{
    static Level l = initial_level();
    return l;
}
inline void set_level(Level l) { min_level() = l; }

inline void log(Level level, const char *module, const char *fmt, ...)
{
    if (level < min_level()) return;
    static const char *names[] = {"DEBUG", "INFO", "WARN", "ERROR"};
    struct timespec ts;
    clock_gettime(CLOCK_REALTIME, &ts);
    struct tm tm;
    localtime_r(&ts.tv_sec, &tm);
    std::fprintf(stderr, "[%02d:%02d:%02d.%03ld] [%5s] [%s] ", tm.tm_hour, tm.tm_min, tm.tm_sec,
                 ts.tv_nsec / 1000000, names[(int)level], module);
    va_list ap;
    va_start(ap, fmt);
    std::vfprintf(stderr, fmt, ap);
    va_end(ap);
    std::fputc('\n', stderr);
}

} // namespace log
} // namespace deusridet

#define LOG_DEBUG(mod, ...) ::deusridet::log::log(::deusridet::log::Level::DEBUG, mod, __VA_ARGS__)
#define LOG_INFO(mod, ...)  ::deusridet::log::log(::deusridet::log::Level::INFO, mod, __VA_ARGS__)
#define LOG_WARN(mod, ...)  ::deusridet::log::log(::deusridet::log::Level::WARN, mod, __VA_ARGS__)
#define LOG_ERROR(mod, ...) ::deusridet::log::log(::deusridet::log::Level::ERROR, mod, __VA_ARGS__)
