// Levelled stderr logging.  HCCL_LOG_LEVEL: 0 debug, 1 info, 2 warning, 3 error (default), 4 silent.
#pragma once
#include <cstdio>
#include <cstdlib>

namespace hcclamd {

inline int LogLevel()
{
    static int level = [] {
        const char *e = std::getenv("HCCL_LOG_LEVEL");
        return e ? std::atoi(e) : 3;
    }();
    return level;
}

}  // namespace hcclamd

#define HCCL_LOG_AT(lvl, tag, fmt, ...)                                              \
    do {                                                                             \
        if (::hcclamd::LogLevel() <= (lvl)) {                                        \
            std::fprintf(stderr, "[HCCL][" tag "] " fmt "\n", ##__VA_ARGS__);        \
        }                                                                            \
    } while (0)
#define HCCL_LOG_DEBUG(fmt, ...) HCCL_LOG_AT(0, "DEBUG", fmt, ##__VA_ARGS__)
#define HCCL_LOG_INFO(fmt, ...) HCCL_LOG_AT(1, "INFO", fmt, ##__VA_ARGS__)
#define HCCL_LOG_WARN(fmt, ...) HCCL_LOG_AT(2, "WARNING", fmt, ##__VA_ARGS__)
#define HCCL_LOG_ERROR(fmt, ...) HCCL_LOG_AT(3, "ERROR", fmt, ##__VA_ARGS__)
