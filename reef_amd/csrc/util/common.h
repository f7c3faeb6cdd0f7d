// Status codes, logging and small helpers shared by the host side.
// Mirrors the error convention of the reference (src/reef/util/common.h:46-63):
// every call returns a reef::Status, failures are logged with file:line and
// propagated, nothing throws.  glog is not required: messages go to stderr
// when REEF_LOG_LEVEL >= 1 (errors) or >= 2 (info).
#pragma once
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <string>

namespace reef {

enum Status { Succ = 0, Fail = 1, NotFound = 2, OutOfRange = 3, Full = 4 };

int log_level();  // 0 silent, 1 errors (default), 2 info

template <typename T>
T align_up(T value, T alignment) {
    T r = value % alignment;
    return r == 0 ? value : value - r + alignment;
}
template <typename T>
T align_down(T value, T alignment) {
    return value - value % alignment;
}
template <typename T>
T ceil_div(T a, T b) {
    return (a + b - 1) / b;
}

}  // namespace reef

#define REEF_LOG_ERROR(...)                                            \
    do {                                                               \
        if (::reef::log_level() >= 1) {                                \
            std::fprintf(stderr, "[reef E %s:%d] ", __FILE__, __LINE__); \
            std::fprintf(stderr, __VA_ARGS__);                         \
            std::fprintf(stderr, "\n");                                \
        }                                                              \
    } while (0)
#define REEF_LOG_INFO(...)                                   \
    do {                                                     \
        if (::reef::log_level() >= 2) {                      \
            std::fprintf(stderr, "[reef I] ");               \
            std::fprintf(stderr, __VA_ARGS__);               \
            std::fprintf(stderr, "\n");                      \
        }                                                    \
    } while (0)

// Propagate a non-Succ Status (reference: RETURN_STATUS, common.h:25-32).
#define RETURN_STATUS(cmd)                           \
    do {                                             \
        ::reef::Status _s = (cmd);                   \
        if (_s != ::reef::Status::Succ) {            \
            REEF_LOG_ERROR("%s -> status %d", #cmd, (int)_s); \
            return _s;                               \
        }                                            \
    } while (0)

// HAL call failed -> Status::Fail (reference: GPU_RETURN_STATUS, hip_impl.h:25-32).
#define GPU_RETURN_STATUS(cmd)                                             \
    do {                                                                   \
        if ((cmd) != 0) {                                                  \
            REEF_LOG_ERROR("gpu error: %s (%s)", reef_hal_last_error(), #cmd); \
            return ::reef::Status::Fail;                                   \
        }                                                                  \
    } while (0)
