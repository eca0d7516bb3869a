// Shared host-side helpers of libeet_hip.so: error reporting across the C ABI.
#pragma once
#include <cstdarg>
#include <cstdio>
#include <string>

#include "eet_hip.h"

namespace eet {

std::string &last_error_slot();

inline int fail(int code, const char *fmt, ...)
{
    char buf[512];
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(buf, sizeof(buf), fmt, ap);
    va_end(ap);
    last_error_slot() = buf;
    return code;
}

}  // namespace eet

#define EET_REQUIRE(cond, code, ...)              \
    do {                                          \
        if (!(cond))                              \
            return ::eet::fail((code), __VA_ARGS__); \
    } while (0)

#define EET_HIP_CHECK(expr)                                                                   \
    do {                                                                                      \
        hipError_t _e = (expr);                                                               \
        if (_e != hipSuccess)                                                                 \
            return ::eet::fail(EET_ERR_HIP, "%s failed: %s", #expr, hipGetErrorString(_e));   \
    } while (0)
