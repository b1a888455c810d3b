// Shared helpers of the C-ABI library: per-thread error text and argument checks.
#pragma once
#include <cstdarg>
#include <cstdio>

#include "../../include/raptor_t_hip.h"

namespace rt {

char* error_buffer();                       // per-thread, 512 bytes
int fail(int code, const char* fmt, ...);   // formats into the buffer, returns code

}  // namespace rt

#define RT_REQUIRE(cond, code, ...) \
  do {                              \
    if (!(cond)) return rt::fail((code), __VA_ARGS__); \
  } while (0)
