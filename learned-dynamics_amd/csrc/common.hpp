// Shared host-side helpers for the C-ABI entry points (gfx950 only).
#pragma once
#include <hip/hip_runtime.h>
#include <cstdarg>
#include <cstdio>
#include <cstdint>
#include "managan_hip.h"

namespace mg {

constexpr int kWave = 64;  // CDNA4 wavefront width

char* last_error_buffer();  // thread-local, 512 bytes

inline int fail(int status, const char* fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(last_error_buffer(), 512, fmt, ap);
    va_end(ap);
    return status;
}

inline int check_launch(const char* what) {
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return fail(MG_ERR_HIP, "%s: %s", what, hipGetErrorString(e));
    return MG_OK;
}

inline long ceil_div(long a, long b) { return (a + b - 1) / b; }

inline bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

}  // namespace mg

#define MG_REQUIRE(cond, ...)                                              \
    do {                                                                   \
        if (!(cond)) return mg::fail(MG_ERR_INVALID_ARGUMENT, __VA_ARGS__); \
    } while (0)

#define MG_HIP(call)                                                                          \
    do {                                                                                      \
        hipError_t e_ = (call);                                                               \
        if (e_ != hipSuccess) return mg::fail(MG_ERR_HIP, "%s: %s", #call, hipGetErrorString(e_)); \
    } while (0)
