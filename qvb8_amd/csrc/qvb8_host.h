// Host-side plumbing of the C ABI: per-thread error text, launch checks, cached device facts, read-once knobs.
#pragma once
#include <hip/hip_runtime.h>
#include <stdarg.h>
#include <stdio.h>
#include <stdlib.h>
#include <string>

namespace qvb8 {
namespace host {

inline std::string& last_error() {
    static thread_local std::string msg;
    return msg;
}

inline int fail(int code, const char* fmt, ...) {
    char buf[512];
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(buf, sizeof buf, fmt, ap);
    va_end(ap);
    last_error() = buf;
    return code;
}

inline int check_launch(const char* who) {
    const hipError_t e = hipGetLastError();
    if (e != hipSuccess) return fail(-3, "%s: launch failed: %s", who, hipGetErrorString(e));
    return 0;
}

// Compute units of the current device (cached per device index).
inline int device_cus() {
    static int cached[64] = {0};
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return 256;
    if (cached[dev] == 0) {
        int n = 0;
        if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0) n = 256;
        cached[dev] = n;
    }
    return cached[dev];
}

// Integer knob from the environment, read on every call (cheap; lets a test change it between calls).
inline int env_int(const char* name, int dflt) {
    const char* e = getenv(name);
    return (e && *e) ? atoi(e) : dflt;
}

}  // namespace host
}  // namespace qvb8
