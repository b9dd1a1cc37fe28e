// Host-side helpers shared by the entry points: thread-local error text and launch checking.
#pragma once

#include <hip/hip_runtime.h>

#include <cstdio>
#include <cstring>

#include "../../include/aimet_amd.h"

namespace ahq {

inline char* error_buffer() {
    static thread_local char buf[512] = {0};
    return buf;
}

inline void set_error(const char* msg) {
    std::snprintf(error_buffer(), 512, "%s", msg ? msg : "unknown error");
}

// Reports an error left by the launches just enqueued (configuration errors surface here; faults do not).
inline int check_launch(const char* where) {
    const hipError_t e = hipGetLastError();
    if (e == hipSuccess) return AHQ_OK;
    std::snprintf(error_buffer(), 512, "%s: %s", where, hipGetErrorString(e));
    return AHQ_ERR_LAUNCH;
}

}  // namespace ahq
