// Shared host-side helpers of the library: per-thread error record and HIP call checking.
#pragma once
#include <hip/hip_runtime.h>
#include <cstdarg>
#include <cstddef>
#include <cstdint>
#include <cstdio>

#include "../../include/bitnet_hip.h"

namespace bitnet {

struct ErrorRecord {
    char msg[512] = {0};
    size_t expected[4] = {0, 0, 0, 0};
    size_t actual[4] = {0, 0, 0, 0};
    int expected_rank = 0;
    int actual_rank = 0;
};

ErrorRecord &error_record();

// Records the message for this thread and returns `code`, so call sites read `return fail(...)`.
int fail(int code, const char *fmt, ...) __attribute__((format(printf, 2, 3)));
int fail_shape(const size_t *expected, int erank, const size_t *actual, int arank, const char *what);

inline hipStream_t as_stream(void *s) { return reinterpret_cast<hipStream_t>(s); }

}  // namespace bitnet

#define BITNET_HIP_TRY(expr)                                                                       \
    do {                                                                                           \
        hipError_t err__ = (expr);                                                                 \
        if (err__ != hipSuccess)                                                                   \
            return ::bitnet::fail(BITNET_HIP_DEVICE_ERROR, "%s failed: %s", #expr,                 \
                                  hipGetErrorString(err__));                                       \
    } while (0)

// After a kernel launch: a launch that could not be queued is reported, never swallowed.
#define BITNET_HIP_CHECK_LAUNCH(name)                                                              \
    do {                                                                                           \
        hipError_t err__ = hipGetLastError();                                                      \
        if (err__ != hipSuccess)                                                                   \
            return ::bitnet::fail(BITNET_HIP_KERNEL_ERROR, "launch of %s failed: %s", name,        \
                                  hipGetErrorString(err__));                                       \
    } while (0)
