// Internal helpers shared by the HIP translation units of libag_hip.so.
#pragma once
#include <hip/hip_runtime.h>

#include <cstdarg>
#include <cstdint>
#include <cstdio>

#include "ag_hip.h"

namespace ag {

// Records a message for the calling thread and returns `code`.
ag_status_t fail(ag_status_t code, const char *fmt, ...) __attribute__((format(printf, 2, 3)));

// Turns the status of the last launch / HIP call into an ag_status_t.
ag_status_t check_hip(hipError_t e, const char *what);

inline ag_status_t check_launch(const char *what) { return check_hip(hipGetLastError(), what); }

inline hipStream_t as_stream(ag_stream_t s) { return reinterpret_cast<hipStream_t>(s); }

inline bool aligned16(const void *p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

constexpr int kWave = 64;  // CDNA wavefront width

// Largest grid.x HIP accepts.
constexpr long long kMaxGridX = 2147483647LL;

}  // namespace ag

#define AG_REQUIRE(cond, code, ...)                      \
    do {                                                 \
        if (!(cond)) return ::ag::fail(code, __VA_ARGS__); \
    } while (0)
