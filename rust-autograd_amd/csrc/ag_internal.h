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

constexpr int kXcds = 8;

// Compute units of the current device (queried once per process; 256 when the query fails).
int device_cus();

#if defined(__HIPCC__)
// Hardware hands consecutive workgroup ids to the XCDs round-robin; give XCD x the x-th
// contiguous slice of the logical block range instead, so that blocks which touch neighbouring
// memory share an L2 (partial cache lines at the seams of their outputs merge there).
__device__ inline unsigned xcd_remap(unsigned id, unsigned total)
{
    const unsigned per = total / kXcds, rem = total % kXcds;
    const unsigned xcd = id % kXcds, pos = id / kXcds;
    return xcd * per + (xcd < rem ? xcd : rem) + pos;
}
#endif

#if defined(__HIPCC__)
// Streaming (non-temporal) accesses for data that is touched once: they do not displace the
// operands other kernels keep in L2 and measured ~10 % faster than plain accesses on MI355X.
typedef float f32x4_t __attribute__((ext_vector_type(4)));
__device__ inline float4 ld_stream(const float4 *p)
{
    const f32x4_t v = __builtin_nontemporal_load(reinterpret_cast<const f32x4_t *>(p));
    return make_float4(v.x, v.y, v.z, v.w);
}
__device__ inline void st_stream(float4 *p, const float4 &v)
{
    const f32x4_t t = {v.x, v.y, v.z, v.w};
    __builtin_nontemporal_store(t, reinterpret_cast<f32x4_t *>(p));
}
__device__ inline float ld_stream(const float *p) { return __builtin_nontemporal_load(p); }
__device__ inline int ld_stream(const int *p) { return __builtin_nontemporal_load(p); }
__device__ inline void st_stream(float *p, float v) { __builtin_nontemporal_store(v, p); }
__device__ inline void st_stream(int *p, int v) { __builtin_nontemporal_store(v, p); }
#endif

// Validates reduction axes (range, rank <= 8) and writes them to `sorted` in ascending order.
ag_status_t check_axes(const char *who, const int *shape, int rank, const int *axes, int n_axes, int *sorted);

}  // namespace ag

#define AG_REQUIRE(cond, code, ...)                      \
    do {                                                 \
        if (!(cond)) return ::ag::fail(code, __VA_ARGS__); \
    } while (0)
