// Shared helpers of libdeep8_hip.so: error reporting, element types, launch geometry.
#ifndef DEEP8_AMD_COMMON_H
#define DEEP8_AMD_COMMON_H

#include <hip/hip_runtime.h>
#include <hip/hip_fp16.h>

#include <cstdarg>
#include <cstdio>
#include <cstring>

#include "../../include/deep8_hip.h"

namespace d8 {

typedef _Float16 f16;
typedef _Float16 f16x2 __attribute__((ext_vector_type(2)));
typedef _Float16 f16x4 __attribute__((ext_vector_type(4)));
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef float f32x2 __attribute__((ext_vector_type(2)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef float f32x16 __attribute__((ext_vector_type(16)));

// Text of the most recent failure on this thread.
char *error_buffer();
int fail(int code, const char *fmt, ...);

#define D8_HIP(expr)                                                                   \
    do {                                                                               \
        hipError_t e_ = (expr);                                                        \
        if (e_ != hipSuccess) return d8::fail((int)e_, "%s: %s", #expr, hipGetErrorString(e_)); \
    } while (0)

#define D8_REQUIRE(cond, ...)                                  \
    do {                                                       \
        if (!(cond)) return d8::fail(D8_ERR_ARGUMENT, __VA_ARGS__); \
    } while (0)

inline hipStream_t as_stream(void *s) { return (hipStream_t)s; }

inline size_t dtype_bytes(int dtype) { return dtype == D8_FLOAT16 ? 2 : (dtype == D8_FLOAT32 ? 4 : (dtype == D8_FLOAT64 ? 8 : 0)); }

// After a kernel launch: surface launch-configuration errors immediately.
#define D8_LAUNCH_CHECK() D8_HIP(hipGetLastError())

inline int ceil_div(long a, long b) { return (int)((a + b - 1) / b); }

// Number of compute units of the current device (cached).
int cu_count();

// Looks up, once per device, where the current device keeps its copy of the static scratch array
// (static_scratch.hip).  Called by d8_device_init and, failing that, by the first call that needs it.
int static_scratch_setup();

}  // namespace d8

#endif
