// Shared host-side helpers of libmdx: error reporting and argument checks.
#pragma once
#include <hip/hip_runtime.h>
#include <cstdarg>
#include <cstdint>
#include <cstdio>
#include "../../include/mdx.h"

namespace mdx {

// Thread-local message behind mdx_last_error().
char* error_buffer();

inline int fail(int code, const char* fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(error_buffer(), 512, fmt, ap);
    va_end(ap);
    return code;
}

// Checks the launch that was just enqueued; never synchronises.
inline int check_launch(const char* what) {
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return fail(MDX_ELAUNCH, "%s: %s", what, hipGetErrorString(e));
    return MDX_OK;
}

inline bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

constexpr int kWave = 64;          // gfx950 wavefront

}  // namespace mdx

// 16-byte vector used for every wide load/store (a native vector type, so the
// nontemporal builtins accept it).
typedef __attribute__((ext_vector_type(4))) uint32_t u32x4;

namespace mdx {

}  // namespace mdx

#define MDX_REQUIRE(cond, code, ...) \
    do { if (!(cond)) return ::mdx::fail(code, __VA_ARGS__); } while (0)
