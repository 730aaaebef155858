// Shared host-side helpers of libdistdl_hip: error reporting, launch checks,
// exact 32-bit division by invariant integers.
#pragma once

#include <hip/hip_runtime.h>
#include <stdarg.h>
#include <stdint.h>
#include <stdio.h>

#include "../../include/distdl_hip.h"

namespace ddl {

// Thread-local message behind ddl_last_error().
char* error_buffer();
int fail(int code, const char* fmt, ...);

// Checks the launch that has just been enqueued; returns 0 or the hipError_t.
int check_launch(const char* what);

inline bool aligned_to(const void* p, uint64_t a) {
    return (reinterpret_cast<uintptr_t>(p) & (a - 1)) == 0;
}

// Division of a 31-bit unsigned dividend by a fixed divisor as one multiply-high
// and one shift.  q = n / d for every 0 <= n < 2^31 and 1 <= d < 2^31.
struct FastDiv {
    uint32_t mul;
    uint32_t shr;
    uint32_t div;
    uint32_t pad;
};

inline FastDiv make_fastdiv(uint32_t d) {
    FastDiv f;
    f.div = d;
    f.pad = 0;
    if (d <= 1) {
        f.mul = 0;
        f.shr = 0;
        return f;
    }
    uint32_t lg = 0;  // ceil(log2(d))
    while ((1ull << lg) < d) ++lg;
    const uint32_t p = 31 + lg;
    f.mul = static_cast<uint32_t>(((1ull << p) + d - 1) / d);
    f.shr = p - 32;
    return f;
}

__host__ __device__ inline uint32_t fd_div(uint32_t n, const FastDiv& f) {
#if defined(__HIP_DEVICE_COMPILE__)
    return f.div == 1 ? n : (__umulhi(n, f.mul) >> f.shr);
#else
    return f.div == 1 ? n : static_cast<uint32_t>((static_cast<uint64_t>(n) * f.mul) >> 32) >> f.shr;
#endif
}

}  // namespace ddl
