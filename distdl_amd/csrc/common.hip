// Error state and identification of libdistdl_hip.
#include "ddl_common.h"

namespace ddl {

char* error_buffer() {
    static thread_local char buf[512] = {0};
    return buf;
}

int fail(int code, const char* fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(error_buffer(), 512, fmt, ap);
    va_end(ap);
    return code;
}

int check_launch(const char* what) {
    const hipError_t e = hipGetLastError();
    if (e == hipSuccess) return 0;
    return fail(static_cast<int>(e), "%s: %s", what, hipGetErrorString(e));
}

}  // namespace ddl

extern "C" {

const char* ddl_version(void) { return "distdl_hip 0.1.0 gfx950"; }

const char* ddl_last_error(void) { return ddl::error_buffer(); }

}  // extern "C"
